"""Writes tests/golden/ref_fixtures_avg_uv.npz: inputs and outputs of the reference's own CPU
extensions (compiled by `make -C oracle ref` from the reference sources) for mapped average
pooling / unpooling (unweighted and weighted, all three interpolations, float32 and float64;
the reference's tests hold one bilinear float64 vector) and for UV resampling in both
directions and for voting resample (the reference's tests hold none for either).

Run in the build container only (it needs the compiled reference):
    python tests/golden/make_ref_fixtures_avg_uv.py
The committed .npz is plain data: seeded inputs and the reference's outputs.
"""
import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import ref  # noqa: E402

R = ref.load()
IT = R.InterpolationType
OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "ref_fixtures_avg_uv.npz")

B, C, H, W, OH, OW, K, P = 2, 3, 6, 7, 4, 5, 3, 2
NT, TH, TW = 5, 4, 6          # textures of the UV pair; the image side is H x W


def coords(gen, shape, dtype, width, height):
    """(x, y) samples covering a width x height plane plus an out-of-bounds margin, with a
    sprinkling of exact integers and exact .5 ties."""
    xy = torch.rand(*shape, 2, generator=gen, dtype=torch.float64)
    xy = xy * torch.tensor([width + 3.0, height + 3.0], dtype=torch.float64) - 1.5
    sel = torch.rand(*shape, generator=gen) < 0.25
    xy[sel] = torch.round(xy[sel])
    sel = torch.rand(*shape, generator=gen) < 0.1
    xy[sel] = torch.floor(xy[sel]) + 0.5
    return xy.to(dtype).contiguous()


def main():
    data = {}
    for dname, dtype in (("f64", torch.float64), ("f32", torch.float32)):
        gen = torch.Generator().manual_seed(77100 + (dtype == torch.float32))
        x = torch.randn(B, C, H, W, generator=gen, dtype=torch.float64).to(dtype)
        g = torch.randn(B, C, OH, OW, generator=gen, dtype=torch.float64).to(dtype)
        m_u = coords(gen, (OH, OW, K), dtype, W, H)
        m_w = coords(gen, (OH, OW, K, P), dtype, W, H)
        iw = torch.rand(OH, OW, K, P, generator=gen, dtype=torch.float64).to(dtype)
        tex = torch.randn(B, C, NT, TH, TW, generator=gen, dtype=torch.float64).to(dtype)
        quad = torch.randint(0, NT, (H, W), generator=gen, dtype=torch.int64)
        uv = coords(gen, (H, W), dtype, TW, TH)
        for k_, v_ in dict(x=x, g=g, m_u=m_u, m_w=m_w, iw=iw, tex=tex, quad=quad, uv=uv).items():
            data["%s/in/%s" % (dname, k_)] = v_.numpy()
        for interp in (0, 1, 2):
            it = IT(interp)
            pre = "%s/i%d/" % (dname, interp)
            A = R._mapped_avg_pooling
            data[pre + "avg_pool"] = A.mapped_avg_pool(x, m_u, K, it).numpy()
            data[pre + "avg_unpool"] = A.mapped_avg_unpool(g, m_u, H, W, K, it).numpy()
            A = R._weighted_mapped_avg_pooling
            data[pre + "wavg_pool"] = A.weighted_mapped_avg_pool(x, m_w, iw, K, it).numpy()
            data[pre + "wavg_unpool"] = A.weighted_mapped_avg_unpool(g, m_w, iw, H, W, K,
                                                                     it).numpy()
            U = R._uv_resample
            data[pre + "from_uv"] = U.resample_from_uv_maps(tex, quad, uv, it).numpy()
            data[pre + "to_uv"] = U.resample_to_uv_maps(x, quad, uv, NT, TH, TW, it).numpy()
    # voting resample: integer labels through an integer map, targets partly outside the output,
    # several sources per target so that ties and clear majorities both occur
    gen = torch.Generator().manual_seed(77300)
    NC, VH, VW = 5, 9, 11
    labels = torch.randint(0, NC, (B, C, VH, VW), generator=gen, dtype=torch.int64)
    vmap = torch.stack([torch.randint(-1, W + 1, (VH, VW), generator=gen, dtype=torch.int64),
                        torch.randint(-1, H + 1, (VH, VW), generator=gen, dtype=torch.int64)], -1)
    data["vote/in/labels"], data["vote/in/map"] = labels.numpy(), vmap.contiguous().numpy()
    data["vote/out"] = R._voting_resample.voting_resample_to_map(
        labels, vmap.contiguous(), H, W, NC).numpy()
    np.savez_compressed(OUT, **data)
    print("wrote", OUT, len(data), "arrays", os.path.getsize(OUT), "bytes")


if __name__ == "__main__":
    main()
