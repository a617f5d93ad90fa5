"""Writes tests/golden/ref_fixtures.npz: inputs and outputs of the reference's own
CPU extensions (compiled by `make -C oracle ref` from the reference sources) for
the variants none of the reference's tests cover: weighted convolution /
transposed convolution / pooling, NEAREST and BISPHERICAL inside convolution
and pooling, float32, the pooling index tensor (including the host branch's
initial-value behaviour on all-negative windows), unpooling and the forward
values of the scatter direction.

Run in the build container only (it needs the compiled reference):
    python tests/golden/make_ref_fixtures.py
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
OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "ref_fixtures.npz")

B, CIN, COUT, H, W, OH, OW, K, P = 2, 3, 4, 6, 7, 4, 5, 3, 2
TOH, TOW = 7, 8  # transposed-convolution output size


def coords(gen, shape, dtype):
    """Real-valued (x, y) samples covering the image plus an out-of-bounds margin,
    with a sprinkling of exact integers and exact .5 ties."""
    xy = torch.rand(*shape, 2, generator=gen, dtype=torch.float64)
    xy = xy * torch.tensor([W + 3.0, H + 3.0], dtype=torch.float64) - 1.5
    sel = torch.rand(*shape, generator=gen) < 0.25
    xy[sel] = torch.round(xy[sel])
    sel = torch.rand(*shape, generator=gen) < 0.1
    xy[sel] = torch.floor(xy[sel]) + 0.5
    return xy.to(dtype).contiguous()


def coords_inside(gen, shape, dtype):
    """Samples strictly inside the image, so every window of a positive input has a winner."""
    xy = torch.rand(*shape, 2, generator=gen, dtype=torch.float64)
    xy = xy * torch.tensor([W - 1.0, H - 1.0], dtype=torch.float64)
    sel = torch.rand(*shape, generator=gen) < 0.25
    xy[sel] = torch.round(xy[sel])
    return xy.to(dtype).contiguous()


def main():
    data = {}
    for dname, dtype in (("f64", torch.float64), ("f32", torch.float32)):
        gen = torch.Generator().manual_seed(20240 + (dtype == torch.float32))
        x = torch.randn(B, CIN, H, W, generator=gen, dtype=torch.float64).to(dtype)
        xneg = (-torch.rand(B, CIN, H, W, generator=gen, dtype=torch.float64) - 0.1).to(dtype)
        weight = torch.randn(COUT, CIN, K, generator=gen, dtype=torch.float64).to(dtype)
        tweight = torch.randn(CIN, COUT, K, generator=gen, dtype=torch.float64).to(dtype)
        bias = torch.randn(COUT, generator=gen, dtype=torch.float64).to(dtype)
        gout = torch.randn(B, COUT, OH, OW, generator=gen, dtype=torch.float64).to(dtype)
        gpool = torch.randn(B, CIN, OH, OW, generator=gen, dtype=torch.float64).to(dtype)
        tx = torch.randn(B, CIN, OH, OW, generator=gen, dtype=torch.float64).to(dtype)
        tgout = torch.randn(B, COUT, TOH, TOW, generator=gen, dtype=torch.float64).to(dtype)
        m_u = coords(gen, (OH, OW, K), dtype)          # unweighted kernel map
        m_w = coords(gen, (OH, OW, K, P), dtype)       # weighted kernel map
        iw = torch.rand(OH, OW, K, P, generator=gen, dtype=torch.float64).to(dtype)
        r_u = coords(gen, (OH, OW), dtype)             # unweighted resample map
        r_w = coords(gen, (OH, OW, P), dtype)
        riw = torch.rand(OH, OW, P, generator=gen, dtype=torch.float64).to(dtype)
        rin = torch.randn(B, CIN, OH, OW, generator=gen, dtype=torch.float64).to(dtype)
        xpos = (x.double().abs() + 0.5).to(dtype)
        m_ui = coords_inside(gen, (OH, OW, K), dtype)
        m_wi = coords_inside(gen, (OH, OW, K, P), dtype)
        data["%s/in/xpos" % dname] = xpos.numpy()
        data["%s/in/m_ui" % dname] = m_ui.numpy()
        data["%s/in/m_wi" % dname] = m_wi.numpy()
        for k_, v_ in dict(x=x, xneg=xneg, weight=weight, tweight=tweight, bias=bias, gout=gout,
                           gpool=gpool, tx=tx, tgout=tgout, m_u=m_u, m_w=m_w, iw=iw, r_u=r_u,
                           r_w=r_w, riw=riw, rin=rin).items():
            data["%s/in/%s" % (dname, k_)] = v_.numpy()

        for interp in (0, 1, 2):
            it = IT(interp)
            pre = "%s/i%d/" % (dname, interp)
            # convolution, unweighted and weighted
            data[pre + "conv_fwd"] = R._mapped_convolution.mapped_conv_forward(
                x, m_u, weight, bias, K, it).numpy()
            gi, gw, gb = R._mapped_convolution.mapped_conv_backward(gout, m_u, x, weight, bias, K, it)
            data[pre + "conv_gi"], data[pre + "conv_gw"], data[pre + "conv_gb"] = \
                gi.numpy(), gw.numpy(), gb.numpy()
            data[pre + "wconv_fwd"] = R._weighted_mapped_convolution.weighted_mapped_conv_forward(
                x, m_w, iw, weight, bias, K, it).numpy()
            gi, gw, gb = R._weighted_mapped_convolution.weighted_mapped_conv_backward(
                gout, m_w, iw, x, weight, bias, K, it)
            data[pre + "wconv_gi"], data[pre + "wconv_gw"], data[pre + "wconv_gb"] = \
                gi.numpy(), gw.numpy(), gb.numpy()
            # transposed convolution (map grid = input grid OH x OW, output TOH x TOW;
            # the coordinates cover 0..W+1.5 x 0..H+1.5, inside and outside the output)
            T = R._mapped_transposed_convolution
            data[pre + "tconv_fwd"] = T.mapped_transposed_conv_forward(
                tx, m_u, tweight, bias, TOH, TOW, K, it).numpy()
            gi, gw, gb = T.mapped_transposed_conv_backward(tgout, m_u, tx, tweight, bias, K, it)
            data[pre + "tconv_gi"], data[pre + "tconv_gw"], data[pre + "tconv_gb"] = \
                gi.numpy(), gw.numpy(), gb.numpy()
            T = R._weighted_mapped_transposed_convolution
            data[pre + "wtconv_fwd"] = T.weighted_mapped_transposed_conv_forward(
                tx, m_w, iw, tweight, bias, TOH, TOW, K, it).numpy()
            gi, gw, gb = T.weighted_mapped_transposed_conv_backward(
                tgout, m_w, iw, tx, tweight, bias, K, it)
            data[pre + "wtconv_gi"], data[pre + "wtconv_gw"], data[pre + "wtconv_gb"] = \
                gi.numpy(), gw.numpy(), gb.numpy()
            # pooling: values, indices, unpool; also on an all-negative input
            for tag, src in (("pool", x), ("poolneg", xneg)):
                v, i = R._mapped_max_pooling.mapped_max_pool(src, m_u, K, it)
                data[pre + tag + "_val"], data[pre + tag + "_idx"] = v.numpy(), i.numpy()
                v, i = R._weighted_mapped_max_pooling.weighted_mapped_max_pool(src, m_w, iw, K, it)
                data[pre + "w" + tag + "_val"], data[pre + "w" + tag + "_idx"] = \
                    v.numpy(), i.numpy()
            # unpool needs every index >= 0 (the reference reads sample_map[-1] otherwise)
            v, i = R._mapped_max_pooling.mapped_max_pool(xpos, m_ui, K, it)
            assert (i >= 0).all()
            data[pre + "pospool_val"], data[pre + "pospool_idx"] = v.numpy(), i.numpy()
            data[pre + "unpool"] = R._mapped_max_pooling.mapped_max_unpool(
                gpool, i, m_ui, H, W, K, it).numpy()
            v, i = R._weighted_mapped_max_pooling.weighted_mapped_max_pool(xpos, m_wi, iw, K, it)
            assert (i >= 0).all()
            data[pre + "wpospool_val"], data[pre + "wpospool_idx"] = v.numpy(), i.numpy()
            data[pre + "wunpool"] = R._weighted_mapped_max_pooling.weighted_mapped_max_unpool(
                gpool, i, m_wi, iw, H, W, K, it).numpy()
            # resampling, both directions
            data[pre + "from"] = R._resample.resample_from_map(x, r_u, it).numpy()
            data[pre + "to"] = R._resample.resample_to_map(rin, r_u, H, W, it).numpy()
            data[pre + "wfrom"] = R._weighted_resample.weighted_resample_from_map(
                x, r_w, riw, it).numpy()
            data[pre + "wto"] = R._weighted_resample.weighted_resample_to_map(
                rin, r_w, riw, H, W, it).numpy()
    np.savez_compressed(OUT, **data)
    print("wrote", OUT, len(data), "arrays", os.path.getsize(OUT), "bytes")


if __name__ == "__main__":
    main()
