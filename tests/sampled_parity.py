"""Element-wise oracle checks at sizes where the oracle cannot evaluate a whole tensor.

TEST INFRASTRUCTURE: used by tests/ and by the benchmark's verification step after its timed
loop.  The mapped operators are local in the map: output pixel m depends on the map entry of m
only, and the gradients are linear in grad_output.  So the oracle, handed the *full* image and
the map *sliced* to a set of pixels, returns exactly the values the full evaluation would give
on those pixels:

  forward            y[:, :, pix]            = oracle_forward(x, map[pix])
  backward, sparse g grad_input, grad_weight = oracle_backward(g[pix], map[pix], x)   for a
                                               grad_output that is zero outside pix
  backward, dense g  grad_input[:, :, tgt]   = oracle_backward_input(g[src], map[src])[tgt]
                                               where src = every map pixel with a tap in tgt
                     grad_weight[ns][:, cs]  = oracle_backward(g[:, ns], map, x[:, cs])'s
                                               grad_weight: an entry (n, c, k) of the weight
                                               gradient sums over batch and pixels only, so
                                               the oracle on channel subsets of x and g (whole
                                               map, every pixel) returns the full evaluation's
                                               entries for those channels

No formula is restated here: only the oracle's own entry points are called, on sliced maps.
"""
import numpy as np


def relerr(a, b):
    """max|a-b| / max|b| (the norm-relative error every tolerance in this suite refers to)."""
    a = np.asarray(a, np.float64)
    b = np.asarray(b, np.float64)
    return float(np.abs(a - b).max() / max(np.abs(b).max(), 1e-30))


def sample_pixels(OH, OW, n_random, seed, rows=(0, 1, -2, -1), cols=(0, -1)):
    """Sorted flat indices: whole rows (the poles of an equirectangular grid), whole columns (the
    longitude seam) and n_random pixels drawn uniformly."""
    rng = np.random.default_rng(seed)
    sel = np.zeros((OH, OW), bool)
    for r in rows:
        if -OH <= r < OH:
            sel[r] = True
    for c in cols:
        if -OW <= c < OW:
            sel[:, c] = True
    flat = sel.reshape(-1)
    flat[rng.integers(0, OH * OW, n_random)] = True
    return np.flatnonzero(flat)


def slice_map(sample_map, interp_weights, pix):
    """The map and weights of the pixels `pix` as a one-row grid [1, n, K, (P,) 2]."""
    OH, OW = sample_map.shape[:2]
    m = np.ascontiguousarray(sample_map.reshape((OH * OW,) + sample_map.shape[2:])[pix][None])
    if interp_weights is None:
        return m, None
    w = interp_weights.reshape((OH * OW,) + interp_weights.shape[2:])[pix][None]
    return m, np.ascontiguousarray(w)


def sources_touching(sample_map, H, W, targets):
    """Flat indices of the map pixels that own a tap which can fall on one of the image pixels
    `targets` (flat indices into H x W).  A superset for every interpolation type: a sample at
    (x, y) touches at most columns floor(x), floor(x)+1 (taken modulo W, which covers the
    wrapped neighbours of bispherical interpolation and the rounded one of nearest) and rows
    floor(y), floor(y)+1."""
    mask = np.zeros(H * W, bool)
    mask[targets] = True
    mask = mask.reshape(H, W)
    OH, OW = sample_map.shape[:2]
    pts = sample_map.reshape(OH * OW, -1, 2).astype(np.float64)
    fx = np.floor(pts[..., 0]).astype(np.int64)
    fy = np.floor(pts[..., 1]).astype(np.int64)
    hit = np.zeros(OH * OW, bool)
    for dy in (0, 1):
        ty = fy + dy
        ok = (ty >= 0) & (ty <= H - 1)
        tyc = np.clip(ty, 0, H - 1)
        for dx in (0, 1):
            tx = np.mod(fx + dx, W)
            hit |= (mask[tyc, tx] & ok).any(axis=1)
    return np.flatnonzero(hit)


def at(t, pix):
    """[B, C, OH, OW] tensor or array -> numpy [B, C, 1, n] at the flat pixels pix."""
    if hasattr(t, "detach"):
        import torch
        idx = torch.from_numpy(np.asarray(pix)).to(t.device)
        t = t.detach().reshape(t.shape[0], t.shape[1], -1).index_select(2, idx).cpu().numpy()
    else:
        t = t.reshape(t.shape[0], t.shape[1], -1)[:, :, pix]
    return np.ascontiguousarray(t[:, :, None, :])


def sparse_like(g, pix):
    """A copy of the numpy tensor g [B, C, OH, OW] that is zero outside the flat pixels pix."""
    out = np.zeros_like(g)
    flat = out.reshape(g.shape[0], g.shape[1], -1)
    flat[:, :, pix] = g.reshape(g.shape[0], g.shape[1], -1)[:, :, pix]
    return out


class ConvOracle:
    """Oracle answers of one mapped-convolution configuration on pixel samples, computed once
    and compared with any number of GPU evaluations (compute modes) of the same inputs.

    cfg: dict of numpy arrays as workloads.config4 / config5 return them."""

    def __init__(self, oracle, cfg, n_random, n_targets, seed=0, rows=(0, 1, -2, -1),
                 cols=(0, -1), n_weight_channels=0):
        """n_weight_channels: how many output and input channels (first, last and random ones
        between) the dense weight gradient is evaluated on by the oracle; 0 leaves it out."""
        self.cfg = cfg
        m, iw = cfg["sample_map"], cfg.get("interp_weights")
        x, w, b, g = cfg["x"], cfg["weight"], cfg["bias"], cfg["grad_output"]
        K, it = cfg["kernel_size"], cfg["interp"]
        H, W = x.shape[2:]
        OH, OW = m.shape[:2]
        self.pix = sample_pixels(OH, OW, n_random, seed, rows, cols)
        ms, ws = slice_map(m, iw, self.pix)
        self.forward = oracle.mapped_conv_forward(x, ms, w, b, K, it, ws)
        self.g_sparse = sparse_like(g, self.pix)
        self.grad_input, self.grad_weight, self.grad_bias = oracle.mapped_conv_backward(
            at(g, self.pix), ms, x, w, b, K, it, ws)
        # dense grad_output, grad_input on sampled image pixels
        self.targets = sample_pixels(H, W, n_targets, seed + 1, rows[:1] + rows[-1:], cols[:1])
        self.sources = sources_touching(m, H, W, self.targets)
        ms, ws = slice_map(m, iw, self.sources)
        gi = oracle.mapped_conv_backward_input(at(g, self.sources), ms, x.shape, w, K, it, ws)
        self.grad_input_dense = at(gi, self.targets)
        # dense grad_output, grad_weight on channel subsets
        self.w_out = self.w_in = None
        if n_weight_channels:
            rng = np.random.default_rng(seed + 2)

            def pick(n):
                k = min(int(n_weight_channels), n)
                mid = rng.choice(np.arange(1, n - 1), size=max(k - 2, 0), replace=False) \
                    if n > 2 else np.zeros(0, np.int64)
                return np.unique(np.concatenate([[0, n - 1], mid]).astype(np.int64))[:max(k, 1)]
            self.w_out, self.w_in = pick(w.shape[0]), pick(w.shape[1])
            _, self.grad_weight_dense, _ = oracle.mapped_conv_backward(
                np.ascontiguousarray(g[:, self.w_out]), m, np.ascontiguousarray(x[:, self.w_in]),
                np.ascontiguousarray(w[self.w_out][:, self.w_in]), b[self.w_out], K, it, iw)

    def check_forward(self, y):
        return relerr(at(y, self.pix), self.forward)

    def check_backward_sparse(self, gi, gw, gb):
        """gi, gw, gb: what the GPU returned for grad_output = self.g_sparse."""
        n = lambda t: t.detach().cpu().numpy()  # noqa: E731
        return (relerr(n(gi), self.grad_input), relerr(n(gw), self.grad_weight),
                relerr(n(gb), self.grad_bias))

    def check_backward_dense(self, gi):
        """gi: the GPU's grad_input for the configuration's dense grad_output."""
        return relerr(at(gi, self.targets), self.grad_input_dense)

    def check_weight_dense(self, gw):
        """gw: the GPU's grad_weight [Cout, Cin, K] for the dense grad_output, compared on
        the channel subsets the oracle evaluated."""
        gw = gw.detach().cpu().numpy() if hasattr(gw, "detach") else np.asarray(gw)
        return relerr(gw[self.w_out][:, self.w_in], self.grad_weight_dense)
