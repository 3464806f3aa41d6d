"""Seeded problem generators and host<->device conversions shared by the tests.

Inputs come from numpy's Philox generator so that the oracle and the HIP path
see identical bits (the reference's jax.random streams cannot be reproduced
without JAX)."""
import numpy as np

from oracle import moe_oracle as O


def rng_for(seed):
    return np.random.Generator(np.random.Philox(seed))


def make_problem(M, D, E, k, I, SI=0, seed=0, routing="softmax", w_std=0.02):
    """Host-side problem: x (bf16-representable f32), router logits, bias, block-fp8 experts."""
    rng = rng_for(seed)
    x = O.bf16_round(rng.standard_normal((M, D), dtype=np.float32))
    logits = rng.standard_normal((M, E), dtype=np.float32)
    bias = (rng.standard_normal(E, dtype=np.float32) * np.float32(0.1)) if routing == "sigmoid_grouped" else None

    def mk(e, n, kk):
        return O.quant_weight_block(rng.standard_normal((e, n, kk), dtype=np.float32) * np.float32(w_std))

    experts = dict(gate=mk(E, I, D), up=mk(E, I, D), down=mk(E, D, I))
    shared = dict(gate=mk(1, SI, D), up=mk(1, SI, D), down=mk(1, D, SI)) if SI else None
    return dict(x=x, logits=logits, bias=bias, experts=experts, shared=shared)


# ---- torch conversions (imported lazily so CPU-only oracle tests do not need CUDA) ----

def to_bf16_cuda(x_f32):
    import torch
    return torch.from_numpy(np.ascontiguousarray(x_f32)).to(torch.bfloat16).cuda()


def bf16_to_np(t):
    import torch
    return t.detach().to(torch.float32).cpu().numpy()


def to_cuda(a):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def codes_np(t):
    import torch
    if t.dtype == torch.float8_e4m3fn:
        t = t.view(torch.uint8)
    return t.detach().cpu().numpy()


def experts_to_cuda(ex):
    """oracle dict gate/up/down -> (codes, scale_inv)  ==>  product dict gate_proj/... -> {'w','scale_inv'}."""
    import torch
    return {n + "_proj": {"w": to_cuda(q).view(torch.float8_e4m3fn), "scale_inv": to_cuda(s)} for n, (q, s) in ex.items()}


def assert_close_out(got, want, tol=1e-2, inner=None):
    """The output tolerance (bf16 results against the oracle's exact arithmetic).

    (1) max|y - ref| / max|ref| <= tol          -- the bound the benchmark definition states; for a
        contraction shorter than 1024 after the fp8 re-quantisation the bound is tol * sqrt(1024 / inner),
        because one flipped intermediate code (below) weighs more against a shorter sum: random small
        shapes reach 1.0e-2 ... 1.15e-2 at inner = 256 / 512 in about one case in twenty (median row
        error stays below 1e-3); every config of BASELINE.json with inner >= 1024 is held to tol itself;
    (2) row-wise ||y - ref||_2 / ||ref||_2: mean over rows <= 0.4*tol (16 rows or more), every row
        <= tol + 0.45/sqrt(inner), where `inner` is the length of the contraction that
        follows an fp8 re-quantisation (the expert intermediate size; None = no such stage);
    (3) every element within 5x of |y - ref| <= tol*|ref| + tol*rms(ref) (5x * sqrt(1024 / inner) for a
        contraction shorter than 1024, as in (1)).
    A strict elementwise allclose cannot hold end to end: the fp8 matrix instruction
    sums a 128-long block with about 2^-16 relative error (measured on gfx950, both
    the K=128 and K=32 forms), so a few of the intermediate h values land on the
    other side of an e4m3 rounding boundary than the oracle's.  One such step (up to
    2^-3 relative) on an outlier h element (~4.5 rms) moves its whole output row by
    up to ~0.45/sqrt(inner) in relative L2 -- hence the second term of (2).  The
    stage-wise tests, which feed each kernel the oracle's own inputs, carry the
    tight bounds."""
    got = np.asarray(got, np.float64)
    want = np.asarray(want, np.float64)
    assert got.shape == want.shape
    assert np.isfinite(got).all()
    denom = np.abs(want).max()
    err = np.abs(got - want).max() / (denom if denom > 0 else 1.0)
    short = max(1.0, float(np.sqrt(1024.0 / inner))) if inner else 1.0   # > 1 only for contractions shorter than 1024
    max_tol = tol * short
    assert err <= max_tol, f"max-normalised error {err:.3e} > {max_tol:.3e}"
    g2, w2 = got.reshape(-1, got.shape[-1]), want.reshape(-1, want.shape[-1])
    rown = np.linalg.norm(w2, axis=1)
    rel = np.linalg.norm(g2 - w2, axis=1) / np.where(rown > 0, rown, 1.0)
    row_tol = tol + (0.45 / np.sqrt(inner) if inner else 0.0)
    assert rel.max() <= row_tol, f"row {rel.argmax()} has relative L2 error {rel.max():.3e} > {row_tol:.3e}"
    if rel.size >= 16:   # a statistic over rows: with a handful of rows one flipped code is the whole mean
        assert rel.mean() <= 0.4 * tol, f"mean row relative L2 error {rel.mean():.3e} > {0.4 * tol}"
    rms = np.sqrt(np.mean(want ** 2))
    ratio = np.abs(got - want) / (tol * np.abs(want) + tol * rms + 1e-30)
    assert ratio.max() <= 5.0 * short, f"worst element is {ratio.max():.1f}x the elementwise bound (limit {5.0 * short:.1f}x)"
    return err
