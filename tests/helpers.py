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


def assert_close_out(got, want, tol=1e-2):
    """The output tolerance of the benchmark definition, as it stands: bf16 results against the oracle's exact
    arithmetic must satisfy  max|y - ref| / max|ref| <= tol  and  allclose(rtol=tol, atol=tol * rms(ref)).
    Returns the max-normalised error."""
    got = np.asarray(got, np.float64)
    want = np.asarray(want, np.float64)
    assert got.shape == want.shape
    assert np.isfinite(got).all()
    denom = np.abs(want).max()
    err = np.abs(got - want).max() / (denom if denom > 0 else 1.0)
    assert err <= tol, f"max-normalised error {err:.3e} > {tol:.3e}"
    rms = np.sqrt(np.mean(want ** 2))
    excess = np.abs(got - want) - (tol * np.abs(want) + tol * rms)
    assert excess.max() <= 0, (f"allclose(rtol={tol}, atol={tol}*rms) fails at {np.unravel_index(excess.argmax(), excess.shape)}: "
                               f"got {got.flat[excess.argmax()]:.6g}, want {want.flat[excess.argmax()]:.6g}, rms {rms:.3g}")
    return err


def max_norm_err(got, want):
    """max|y - ref| / max|ref| (a printed diagnostic where the assertion is made elsewhere)."""
    got, want = np.asarray(got, np.float64), np.asarray(want, np.float64)
    denom = np.abs(want).max()
    return float(np.abs(got - want).max() / (denom if denom > 0 else 1.0))


def _code_ordinal(codes):
    """e4m3fn codes as signed ordinals: neighbouring representable values differ by one."""
    c = np.asarray(codes, np.uint8).astype(np.int32)
    mag = c & 0x7F
    return np.where(c & 0x80, -mag, mag)


def assert_h_close(hq, sh, ref_hq, ref_sh, what="h"):
    """The quantised SwiGLU intermediate of the kernel against the oracle's.  The two differ where the matrix
    unit's f32 block sums (about 2^-16 relative to the sum of magnitudes) put a value on the other side of an
    e4m3 rounding boundary than exact arithmetic does: on fewer than 0.5 % of the elements (or two), and there by one code
    step -- or, for values that cancel to nearly zero, by less than a tenth of a scale unit in absolute terms.
    Scales (amax / 448 of a 128-wide group) agree to 1e-3."""
    hq, ref_hq = np.asarray(hq, np.uint8), np.asarray(ref_hq, np.uint8)
    sh, ref_sh = np.asarray(sh, np.float32), np.asarray(ref_sh, np.float32)
    assert hq.shape == ref_hq.shape and sh.shape == ref_sh.shape
    assert np.allclose(sh, ref_sh, rtol=1e-3, atol=0), f"{what}: scales differ"
    diff = hq != ref_hq
    frac = float(diff.mean()) if diff.size else 0.0
    # (a handful of codes in a small array is not a rate: two are let through whatever the size)
    assert int(diff.sum()) <= max(2, int(5e-3 * diff.size)), f"{what}: {frac:.2%} of the codes differ from the oracle's"
    if diff.any():
        step = np.abs(_code_ordinal(hq) - _code_ordinal(ref_hq))
        from oracle import moe_oracle as O_
        absd = np.abs(O_.dequant_act_group(hq, sh) - O_.dequant_act_group(ref_hq, ref_sh))
        near_zero = absd <= 0.1 * np.repeat(ref_sh, 128, axis=-1)
        bad = diff & (step > 1) & ~near_zero
        assert not bad.any(), f"{what}: {int(bad.sum())} codes are more than one step from the oracle's"
    return frac


# Intermediate sizes below this are outside the end-to-end contract: one e4m3 step on one element of h moves its
# output row by up to ~0.45 / sqrt(I) of the row's size, so a single boundary case among a few hundred h elements
# can exceed 1e-2 end to end (measured on random small layers: 2.3e-2 at I = 128, 1.5e-2 at I = 384, <= 7.5e-3 from
# I = 512 up, which covers every configuration of the benchmark definition: I = 768, 1024, 2048).
E2E_MIN_INTERMEDIATE = 512
E2E_SMALL_TOL = 3e-2


def end_to_end_tol(I, tol=1e-2):
    """The bound on max|out - oracle| / max|oracle| of a whole-path call against the oracle on its own."""
    return tol if I >= E2E_MIN_INTERMEDIATE else E2E_SMALL_TOL


def check_layer_output(out, dbg, ref, rerun, tol=1e-2, shared_gate=None, residual=None):
    """End-to-end check of a whole-path call against the oracle.  The path rounds twice on the way (the SwiGLU
    output to fp8, the down GEMM's rows to bf16, as the reference's ragged_dot does), and a value that exact
    arithmetic puts just on one side of such a rounding boundary may land on the other side in f32 matrix
    arithmetic; one such step is larger than the output tolerance allows for a whole element.  So the comparison is
    made stage by stage, every stage held to the benchmark's tolerance AS IT STANDS (assert_close_out: 1e-2
    max-normalised and allclose(rtol=1e-2, atol=1e-2 rms)) on the kernel's own inputs to that stage:
      (1) the kernel's fp8 intermediate h (hq/sh; hsq/shs of the shared expert) against the oracle's own: codes
          equal but for < 0.5 % that sit on a rounding boundary, those one code step apart (assert_h_close);
      (2) the kernel's down-GEMM rows y (and ys) against the oracle continued from the kernel's h;
      (3) the kernel's output against the oracle's combine of the kernel's y, ys, routing weights and gate:
          bit for bit (an f32 sum in slot order and one rounding);
      (4) the output against the oracle continued from the kernel's h: max-normalised error <= 1e-2, and the
          elementwise allclose wherever no bf16 step of a y row explains the difference (every exception is
          counted; they stay below 0.1 % of the elements);
      (5) the output against the oracle ON ITS OWN (identical inputs, nothing taken from the kernel): max-normalised
          error <= 1e-2, the tolerance of the benchmark definition, for intermediate sizes from
          E2E_MIN_INTERMEDIATE up (end_to_end_tol; below that a single fp8 boundary case can exceed it and the
          bound is E2E_SMALL_TOL).
    `ref` is the oracle on its own, `rerun(routed_h=, shared_h=)` the oracle continued from given intermediates.
    Returns (error of (4), end-to-end error against `ref`, fraction of h codes that differ)."""
    from oracle import moe_oracle as O_
    hq, sh = codes_np(dbg["hq"]), dbg["sh"].cpu().numpy()
    frac = assert_h_close(hq, sh, ref["hq"], ref["sh"], "routed h")
    shared_h = None
    if ref.get("hsq") is not None:
        hsq, shs = codes_np(dbg["hsq"]), dbg["shs"].cpu().numpy()
        assert_h_close(hsq, shs, ref["hsq"], ref["shs"], "shared h")
        shared_h = (hsq, shs)
    ref2 = rerun(routed_h=(hq, sh), shared_h=shared_h)
    y = bf16_to_np(dbg["y"])
    assert_close_out(y, ref2["y"], tol)
    ys = None
    if shared_h is not None:
        ys = bf16_to_np(dbg["ys"])
        assert_close_out(ys, ref2["shared_out"], tol)
    got = bf16_to_np(out)
    w = dbg["weights"].cpu().numpy()
    exact = O_.combine(y, w, ref["inv_perm"], ys, shared_gate, residual)
    assert np.array_equal(got, exact), "the output is not the exact combine of the kernel's own rows"
    err = max_norm_err(got, ref2["out"])
    assert err <= tol, f"max-normalised error {err:.3e} > {tol:.3e}"
    assert_allclose_but_for_row_steps(got, ref2["out"], y, ref2["y"], ys, ref2["shared_out"], w, ref["inv_perm"], shared_gate, tol)
    e2e = max_norm_err(got, ref["out"])
    bound = end_to_end_tol(hq.shape[-1], tol)
    assert e2e <= bound, f"end-to-end max-normalised error {e2e:.3e} > {bound:.1e} against the oracle on identical inputs"
    return err, e2e, frac


def _bf16_step(v):
    """spacing of bf16 values at |v| (2^-7 of the power of two below it)"""
    v = np.abs(np.asarray(v, np.float64))
    return np.where(v > 0, 2.0 ** (np.floor(np.log2(np.maximum(v, 1e-300))) - 7), 0.0)


def assert_allclose_but_for_row_steps(got, want, y, y_ref, ys, ys_ref, w, inv_perm, shared_gate, tol):
    """allclose(rtol=tol, atol=tol*rms) of the output, except where the kernel's bf16 rows y differ from the oracle's
    (by a rounding step): there the bound is widened by exactly the weighted size of those differences."""
    M, k = w.shape
    pos = np.asarray(inv_perm).reshape(M, k)
    slack = np.zeros_like(np.asarray(want, np.float64))
    for s_ in range(k):
        slack += np.abs(y[pos[:, s_]].astype(np.float64) - y_ref[pos[:, s_]]) * np.abs(w[:, s_:s_ + 1]).astype(np.float64)
    if ys is not None:
        g = 1.0 if shared_gate is None else np.asarray(shared_gate, np.float64)[:, None]
        slack += np.abs(ys.astype(np.float64) - ys_ref) * g
    got, want = np.asarray(got, np.float64), np.asarray(want, np.float64)
    rms = np.sqrt(np.mean(want ** 2))
    bound = tol * np.abs(want) + tol * rms
    diff = np.abs(got - want)
    # (where a y row differs, the rounded sum may also land one bf16 step of the output away: that step is granted
    # only there)
    widened = bound + np.where(slack > 0, 1.01 * slack + _bf16_step(want), 0.0)
    assert (diff <= widened).all(), "an output element is outside the tolerance and no row step explains it"
    outside = diff > bound
    assert outside.mean() < 1e-3, f"{outside.mean():.3%} of the output elements lean on a row's rounding step"
    return int(outside.sum())


def kernel_gate(dbg, oracle_gate):
    """The shared expert's gate values the kernel computed (a bf16 sigmoid of a bf16 matmul result), checked against
    the oracle's order-free ones: equal but for the few tokens whose logit sits on a bf16 rounding boundary, and
    there within two bf16 steps.  Returned for the oracle to continue from, as it continues from the kernel's
    router logits."""
    got = dbg["shared_gate"].cpu().numpy()
    want = np.asarray(oracle_gate, np.float32)
    assert got.shape == want.shape
    assert float((got != want).mean()) < 0.02 or got.size < 100 and int((got != want).sum()) <= 2
    assert np.abs(got - want).max() <= 2.0 ** -7
    return got
