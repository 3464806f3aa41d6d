"""Pins the CPU oracle (oracle/moe_oracle.py) against independent statements:
torch's CPU casts, float64 library routines, brute force, closed forms and the
one known-answer test the reference holds for this path."""
import itertools

import numpy as np
import pytest
import torch

from oracle import moe_oracle as O
from tests import helpers as H


# ---------------------------------------------------------------- codecs

def test_e4m3_table_matches_torch_exhaustively():
    codes = np.arange(256, dtype=np.uint8)
    ref = torch.from_numpy(codes).view(torch.float8_e4m3fn).to(torch.float32).numpy()
    got = O.e4m3_decode(codes)
    assert np.array_equal(np.isnan(ref), np.isnan(got))
    m = ~np.isnan(ref)
    assert np.array_equal(ref[m], got[m])
    assert got[0x7E] == 448.0 and got[0x08] == 2.0 ** -6 and got[0x01] == 2.0 ** -9


def test_e4m3_encode_matches_torch_dense_sweep():
    rng = np.random.default_rng(0)
    x = np.concatenate([
        rng.normal(0, 1, 200000), rng.normal(0, 100, 200000), rng.normal(0, 0.01, 200000),
        np.linspace(-448, 448, 100001), np.array([0.0, -0.0, 448.0, -448.0, 2.0 ** -9, 2.0 ** -10, 3 * 2.0 ** -10]),
    ]).astype(np.float32)
    x = np.clip(x, -448, 448)
    # every midpoint between adjacent codes (the ties that decide round-to-nearest-even)
    pos = np.sort(O.E4M3_TABLE[:0x7F])
    mids = ((pos[:-1].astype(np.float64) + pos[1:]) / 2).astype(np.float32)
    x = np.concatenate([x, mids, -mids, np.nextafter(mids, np.float32(0)), np.nextafter(mids, np.float32(1e9))])
    ref = torch.from_numpy(x).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    got = O.e4m3_encode(x)
    assert np.array_equal(ref, got)


def test_e4m3_roundtrip_identity_on_codes():
    codes = np.array([c for c in range(256) if c & 0x7F != 0x7F], dtype=np.uint8)
    assert np.array_equal(O.e4m3_encode(O.e4m3_decode(codes)), codes)


def test_bf16_matches_torch():
    rng = np.random.default_rng(1)
    x = np.concatenate([rng.normal(0, 1, 100000), rng.normal(0, 1e-3, 1000), [0.0, -0.0, 1.0, 65504.0, 3.3895314e38]]).astype(np.float32)
    ref = torch.from_numpy(x).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(O.f32_to_bf16_bits(x), ref)
    assert np.array_equal(O.bf16_bits_to_f32(ref), torch.from_numpy(x).to(torch.bfloat16).float().numpy())


# ---------------------------------------------------------------- quantisers

def test_quant_weight_block_scales_and_bound():
    rng = np.random.default_rng(2)
    w = (rng.normal(0, 0.02, (3, 256, 384))).astype(np.float32)
    w[1, :128, 128:256] = 0.0                      # an all-zero block keeps scale 1
    q, sinv = O.quant_weight_block(w)
    assert q.shape == w.shape and sinv.shape == (3, 2, 3)
    blocks = np.abs(w.reshape(3, 2, 128, 3, 128)).max(axis=(2, 4))
    want = np.where(blocks > 0, blocks / 448.0, 1.0)
    assert np.allclose(sinv, want, rtol=3e-7)
    assert sinv[1, 0, 1] == 1.0 and not q[1, :128, 128:256].any()
    deq = O.dequant_weight_block(q, sinv)
    s = np.repeat(np.repeat(sinv, 128, axis=1), 128, axis=2)
    assert np.all(np.abs(deq - w) <= 2.0 ** -4 * np.abs(w) + 2.0 ** -10 * s + 1e-12)
    # the block maximum lands exactly on +-448
    assert np.abs(O.e4m3_decode(q)).reshape(3, 2, 128, 3, 128).max(axis=(2, 4))[0, 0, 0] == 448.0
    # blocks are independent: changing one block leaves every other code alone
    w2 = w.copy(); w2[0, :128, :128] *= 3.0
    q2, _ = O.quant_weight_block(w2)
    same = np.ones_like(w, dtype=bool); same[0, :128, :128] = False
    assert np.array_equal(q[same], q2[same])


def test_quant_matches_hf_block_formula_in_torch():
    """HF finegrained_fp8 block quantiser restated with torch ops (scale=448/amax,
    clamp, cast) gives the same codes and inverse scales."""
    rng = np.random.default_rng(3)
    w = rng.normal(0, 0.02, (256, 256)).astype(np.float32)
    t = torch.from_numpy(w).reshape(2, 128, 2, 128)
    amax = t.abs().amax(dim=(1, 3))
    scale = torch.full_like(amax, 448.0) / amax     # tensor/tensor: IEEE quotient (scalar/tensor is mul-by-reciprocal)
    qt = torch.clamp(t * scale[:, None, :, None], -448, 448).to(torch.float8_e4m3fn).reshape(256, 256)
    q, sinv = O.quant_weight_block(w)
    assert np.array_equal(q, qt.view(torch.uint8).numpy())
    assert np.array_equal(sinv, (torch.ones_like(scale) / scale).numpy())
    assert np.array_equal(sinv, (1.0 / scale.numpy().astype(np.float64)).astype(np.float32))


def test_quant_act_group():
    rng = np.random.default_rng(4)
    x = O.bf16_round(rng.normal(0, 1, (37, 512)).astype(np.float32))
    x[5] = 0.0
    q, sinv = O.quant_act_group(x)
    assert q.shape == (37, 512) and sinv.shape == (37, 4)
    assert np.all(sinv[5] == 1.0) and not q[5].any()
    deq = O.dequant_act_group(q, sinv)
    assert np.all(np.abs(deq - x) <= 2.0 ** -4 * np.abs(x) + 2.0 ** -10 * np.repeat(sinv, 128, axis=1))
    # row groups are independent of each other
    qa, sa = O.quant_act_group(x[:, 128:256])
    assert np.array_equal(qa, q[:, 128:256]) and np.array_equal(sa[:, 0], sinv[:, 1])


# ---------------------------------------------------------------- exp / sigmoid

def _ulp_err(got, ref64):
    ref32 = ref64.astype(np.float32)
    return np.abs(got.astype(np.float64) - ref64) / np.spacing(np.abs(ref32)).astype(np.float64)


def test_exp_det_accuracy():
    x = np.linspace(-80, 80, 400001).astype(np.float32)
    assert _ulp_err(O.exp_det(x), np.exp(x.astype(np.float64))).max() <= 2.0
    assert O.exp_det(np.float32(0.0)) == 1.0


def test_sigmoid_det_accuracy_and_monotone():
    x = np.linspace(-30, 30, 200001).astype(np.float32)
    s = O.sigmoid_det(x)
    ref = 1.0 / (1.0 + np.exp(-x.astype(np.float64)))
    assert _ulp_err(s, ref).max() <= 4.0
    assert np.all(np.diff(s) >= 0) and O.sigmoid_det(np.float32(0)) == 0.5


# ---------------------------------------------------------------- routing

def _brute_topk(row, k):
    """rank(i) = #{j: v_j > v_i} + #{j < i: v_j == v_i}; the k smallest ranks in rank order."""
    E = len(row)
    rank = [sum(1 for j in range(E) if row[j] > row[i] or (row[j] == row[i] and j < i)) for i in range(E)]
    out = [0] * k
    for i, r in enumerate(rank):
        if r < k:
            out[r] = i
    return out


def test_softmax_routing_brute_force_and_sum_to_one():
    rng = np.random.default_rng(5)
    logits = rng.normal(0, 1, (64, 16)).astype(np.float32)
    logits[3, 4] = logits[3, 9] = logits[3].max() + 1       # a tie for first place
    logits[7, :] = 0.25                                      # all tied
    logits[8, 2] = -0.0; logits[8, 5] = 0.0; logits[8, [0, 1, 3, 4] + list(range(6, 16))] = -1
    for k in (1, 2, 8):
        idx, w = O.route_softmax_topk(logits, k)
        for t in range(64):
            assert list(idx[t]) == _brute_topk(list(logits[t]), k)
        assert np.allclose(w.sum(-1), 1.0, atol=1e-5)        # reference tests/qwen35/test_moe.py:52-60
        p = np.exp(logits.astype(np.float64)); p /= p.sum(-1, keepdims=True)
        sel = np.take_along_axis(p, idx.astype(np.int64), -1)
        assert np.allclose(w, sel / sel.sum(-1, keepdims=True), rtol=1e-5)
        # top-k of softmax == top-k of logits
        assert np.array_equal(idx, O._topk_desc(p.astype(np.float32), k)) or k == 8
    assert list(idx[3][:2]) == [4, 9] and list(idx[7]) == list(range(8)) and idx[8][0] == 2
    idx, w = O.route_softmax_topk(logits, 2, renorm=False)
    assert np.allclose(w, np.take_along_axis(p, idx.astype(np.int64), -1), rtol=1e-5)


def _brute_grouped(logit_row, bias, n_group, topk_group, k):
    E = len(logit_row)
    per = E // n_group
    sc = [float(O.sigmoid_det(np.float32(v))) for v in logit_row]
    ch = [np.float32(np.float32(sc[i]) + np.float32(bias[i])) for i in range(E)]
    gs = []
    for g in range(n_group):
        grp = [ch[g * per + j] for j in range(per)]
        t2 = _brute_topk(grp, 2)
        gs.append(np.float32(grp[t2[0]] + grp[t2[1]]))
    keep = set(_brute_topk(gs, topk_group))
    masked = [ch[i] if (i // per) in keep else np.float32(-np.inf) for i in range(E)]
    return _brute_topk(masked, k), sc


def test_sigmoid_grouped_routing_brute_force():
    rng = np.random.default_rng(6)
    M, E, G, TG, k = 48, 32, 4, 2, 4
    logits = rng.normal(0, 1, (M, E)).astype(np.float32)
    bias = rng.normal(0, 0.1, E).astype(np.float32)
    logits[5, :] = 0.0                                      # every score tied -> bias decides, then index
    idx, w = O.route_sigmoid_grouped(logits, bias, G, TG, k, renorm=True, routed_scale=2.5)
    for t in range(M):
        want, sc = _brute_grouped(logits[t], bias, G, TG, k)
        assert list(idx[t]) == want
        sel = np.array([sc[i] for i in want], dtype=np.float64)
        assert np.allclose(w[t], 2.5 * sel / (sel.sum() + 1e-20), rtol=1e-5)
    assert np.allclose(w.sum(-1), 2.5, rtol=1e-5)


def test_sigmoid_grouped_special_cases_reduce_to_plain_topk():
    rng = np.random.default_rng(7)
    logits = rng.normal(0, 1, (40, 64)).astype(np.float32)
    plain = O._topk_desc(logits, 6)                          # sigmoid is monotone, bias 0
    for G, TG in ((1, 1), (8, 8), (4, 4)):
        idx, w = O.route_sigmoid_grouped(logits, None, G, TG, 6, renorm=False)
        assert np.array_equal(idx, plain)
        assert np.allclose(w, 1 / (1 + np.exp(-np.take_along_axis(logits, plain.astype(np.int64), -1).astype(np.float64))), rtol=1e-6)
    # selected experts always lie in the kept groups and never exceed them
    bias = rng.normal(0, 0.1, 64).astype(np.float32)
    idx, _ = O.route_sigmoid_grouped(logits, bias, 8, 3, 6)
    assert all(len(set(r // 8)) <= 3 for r in idx)
    assert all(len(set(r)) == 6 for r in idx)


# ---------------------------------------------------------------- sort / group

@pytest.mark.parametrize("M,k,E", [(1, 1, 4), (7, 2, 8), (256, 2, 8), (333, 8, 128), (64, 8, 256)])
def test_sort_and_group_invariants(M, k, E):
    rng = np.random.default_rng(8)
    idx = np.stack([rng.choice(E, k, replace=False) for _ in range(M)]).astype(np.int32)
    if E >= 8:
        idx[idx == 3] = 4 if k == 1 else idx[idx == 3]       # harmless; keeps rows distinct for k>1
    sg = O.sort_and_group(idx, E)
    R = M * k
    flat = idx.reshape(-1)
    assert np.array_equal(sg["group_sizes"], np.bincount(flat, minlength=E))
    assert sg["group_sizes"].sum() == R and sg["group_offsets"][-1] == R
    se = flat[sg["sort_order"]]
    assert np.all(np.diff(se) >= 0)
    for e in range(E):                                        # within an expert: ascending flat index
        seg = sg["sort_order"][sg["group_offsets"][e]:sg["group_offsets"][e + 1]]
        assert np.all(np.diff(seg) > 0) and np.all(flat[seg] == e)
    assert np.array_equal(sg["sorted_token_ids"], sg["sort_order"] // k)
    assert np.array_equal(sg["sort_order"][sg["inv_perm"]], np.arange(R))
    assert np.array_equal(np.bincount(sg["sorted_token_ids"], minlength=M), np.full(M, k))
    # textbook counting sort gives the same permutation
    pos = sg["group_offsets"][:-1].copy(); want = np.empty(R, np.int32)
    for f in range(R):
        want[pos[flat[f]]] = f; pos[flat[f]] += 1
    assert np.array_equal(want, sg["sort_order"])


# ---------------------------------------------------------------- GEMM / combine

def test_grouped_gemm_reference_known_answer():
    """reference tests/qwen35/test_fp8.py:65-75: ones(2,K) . ones(3,K)^T with the weight
    worth 0.5 per element -> K/2 (the reference uses K=4 -> 2.0; blocks here need K=128 -> 64)."""
    K = 128
    xq, sx = O.quant_act_group(np.ones((2, K), np.float32))
    wq = O.e4m3_encode(np.ones((1, 128, K), np.float32))
    sw = np.full((1, 1, 1), 0.5, np.float32)
    out = O.grouped_gemm(xq, sx, wq, sw, np.array([0, 2]))
    assert out.shape == (2, 128) and np.allclose(out, K * 0.5, rtol=1e-6)
    assert np.allclose(out / (K / 4), 2.0, atol=0.1)


def test_grouped_gemm_vs_per_row_bruteforce_and_ragged_edges():
    rng = np.random.default_rng(9)
    E, N, K = 5, 128, 256
    sizes = np.array([3, 0, 7, 1, 0]); off = np.concatenate([[0], np.cumsum(sizes)])
    R = off[-1]
    xq, sx = O.quant_act_group(rng.normal(0, 1, (R + 2, K)).astype(np.float32))   # 2 rows beyond sum(gs)
    wq, sw = O.quant_weight_block(rng.normal(0, 0.02, (E, N, K)).astype(np.float32))
    out = O.grouped_gemm(xq, sx, wq, sw, off)
    assert not out[R:].any()                                   # rows >= sum(group_sizes) are zero (ragged_dot)
    xd = O.e4m3_decode(xq).astype(np.float64); wd = O.e4m3_decode(wq).astype(np.float64)
    for r in range(R):
        e = int(np.searchsorted(off, r, side="right") - 1)
        for n in (0, 5, 127):
            acc = 0.0
            for kb in range(K // 128):
                part = float(np.dot(xd[r, kb * 128:(kb + 1) * 128], wd[e, n, kb * 128:(kb + 1) * 128]))
                acc += part * float(sx[r, kb]) * float(sw[e, n // 128, kb])
            assert abs(out[r, n] - acc) <= 1e-9 * max(1.0, abs(acc))


def _tiny_problem(seed=10, M=24, D=256, E=4, k=2, I=128, shared=True):
    rng = np.random.default_rng(seed)
    x = O.bf16_round(rng.normal(0, 1, (M, D)).astype(np.float32))
    logits = rng.normal(0, 1, (M, E)).astype(np.float32)
    mk = lambda e, n, kk: O.quant_weight_block(rng.normal(0, 0.05, (e, n, kk)).astype(np.float32))
    experts = dict(gate=mk(E, I, D), up=mk(E, I, D), down=mk(E, D, I))
    sh = dict(gate=mk(1, I, D), up=mk(1, I, D), down=mk(1, D, I)) if shared else None
    return x, logits, experts, sh


def test_moe_experts_vs_per_token_loop():
    x, logits, experts, sh = _tiny_problem()
    res = O.moe_experts(x, logits, experts, top_k=2, shared=sh)
    M, D = x.shape
    xq, sx = O.quant_act_group(x)
    xd = O.dequant_act_group(xq, sx)
    deq = {n: O.dequant_weight_block(*experts[n]) for n in experts}
    dsh = {n: O.dequant_weight_block(*sh[n])[0] for n in sh}

    def mlp(xrow, wg, wu, wd):
        g = wg @ xrow; u = wu @ xrow
        h = (g / (1 + np.exp(-g)) * u).astype(np.float32)[None]
        hq, shh = O.quant_act_group(h)
        return O.bf16_round((wd @ O.dequant_act_group(hq, shh)[0]).astype(np.float32))

    for t in range(M):
        acc = np.zeros(D, np.float32)
        for s in range(2):
            e = res["indices"][t, s]
            acc = acc + mlp(xd[t], deq["gate"][e], deq["up"][e], deq["down"][e]) * res["weights"][t, s]
        acc = acc + mlp(xd[t], dsh["gate"], dsh["up"], dsh["down"])
        want = O.bf16_round(acc.astype(np.float32))
        assert np.allclose(res["out"][t], want, rtol=2e-2, atol=1e-3 * np.abs(want).max())
        # the bf16 grids agree except where an f32 rounding order moved a value across a tie
        assert np.mean(res["out"][t] != want) < 0.02
    rows = O.moe_experts_rows(x, [0, 5, 23], res["indices"], res["weights"],
                              lambda e: {n: (experts[n][0][e], experts[n][1][e]) for n in experts}, shared=sh)
    assert np.array_equal(rows, res["out"][[0, 5, 23]])


def test_combine_expert_relabel_invariance_and_special_cases():
    x, logits, experts, _ = _tiny_problem(seed=11, shared=False)
    base = O.moe_experts(x, logits, experts, top_k=2)
    perm = np.array([2, 0, 3, 1])                               # relabel experts: new id p holds old perm[p]
    ex2 = {n: (q[perm], s[perm]) for n, (q, s) in experts.items()}
    inv = np.argsort(perm)
    lg2 = logits[:, perm]
    res2 = O.moe_experts(x, lg2, ex2, top_k=2)
    assert np.array_equal(inv[base["indices"]], res2["indices"])      # the same experts under their new names, same order
    assert np.allclose(base["weights"], res2["weights"], rtol=1e-6, atol=0)   # (the softmax sums E terms in another order)
    assert np.allclose(base["out"], res2["out"], rtol=2.0 ** -7, atol=1e-6)   # at most one bf16 step apart
    # k = 1 with weight 1: output is exactly the selected expert's bf16 row
    r1 = O.moe_experts(x, logits, experts, top_k=1)
    assert np.allclose(r1["weights"], 1.0)
    assert np.array_equal(r1["out"], r1["y"][r1["inv_perm"]])
    # zero weights give exact zeros
    z = O.combine(base["y"], np.zeros_like(base["weights"]), base["inv_perm"])
    assert not z.any()


def test_swiglu_closed_form():
    v = np.linspace(-10, 10, 1001)
    assert np.allclose(O.silu(v), v * (1 / (1 + np.exp(-v))))
    assert O.silu(np.float64(0)) == 0


# ---------------------------------------------------------------- frozen fixture

def test_oracle_matches_committed_fixture_for_config1():
    """tests/golden/config1_oracle.npz (written by tests/golden/make_fixtures.py) freezes the oracle's results for
    benchmark config 1 (BASELINE.json); the GPU tests compare against the live oracle, this keeps the oracle itself from drifting."""
    import os
    from tests.golden import make_fixtures
    want = np.load(os.path.join(os.path.dirname(make_fixtures.__file__), "config1_oracle.npz"))
    got = make_fixtures.build()
    for name in want.files:
        assert np.array_equal(want[name], got[name]), name


# ---- router in front of the path --------------------------------------------------------------

def test_router_logits_exact_cases_and_python_loop():
    """Small integers: every partial sum is exact in f32, so any summation order (and any correct
    implementation) gives the same bits.  Then a Python-float loop on a tiny random case."""
    rng = H.rng_for(11)
    x = rng.integers(-4, 5, size=(6, 128)).astype(np.float32)
    w = rng.integers(-3, 4, size=(128, 5)).astype(np.float32)
    want = np.array([[sum(int(x[t, k]) * int(w[k, e]) for k in range(128)) for e in range(5)] for t in range(6)], np.float32)
    assert np.abs(want).max() < 256                       # representable in bf16
    assert np.array_equal(O.router_logits(x, w), want)
    # identity weights copy the activations (already bf16 values)
    xb = O.bf16_round(rng.standard_normal((4, 128), dtype=np.float32))
    assert np.array_equal(O.router_logits(xb, np.eye(128, dtype=np.float32)), xb)
    # transposed-operand mistake fails: (D, E) orientation matters
    wb = O.bf16_round(rng.standard_normal((128, 128), dtype=np.float32))
    assert not np.array_equal(O.router_logits(xb, wb), O.router_logits(xb, wb.T.copy()))
    got = O.router_logits(xb, wb)
    for t in range(2):
        for e in range(3):
            exact = sum(float(xb[t, k]) * float(wb[k, e]) for k in range(128))   # Python floats are f64
            assert got[t, e] == O.bf16_round(np.array([exact], np.float32))[0]


def test_shared_gate_values():
    x = np.zeros((3, 128), np.float32)
    w = np.ones((128, 1), np.float32)
    assert np.array_equal(O.shared_gate(x, w), np.full(3, 0.5, np.float32))            # sigmoid(0)
    x[1, :4] = 1.0                                                                      # logit 4
    g = O.shared_gate(x, w)
    assert abs(float(g[1]) - 1.0 / (1.0 + np.exp(-4.0))) < 2 ** -8                      # bf16 rounding of 0.982
    assert np.array_equal(g, O.bf16_round(g)) and g[0] == 0.5


def test_combine_gate_special_cases():
    rng = H.rng_for(12)
    M, k, D = 5, 2, 16
    y = O.bf16_round(rng.standard_normal((M * k, D), dtype=np.float32))
    sh = O.bf16_round(rng.standard_normal((M, D), dtype=np.float32))
    w = rng.random((M, k), dtype=np.float32)
    inv = rng.permutation(M * k).astype(np.int32)
    assert np.array_equal(O.combine(y, w, inv, sh, np.ones(M, np.float32)), O.combine(y, w, inv, sh))
    assert np.array_equal(O.combine(y, w, inv, sh, np.zeros(M, np.float32)), O.combine(y, w, inv))
    g = np.array([0.5, 0.25, 1.0, 0.0, 0.75], np.float32)
    want = np.stack([sum(np.float64(w[t, s]) * y[inv[t * k + s]] for s in range(k)) + np.float64(g[t]) * sh[t] for t in range(M)])
    assert np.abs(O.combine(y, w, inv, sh, g) - want).max() < 0.02


def test_rms_norm_closed_forms():
    """primitives.py:16-32.  A constant row c gives c / sqrt(c^2 + eps) * (1 + w); scaling the input leaves
    the output unchanged (up to eps); weight 0 gives unit mean square; and torch's f32 arithmetic agrees."""
    D = 256
    w = np.linspace(-0.5, 0.5, D).astype(np.float32)
    x = np.full((1, D), 3.0, np.float32)
    want = O.bf16_round((np.float32(3.0) / np.sqrt(np.float32(9.0) + np.float32(1e-6)) * (1 + w)).astype(np.float32))
    assert np.array_equal(O.rms_norm(x, w, 1e-6)[0], want)
    rng = H.rng_for(13)
    xr = O.bf16_round(rng.standard_normal((5, D), dtype=np.float32))
    a, b = O.rms_norm(xr, w, 1e-12), O.rms_norm(4 * xr, w, 1e-12)            # 4x is exact in bf16
    assert np.array_equal(a, b)
    n0 = O.rms_norm(xr, np.zeros(D, np.float32), 0.0)
    assert np.allclose(np.square(n0.astype(np.float64)).mean(-1), 1.0, atol=4e-3)
    xt = torch.from_numpy(xr)
    ref = (xt / torch.sqrt(xt.square().mean(-1, keepdim=True) + 1e-6) * (1 + torch.from_numpy(w))).to(torch.bfloat16).float().numpy()
    got = O.rms_norm(xr, w, 1e-6)
    assert float((got != ref).mean()) < 0.01 and np.abs(got - ref).max() <= 2.0 ** -6   # summation order only
    # a dropped "1 +" or a missing eps would fail these
    assert not np.array_equal(O.rms_norm(xr, w, 1e-6), O.rms_norm(xr, w - 1, 1e-6))
    assert np.isfinite(O.rms_norm(np.zeros((1, D), np.float32), w, 1e-6)).all()


def test_combine_residual():
    rng = H.rng_for(14)
    M, k, D = 4, 2, 8
    y = O.bf16_round(rng.standard_normal((M * k, D), dtype=np.float32))
    w = rng.random((M, k), dtype=np.float32)
    inv = rng.permutation(M * k).astype(np.int32)
    res = O.bf16_round(rng.standard_normal((M, D), dtype=np.float32))
    plain = O.combine(y, w, inv)
    assert np.array_equal(O.combine(y, w, inv, residual=np.zeros((M, D), np.float32)), plain)
    got = O.combine(y, w, inv, residual=res)
    want = np.stack([sum(np.float64(w[t, s]) * y[inv[t * k + s]] for s in range(k)) + res[t] for t in range(M)])
    assert np.abs(got - want).max() < 0.03


def test_continuing_from_given_intermediates_reproduces_the_path():
    """The h overrides (expert_swiglu / moe_experts / moe_experts_rows) are the second half of the same path: fed
    the path's own intermediates they give its own output, fed other codes they give another one."""
    x, logits, experts, shared = _tiny_problem(seed=21, shared=True)
    ref = O.moe_experts(x, logits, experts, top_k=2, shared=shared)
    again = O.moe_experts(x, logits, experts, top_k=2, shared=shared, routed_h=(ref["hq"], ref["sh"]), shared_h=(ref["hsq"], ref["shs"]))
    assert np.array_equal(again["out"], ref["out"]) and np.array_equal(again["y"], ref["y"])
    other = ref["hq"].copy()
    other[0, 0] ^= 0x08                                     # another exponent for one code
    changed = O.moe_experts(x, logits, experts, top_k=2, shared=shared, routed_h=(other, ref["sh"]), shared_h=(ref["hsq"], ref["shs"]))
    assert not np.array_equal(changed["y"][0], ref["y"][0]) and np.array_equal(changed["y"][1:], ref["y"][1:])
    # the per-row form agrees with the whole-problem form and hands back what it computed
    fetch = lambda e: {n: (q[e], s[e]) for n, (q, s) in experts.items()}
    toks = [0, 3, x.shape[0] - 1]
    rows = O.moe_experts_rows(x, toks, ref["indices"], ref["weights"], fetch, shared=shared, return_h=True)
    assert np.array_equal(rows["out"], ref["out"][toks])
    pos = ref["inv_perm"].reshape(-1, 2)[toks]
    assert np.array_equal(rows["routed_h"][0], ref["hq"][pos]) and np.array_equal(rows["y"], ref["y"][pos])
    assert np.array_equal(rows["ys"], ref["shared_out"][toks])
    cont = O.moe_experts_rows(x, toks, ref["indices"], ref["weights"], fetch, shared=shared, routed_h=rows["routed_h"],
                              shared_h=rows["shared_h"])
    assert np.array_equal(cont, ref["out"][toks])


def test_distance_to_the_reference_bf16_activation_dataflow(capsys):
    """The oracle quantises activations to 1x128 fp8 (x and h); the reference feeds bf16 activations to ragged_dot and
    accumulates the combine in bf16 (moe.py:83-94).  Parity with the reference itself is unpinned (JAX is not
    importable here); this reports how far the two arithmetics sit apart on one small layer, through the line-by-line
    port of the reference's dataflow, and bounds it by what two e4m3 quantisations explain."""
    from oracle import reference_dataflow as RD
    x, logits, experts, sh = _tiny_problem(seed=3, M=64, D=512, E=8, k=2, I=256)
    ours = O.moe_experts(x, logits, experts, top_k=2, shared=sh)["out"]
    ref = RD.moe_layer_reference(x, logits, experts, 2, shared=sh)
    err = np.abs(ours - ref)
    scale = np.abs(ref).max()
    rel_rows = np.linalg.norm(ours - ref, axis=1) / np.linalg.norm(ref, axis=1)
    with capsys.disabled():
        print(f"\n  fp8-activation oracle vs reference bf16-activation dataflow: max|d|/max|ref| = {err.max() / scale:.3e}, "
              f"row L2 error median {np.median(rel_rows):.3e} / worst {rel_rows.max():.3e}")
    # an e4m3 value carries 3 mantissa bits (relative step 2^-3 .. 2^-4, rounding error up to 2^-4); errors of
    # independent elements average down over the K-long dot products, so rows agree to a few percent
    assert err.max() / scale < 8e-2
    assert np.median(rel_rows) < 6e-2
