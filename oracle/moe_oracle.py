"""CPU oracle for the MoE expert forward path.  TEST INFRASTRUCTURE ONLY.

This module restates, in NumPy, the algorithm of jax-gpt's MoE layer
(reference: jax_gpt/models/qwen35/moe.py) extended with the block-scaled fp8
format and the DeepSeek-V3 group-limited router that the benchmark configs
name.  Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may
import it, and only as the checker; the product path never does.

What pins each function (tests/test_oracle.py holds the checks):

  e4m3_encode / e4m3_decode     exhaustive 256-code table + dense sweep against
                                torch's CPU float8_e4m3fn cast
  bf16 helpers                  against torch's CPU bfloat16 cast
  quant_weight_block / quant_act_group
                                scale == amax/448 to 1 ulp, round-trip bound,
                                block independence, all-zero blocks
  exp_det / sigmoid_det         against float64 exp (<= 2 ulp)
  route_softmax_topk            brute-force O(E^2) rank count, sum-to-one
                                (reference tests/qwen35/test_moe.py:52-60),
                                top-k of softmax == top-k of logits
  route_sigmoid_grouped         brute force per token in pure Python; the
                                n_group=1 / topk_group=n_group / bias=0
                                special cases that reduce to plain top-k
  sort_and_group                np.argsort(kind='stable') + np.bincount
                                equivalence, permutation invariants
  grouped_gemm                  per-expert dense float64 product on tiny
                                shapes; the scaled ones KAT of the reference
                                (tests/qwen35/test_fp8.py:65-75)
  combine                       per-token Python loop, expert-relabel
                                invariance, k=1 / zero-weight cases; gate = 1
                                equals no gate, gate = 0 drops the shared rows
  rms_norm                      constant rows (closed form), scale invariance,
                                unit mean square at weight 0, torch CPU f32
  router_logits / shared_gate   exact small-integer products (any summation
                                order gives the same value), Python-float
                                loops, identity weights; sigmoid(0) = 0.5

PARITY UNPINNED (nothing in the reference or in the mathematics fixes the
bits): the random streams of jax.random, XLA's bf16 rounding order inside
ragged_dot and scatter-add, XLA's accumulation order inside the router's bf16
matmul (router_logits takes the order-free value: exact sum, one rounding),
and the case of two distinct logits whose f32 softmax probabilities collide (this oracle ranks logits; the reference ranks
probabilities, moe.py:51-52).  The reference cannot be imported here (JAX is
not installed), and it holds no golden vectors for this path.
"""

from __future__ import annotations

import numpy as np

FP8_MAX = np.float32(448.0)          # reference fp8.py:26-27 (e4m3fn finfo.max)
BLOCK = 128                          # 128x128 weight blocks, 1x128 activation groups


# --------------------------------------------------------------------------
# bf16 and e4m3fn codecs (bit-level, so the oracle needs no dtype NumPy lacks)
# --------------------------------------------------------------------------

def f32_to_bf16_bits(x):
    """float32 -> bf16 bit pattern (uint16), round-to-nearest-even; NaN kept quiet."""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    rounded = (u + (np.uint32(0x7FFF) + ((u >> np.uint32(16)) & np.uint32(1)))) >> np.uint32(16)
    nan = (u & np.uint32(0x7FFFFFFF)) > np.uint32(0x7F800000)
    out = np.where(nan, (u >> np.uint32(16)) | np.uint32(0x40), rounded)
    return out.astype(np.uint16)


def bf16_bits_to_f32(b):
    return (np.ascontiguousarray(b, dtype=np.uint16).astype(np.uint32) << np.uint32(16)).view(np.float32)


def bf16_round(x):
    """Round a float32 array to the nearest bf16 value, returned as float32."""
    return bf16_bits_to_f32(f32_to_bf16_bits(x))


def _build_e4m3_table():
    t = np.zeros(256, dtype=np.float32)
    for code in range(256):
        s = -1.0 if code & 0x80 else 1.0
        e = (code >> 3) & 0xF
        m = code & 0x7
        if e == 0xF and m == 0x7:
            v = np.nan                               # the only NaN; e4m3fn has no inf
        elif e == 0:
            v = s * m * 2.0 ** -9                    # subnormals: m/8 * 2^-6
        else:
            v = s * (1.0 + m / 8.0) * 2.0 ** (e - 7)
        t[code] = v
    return t


E4M3_TABLE = _build_e4m3_table()


def e4m3_decode(codes):
    return E4M3_TABLE[np.asarray(codes, dtype=np.uint8)]


def e4m3_encode(x):
    """float32 -> e4m3fn code (uint8): round-to-nearest-even, saturating at +-448.

    The quantisers below clamp to +-448 first (as HF's block quantiser does), so
    saturation versus overflow-to-NaN never matters on this path.
    """
    x = np.asarray(x, dtype=np.float32)
    sign = (x.view(np.uint32) >> np.uint32(24)).astype(np.uint8) & np.uint8(0x80)
    a = np.minimum(np.abs(x), FP8_MAX).astype(np.float64)
    # subnormal range: multiples of 2^-9 below 2^-6
    sub = np.rint(a * 512.0)
    frac, exp = np.frexp(a)                          # a = frac * 2^exp, frac in [0.5,1)
    m = np.rint(frac * 16.0)                         # 8..16
    carry = m == 16.0
    m = np.where(carry, 8.0, m)
    e = exp - 1 + carry                              # unbiased exponent
    normal = ((e + 7).astype(np.int64) << 3) | (m.astype(np.int64) - 8)
    code = np.where(a < 2.0 ** -6, sub.astype(np.int64), normal)
    code = np.where(np.isnan(x), 0x7F, code)
    return (code.astype(np.uint8) | sign).astype(np.uint8)


# --------------------------------------------------------------------------
# quantisers: scale = 448/amax, q = rne(clamp(x*scale)), scale_inv = 1/scale
# (HF finegrained_fp8 block quantiser; activation groups use the same formula)
# --------------------------------------------------------------------------

def _scales_from_amax(amax):
    amax = amax.astype(np.float32)
    safe = np.where(amax > 0, amax, np.float32(1.0)).astype(np.float32)
    scale = (FP8_MAX / safe).astype(np.float32)
    scale = np.where(amax > 0, scale, np.float32(1.0)).astype(np.float32)
    scale_inv = (np.float32(1.0) / scale).astype(np.float32)
    return scale, scale_inv


def quant_weight_block(w):
    """(..., N, K) float32 -> (codes uint8 (..., N, K), scale_inv f32 (..., N/128, K/128)).

    Layout (..., out, in) follows the reference's fp8 expert layout
    (quantize.py:31-42, model.py:89-97); the scale granularity is 128x128.
    """
    w = np.asarray(w, dtype=np.float32)
    *lead, N, K = w.shape
    assert N % BLOCK == 0 and K % BLOCK == 0
    r = w.reshape(*lead, N // BLOCK, BLOCK, K // BLOCK, BLOCK)
    amax = np.abs(r).max(axis=(-3, -1))
    scale, scale_inv = _scales_from_amax(amax)
    scaled = (r * scale[..., :, None, :, None]).astype(np.float32)
    q = e4m3_encode(np.clip(scaled, -FP8_MAX, FP8_MAX)).reshape(w.shape)
    return q, scale_inv


def quant_act_group(x):
    """(R, K) float32 -> (codes uint8 (R, K), scale_inv f32 (R, K/128)); 1x128 groups."""
    x = np.asarray(x, dtype=np.float32)
    R, K = x.shape
    assert K % BLOCK == 0
    r = x.reshape(R, K // BLOCK, BLOCK)
    amax = np.abs(r).max(axis=-1)
    scale, scale_inv = _scales_from_amax(amax)
    scaled = (r * scale[..., None]).astype(np.float32)
    q = e4m3_encode(np.clip(scaled, -FP8_MAX, FP8_MAX)).reshape(R, K)
    return q, scale_inv


def dequant_weight_block(q, scale_inv):
    """w_real = w_fp8 * weight_scale_inv (the meaning the expert path uses, moe.py:29)."""
    w = e4m3_decode(q).astype(np.float64)
    s = np.repeat(np.repeat(scale_inv.astype(np.float64), BLOCK, axis=-2), BLOCK, axis=-1)
    return w * s


def dequant_act_group(q, scale_inv):
    x = e4m3_decode(q).astype(np.float64)
    return x * np.repeat(scale_inv.astype(np.float64), BLOCK, axis=-1)


# --------------------------------------------------------------------------
# deterministic exp / sigmoid: float32 mul/add/div only, no fused multiply-add,
# so a GPU kernel that issues the same operations gets the same bits.
# --------------------------------------------------------------------------

_LOG2E = np.float32(1.44269504088896341)
_LN2_HI = np.float32(0.693145751953125)        # 0x3f317200: n*LN2_HI exact for |n| < 2^15
_LN2_LO = np.float32(1.42860682030941723212e-6)
_EXP_C = [np.float32(c) for c in (1.9875691500e-4, 1.3981999507e-3, 8.3334519073e-3,
                                  4.1665795894e-2, 1.6666665459e-1, 5.0000001201e-1)]


def exp_det(x):
    """exp(x) for float32 x, <= 2 ulp, from a fixed sequence of rounded f32 operations."""
    f = np.float32
    x = np.clip(np.asarray(x, dtype=f), f(-87.0), f(88.0)).astype(f)
    n = np.rint((x * _LOG2E).astype(f)).astype(f)
    r = (x - (n * _LN2_HI).astype(f)).astype(f)
    r = (r - (n * _LN2_LO).astype(f)).astype(f)
    p = np.full_like(r, _EXP_C[0])
    for c in _EXP_C[1:]:
        p = ((p * r).astype(f) + c).astype(f)
    r2 = (r * r).astype(f)
    y = ((p * r2).astype(f) + r).astype(f)
    y = (y + f(1.0)).astype(f)
    two_n = ((n.astype(np.int32) + 127).astype(np.uint32) << np.uint32(23)).view(f)
    return (y * two_n).astype(f)


def sigmoid_det(x):
    f = np.float32
    x = np.asarray(x, dtype=f)
    return (f(1.0) / (f(1.0) + exp_det(-x)).astype(f)).astype(f)


# --------------------------------------------------------------------------
# routing
# --------------------------------------------------------------------------

def _topk_desc(values, k):
    """Indices of the k largest per row, value descending, ties -> lower index
    (lax.top_k's documented order, reference moe.py:52).  -0.0 ranks equal to +0.0."""
    order = np.argsort(-(values + np.float32(0.0)), axis=-1, kind="stable")
    return order[..., :k].astype(np.int32)


def route_softmax_topk(logits, k, renorm=True):
    """reference moe.py:37-55: softmax in f32, top-k, renormalise.

    Ranks the logits (softmax is monotone) -- see the module header for the
    collision corner this leaves unpinned."""
    f = np.float32
    logits = np.asarray(logits, dtype=f)
    idx = _topk_desc(logits, k)
    mx = logits.max(axis=-1, keepdims=True)
    e = exp_det((logits - mx).astype(f))
    denom = e.sum(axis=-1, keepdims=True, dtype=f)
    probs = (e / denom).astype(f)
    v = np.take_along_axis(probs, idx.astype(np.int64), axis=-1)
    if renorm:
        v = (v / v.sum(axis=-1, keepdims=True, dtype=f)).astype(f)
    return idx, v.astype(f)


def route_sigmoid_grouped(logits, bias, n_group, topk_group, k, renorm=True, routed_scale=1.0):
    """DeepSeek-V3 router (HF modeling_deepseek_v3.py DeepseekV3TopkRouter.forward):
    scores = sigmoid(logits); choice = scores + bias; group score = sum of the
    group's top-2 choice scores; keep the topk_group best groups; top-k experts
    among them by choice score; weights = un-biased scores, renormalised with
    +1e-20, times routed_scale.  Order fixed to value-descending, ties -> lower
    index (HF leaves it unsorted).

    Masking convention: experts of dropped groups take -inf before the final
    top-k, as DeepSeek's own inference code does (masked_fill_(..., -inf)); the
    HF port fills 0.0 instead, which differs only when a kept expert's biased
    score is negative (a dropped expert's 0.0 would then outrank it).  With
    -inf a dropped group never contributes an expert as long as the kept
    groups hold at least k experts."""
    f = np.float32
    logits = np.asarray(logits, dtype=f)
    M, E = logits.shape
    assert E % n_group == 0
    scores = sigmoid_det(logits)
    choice = (scores + (np.zeros(E, f) if bias is None else np.asarray(bias, f))[None, :]).astype(f)
    per = E // n_group
    g = choice.reshape(M, n_group, per)
    if per >= 2:
        top2 = np.take_along_axis(g, _topk_desc(g, 2).astype(np.int64), axis=-1)
        gscore = (top2[..., 0] + top2[..., 1]).astype(f)
    else:
        gscore = g[..., 0]
    gsel = _topk_desc(gscore, topk_group)
    gmask = np.zeros((M, n_group), dtype=bool)
    np.put_along_axis(gmask, gsel.astype(np.int64), True, axis=-1)
    masked = np.where(np.repeat(gmask, per, axis=-1), choice, f(-np.inf)).astype(f)
    idx = _topk_desc(masked, k)
    w = np.take_along_axis(scores, idx.astype(np.int64), axis=-1)
    if renorm:
        den = (w.sum(axis=-1, keepdims=True, dtype=f) + f(1e-20)).astype(f)
        w = (w / den).astype(f)
    w = (w * f(routed_scale)).astype(f)
    return idx, w


# --------------------------------------------------------------------------
# sort / group (reference moe.py:58-80)
# --------------------------------------------------------------------------

def sort_and_group(indices, n_experts):
    """Stable sort of the flat (token, slot) list by expert id.

    Returns dict with group_sizes (E,), group_offsets (E+1,), sort_order (R,)
    [flat index f = t*k+s at each sorted position], sorted_token_ids (R,),
    inv_perm (R,) [sorted position of flat index f]."""
    indices = np.asarray(indices, dtype=np.int32)
    M, k = indices.shape
    flat = indices.reshape(-1)
    sort_order = np.argsort(flat, kind="stable").astype(np.int32)          # moe.py:72
    flat_token_ids = np.repeat(np.arange(M, dtype=np.int32), k)            # moe.py:68
    sorted_token_ids = flat_token_ids[sort_order]                          # moe.py:73
    group_sizes = np.zeros(n_experts, dtype=np.int32)
    np.add.at(group_sizes, flat, 1)                                        # moe.py:76-77
    group_offsets = np.zeros(n_experts + 1, dtype=np.int32)
    group_offsets[1:] = np.cumsum(group_sizes)
    inv_perm = np.empty_like(sort_order)
    inv_perm[sort_order] = np.arange(sort_order.size, dtype=np.int32)
    return dict(group_sizes=group_sizes, group_offsets=group_offsets, sort_order=sort_order,
                sorted_token_ids=sorted_token_ids, inv_perm=inv_perm)


# --------------------------------------------------------------------------
# grouped GEMMs (ragged_dot semantics, reference moe.py:83-87) on fp8 operands
# --------------------------------------------------------------------------

def grouped_gemm(xq, sx, wq, sw, group_offsets, dtype=np.float64):
    """rows [off_e, off_e+1) of x times expert e's (N,K) weight, transposed.

    xq (R,K) codes, sx (R,K/128); wq (E,N,K) codes, sw (E,N/128,K/128).
    Returns (R,N) in `dtype` -- float64 is the exact-arithmetic statement,
    float32 (BLAS) is for the big shapes."""
    R, K = xq.shape
    E, N, _ = wq.shape
    out = np.zeros((R, N), dtype=dtype)
    for e in range(E):
        a, b = int(group_offsets[e]), int(group_offsets[e + 1])
        if b <= a:
            continue
        xe = dequant_act_group(xq[a:b], sx[a:b]).astype(dtype)
        we = dequant_weight_block(wq[e], sw[e]).astype(dtype)
        out[a:b] = xe @ we.T
    return out


def silu(x):
    x = np.asarray(x)
    return x / (1.0 + np.exp(-x))


def expert_swiglu(xq, sx, experts, group_offsets, dtype=np.float64, h=None):
    """gate/up grouped GEMM -> silu(g)*u in f32 -> 1x128 fp8 quant -> down grouped GEMM.

    `experts` = dict(gate=(codes, scale_inv), up=..., down=...).  Returns
    (y f32 (R,D), hq, sh) where y is rounded once to bf16-representable f32.
    `h` = (codes, scale_inv) takes the place of the quantised intermediate: the second half of the path alone,
    continued from an intermediate computed elsewhere (the tests pass the kernel's own, so that the comparison of
    the outputs is not blurred by intermediate values that sit on an fp8 rounding boundary)."""
    if h is None:
        g = grouped_gemm(xq, sx, *experts["gate"], group_offsets, dtype=dtype)
        u = grouped_gemm(xq, sx, *experts["up"], group_offsets, dtype=dtype)
        hq, sh = quant_act_group((silu(g) * u).astype(np.float32))
    else:
        hq, sh = np.asarray(h[0], np.uint8), np.asarray(h[1], np.float32)
    y = grouped_gemm(hq, sh, *experts["down"], group_offsets, dtype=dtype)
    return bf16_round(y.astype(np.float32)), hq, sh


def combine(y, weights, inv_perm, shared=None, shared_gate=None, residual=None):
    """out[t] = sum_s w[t,s] * y[inv_perm[t*k+s]] (+ shared_gate[t] * shared[t]); f32 sum in
    slot order, one bf16 rounding (reference moe.py:90-94 accumulates in bf16 and moe.py:279
    rounds the gated shared rows to bf16 before the add of :281; this path keeps f32 until the end)."""
    M, k = weights.shape
    acc = np.zeros((M, y.shape[1]), dtype=np.float32)
    pos = inv_perm.reshape(M, k)
    for s in range(k):
        acc = (acc + (y[pos[:, s]].astype(np.float32) * weights[:, s:s + 1].astype(np.float32))).astype(np.float32)
    if shared is not None:
        sh = shared.astype(np.float32)
        if shared_gate is not None:
            sh = (sh * shared_gate.astype(np.float32)[:, None]).astype(np.float32)
        acc = (acc + sh).astype(np.float32)
    if residual is not None:                 # block.py:58: x + moe_out, here inside the one rounding
        acc = (acc + residual.astype(np.float32)).astype(np.float32)
    return bf16_round(acc)


def rms_norm(x, weight, eps=1e-6):
    """primitives.py:16-32: x / sqrt(mean(x^2) + eps) * (1 + weight) in f32, cast to the input's dtype (bf16
    here).  The mean is taken in float64 and rounded once (order-free, as router_logits does)."""
    x32 = np.asarray(x, np.float32)
    ms = (np.square(x32.astype(np.float64)).mean(axis=-1, keepdims=True)).astype(np.float32)
    rms = np.sqrt(ms + np.float32(eps)).astype(np.float32)
    normed = (x32 / rms).astype(np.float32)
    return bf16_round((normed * (np.float32(1.0) + np.asarray(weight, np.float32))).astype(np.float32))


# --------------------------------------------------------------------------
# router in front of the path (moe.py:50 and :278)
# --------------------------------------------------------------------------

def router_logits(x, gate_weight):
    """moe.py:50-51: logits = (x @ gate_weight) as a bf16 matmul result, widened to f32.
    x (M, D) and gate_weight (D, E) hold bf16-representable values.  The sum is taken in
    float64 (every product of two bf16 values is exact there) and rounded once to f32,
    then to bf16: the value an f32-accumulating matmul approaches, free of any summation
    order.  A hardware matmul differs from it by its f32 accumulation error, which shows
    after the bf16 rounding only for sums that sit on a rounding boundary."""
    acc = np.asarray(x, np.float64) @ np.asarray(gate_weight, np.float64)
    return bf16_round(acc.astype(np.float32))


def shared_gate(x, shared_expert_gate_weight):
    """moe.py:278: sigmoid(x @ shared_expert_gate_weight), a bf16 value per token; (M,) f32."""
    z = router_logits(x, shared_expert_gate_weight)[:, 0]
    return bf16_round(sigmoid_det(z))


def moe_sublayer(x, moe_norm_weight, params, top_k, eps=1e-6, dtype=np.float64, routed_h=None, shared_h=None):
    """block.py:54-58: x + moe_layer(rms_norm(x, moe_norm), params) on (M, D) rows."""
    normed = rms_norm(x, moe_norm_weight, eps)
    r = moe_layer(normed, params, top_k, dtype=dtype, residual=x, routed_h=routed_h, shared_h=shared_h)
    r["normed"] = normed
    return r


def moe_layer(x, params, top_k, dtype=np.float64, residual=None, routed_h=None, shared_h=None):
    """moe.py:235-282 on (M, D) rows: softmax routing on the router's own logits, routed experts,
    shared expert scaled by its sigmoid gate, one add.  params: gate_weight (D, E); experts / shared
    dicts as in moe_experts; shared_expert_gate_weight (D, 1) or absent."""
    logits = router_logits(x, params["gate_weight"])
    r = moe_experts(x, logits, params["experts"], top_k=top_k, routing="softmax", shared=params.get("shared"),
                    shared_gate_values=(shared_gate(x, params["shared_expert_gate_weight"])
                                        if params.get("shared_expert_gate_weight") is not None else None),
                    residual=residual, dtype=dtype, routed_h=routed_h, shared_h=shared_h)
    r["logits"] = logits
    return r


# --------------------------------------------------------------------------
# the whole path: router logits in, combined hidden states out
# --------------------------------------------------------------------------

def moe_experts(x, router_logits, experts, *, top_k, routing="softmax", bias=None, n_group=1,
                topk_group=1, renorm=True, routed_scale=1.0, shared=None, shared_gate_values=None,
                residual=None, dtype=np.float64, routed_h=None, shared_h=None):
    """x: (M,D) float32 holding bf16-representable values.  experts/shared: dicts
    gate/up/down -> (codes, scale_inv) with expert weights (E,N,K) and shared (1,N,K).
    routed_h / shared_h = (codes, scale_inv): continue from these quantised intermediates (rows in sorted
    order / token order) instead of computing them (see expert_swiglu)."""
    E = experts["gate"][0].shape[0]
    if routing == "softmax":
        idx, w = route_softmax_topk(router_logits, top_k, renorm)
    elif routing == "sigmoid_grouped":
        idx, w = route_sigmoid_grouped(router_logits, bias, n_group, topk_group, top_k, renorm, routed_scale)
    else:
        raise ValueError(routing)
    sg = sort_and_group(idx, E)
    xq, sx = quant_act_group(x)
    xs, sxs = xq[sg["sorted_token_ids"]], sx[sg["sorted_token_ids"]]        # moe.py:79
    y, hq, sh = expert_swiglu(xs, sxs, experts, sg["group_offsets"], dtype=dtype, h=routed_h)
    ys = hsq = shs = None
    if shared is not None:
        M = x.shape[0]
        ys, hsq, shs = expert_swiglu(xq, sx, shared, np.array([0, M], dtype=np.int32), dtype=dtype, h=shared_h)
    out = combine(y, w, sg["inv_perm"], ys, shared_gate_values, residual)
    return dict(out=out, indices=idx, weights=w, xq=xq, sx=sx, y=y, hq=hq, sh=sh, shared_out=ys, hsq=hsq, shs=shs, **sg)


def moe_experts_rows(x, tokens, indices, weights, fetch_expert, shared=None, dtype=np.float64, shared_gate_values=None,
                     residual=None, routed_h=None, shared_h=None, return_h=False):
    """The same mathematics for a handful of token rows at full problem size:
    `fetch_expert(e)` returns dict gate/up/down -> (codes (N,K), scale_inv) for
    expert e.  shared_gate_values (M,) and residual (M, D) as in combine.
    routed_h = (codes (len(tokens), k, I), scale_inv (len(tokens), k, I/128)) and shared_h = (codes (len(tokens), SI),
    scale_inv) continue from given intermediates (see expert_swiglu).
    Returns (len(tokens), D) f32 (bf16-representable); with return_h a dict: out, the intermediates this function
    computed or was given (routed_h, shared_h, in the layout of the arguments) and the bf16 rows the combine summed
    (y (len(tokens), k, D), ys (len(tokens), D) or None)."""
    outs, hs, hss, yrows, ysrows = [], [], [], [], []
    for ti, t in enumerate(tokens):
        xq, sx = quant_act_group(x[t:t + 1])
        acc = np.zeros((1, x.shape[1]), dtype=np.float32)
        off = np.array([0, 1], dtype=np.int32)
        row_h = []
        for s in range(indices.shape[1]):
            ex = fetch_expert(int(indices[t, s]))
            ex = {n: (q[None], sc[None]) for n, (q, sc) in ex.items()}
            hin = None if routed_h is None else (routed_h[0][ti, s][None], routed_h[1][ti, s][None])
            y, hq1, sh1 = expert_swiglu(xq, sx, ex, off, dtype=dtype, h=hin)
            row_h.append((hq1[0], sh1[0], y[0]))
            acc = (acc + y * np.float32(weights[t, s])).astype(np.float32)
        hs.append(row_h)
        if shared is not None:
            hin = None if shared_h is None else (shared_h[0][ti][None], shared_h[1][ti][None])
            ys, hq1, sh1 = expert_swiglu(xq, sx, shared, off, dtype=dtype, h=hin)
            hss.append((hq1[0], sh1[0]))
            ysrows.append(ys[0])
            if shared_gate_values is not None:
                ys = (ys * np.float32(shared_gate_values[t])).astype(np.float32)
            acc = (acc + ys).astype(np.float32)
        if residual is not None:
            acc = (acc + residual[t:t + 1].astype(np.float32)).astype(np.float32)
        outs.append(bf16_round(acc)[0])
    if not return_h:
        return np.stack(outs)
    rh = (np.stack([np.stack([q for q, _, _ in r]) for r in hs]), np.stack([np.stack([sc for _, sc, _ in r]) for r in hs]))
    sh_ = (np.stack([q for q, _ in hss]), np.stack([sc for _, sc in hss])) if hss else None
    return dict(out=np.stack(outs), routed_h=rh, shared_h=sh_, y=np.stack([np.stack([yy for _, _, yy in r]) for r in hs]),
                ys=np.stack(ysrows) if ysrows else None)
