/*
 * moe_hip.h -- C ABI of libmoe_hip.so: the MoE expert forward path of
 * jax-gpt's Qwen3.5 / DeepSeek-V3-style MoE layer as hand-written HIP kernels
 * for gfx950 (MI355X).
 *
 * Every entry point is enqueue-only on the caller's stream: no device
 * synchronisation, no host read-back, no allocation.  The caller owns every
 * buffer, including the workspace (size from moe_workspace_bytes).  Inputs are
 * read-only, outputs are fully overwritten.  Return value 0 = ok, < 0 = one of
 * MOE_ERR_*; moe_last_error() gives the thread-local message.
 *
 * Layouts (all row-major, device pointers, 16-byte aligned):
 *   logits   (M, E)  f32          router logits
 *   idx      (M, k)  int32        selected experts, value-descending, ties -> lower index
 *   w        (M, k)  f32          routing weights
 *   x        (M, D)  bf16         hidden states
 *   xq / sx  (R, K) e4m3fn / (R, K/128) f32     activations, 1x128 scale groups
 *   wq / sw  (E, N, K) e4m3fn / (E, N/128, K/128) f32   weights, K contiguous,
 *            128x128 scale blocks; real value = code * scale  ("weight_scale_inv")
 *   flat index f = t*k + s; sorted position p; R = M*k
 *
 * Reference citations are to ultrons/jax-gpt, jax_gpt/models/qwen35/.
 */
#ifndef MOE_HIP_H
#define MOE_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* The library is built with hidden visibility: only what this header declares is exported. */
#if defined(__GNUC__) || defined(__clang__)
#define MOE_API __attribute__((visibility("default")))
#else
#define MOE_API
#endif

#define MOE_OK 0
#define MOE_ERR_BAD_SHAPE (-1)
#define MOE_ERR_BAD_ALIGN (-2)
#define MOE_ERR_WORKSPACE_TOO_SMALL (-3)
#define MOE_ERR_HIP (-4)
#define MOE_ERR_NULL (-5)

#define MOE_ROUTING_SOFTMAX 0          /* moe.py:37-55 */
#define MOE_ROUTING_SIGMOID_GROUPED 1  /* DeepSeek-V3 group-limited router (not in the reference) */

typedef void* moe_stream_t; /* a hipStream_t */

MOE_API int moe_abi_version(void);
MOE_API const char* moe_last_error(void);

/* moe.py:51-53 (softmax in f32, lax.top_k, renormalise).  E <= 1024, k <= 32, k <= E. */
MOE_API int moe_route_softmax_topk(const float* logits, int M, int E, int k, int renorm,
                           int32_t* idx, float* w, moe_stream_t stream);

/* DeepSeek-V3 router: sigmoid scores, +bias for selection only, group score = sum of
 * the group's top-2, keep topk_group groups, top-k among them, weights = un-biased
 * scores (renormalised with +1e-20) * routed_scale.  Replaces moe.py:37-55 for the
 * DeepSeek-shaped configs.  bias may be NULL.  E <= 1024, n_group <= 64. */
MOE_API int moe_route_sigmoid_grouped(const float* logits, const float* bias, int M, int E, int n_group,
                              int topk_group, int k, int renorm, float routed_scale,
                              int32_t* idx, float* w, moe_stream_t stream);

/* moe.py:58-80 (_sort_and_group): stable counting sort of the flat (token, slot)
 * list by expert id.  Outputs group_sizes (E), group_offsets (E+1), sorted_token_ids
 * (R), sort_order (R), inv_perm (R); any of the last three may be NULL. */
MOE_API size_t moe_permute_workspace_bytes(int M, int k, int E);
MOE_API int moe_permute(const int32_t* idx, int M, int k, int E, int32_t* group_sizes,
                int32_t* group_offsets, int32_t* sorted_token_ids, int32_t* sort_order,
                int32_t* inv_perm, void* ws, size_t ws_bytes, moe_stream_t stream);

/* 1x128 activation quantiser (replaces fp8.py:30-45's per-row quantiser):
 * scale = 448/amax, q = e4m3(clamp(x*scale)), sx = 1/scale.  K % 128 == 0. */
MOE_API int moe_quant_act(const void* x_bf16, int R, int K, uint8_t* xq, float* sx, moe_stream_t stream);

/* 128x128 weight block quantiser (replaces quantize.py:18-42's per-row quantiser;
 * layout (E, out, in) as quantize.py:31-35).  src_is_f32: 0 = bf16 source, 1 = f32. */
MOE_API int moe_quant_weight_block(const void* w, int src_is_f32, int E, int N, int K, uint8_t* wq,
                           float* sw, moe_stream_t stream);

/* moe.py:85-86 + silu*mul of :87, fused: for rows [group_offsets[e], group_offsets[e+1])
 * h = silu(x . Wgate[e]^T) * (x . Wup[e]^T), then 1x128 fp8 quantisation of h.
 * row_ids (R) maps sorted position -> row of xq/sx (the gather of moe.py:79 without
 * materialising x_sorted); NULL = identity (pre-dispatched rows).  D, I % 128 == 0. */
MOE_API size_t moe_gemm_workspace_bytes(int R, int E, int N_out);
MOE_API int moe_gemm_gateup_swiglu_fp8(const uint8_t* xq, const float* sx, const int32_t* row_ids,
                               const uint8_t* w_gate, const float* sw_gate,
                               const uint8_t* w_up, const float* sw_up,
                               const int32_t* group_offsets, int E, int R, int D, int I,
                               uint8_t* hq, float* sh, void* ws, size_t ws_bytes,
                               moe_stream_t stream);

/* The same gate/up GEMM for callers that cannot allocate device memory or carry a workspace (code under HIP
 * graph capture, tight serving loops, harnesses that forbid hipMalloc).  No counterpart in the reference.
 * The list of row tiles that the kernels read lives in a static device array of MOE_STATIC_SCRATCH_BYTES inside
 * the library (one copy per GPU, held until the process ends); the call allocates nothing and fails with
 * MOE_ERR_WORKSPACE_TOO_SMALL when moe_gemm_workspace_bytes(R, E, I) exceeds that size.  All calls on one GPU
 * share the array: calls that overlap in time on one GPU (two streams, two threads) race; calls on one stream
 * are ordered and safe.  Results are identical to moe_gemm_gateup_swiglu_fp8. */
#define MOE_STATIC_SCRATCH_BYTES (1u << 20)
MOE_API int moe_gemm_gateup_swiglu_fp8_static(const uint8_t* xq, const float* sx, const int32_t* row_ids,
                                      const uint8_t* w_gate, const float* sw_gate,
                                      const uint8_t* w_up, const float* sw_up,
                                      const int32_t* group_offsets, int E, int R, int D, int I,
                                      uint8_t* hq, float* sh, moe_stream_t stream);

/* Scale layouts of the grouped GEMMs' activation operands (no counterpart in the reference, which has no
 * activation scales).  ROW_MAJOR is what the quantisers write: (rows, K/128), indexed through row_ids like the
 * codes.  BLOCK_MAJOR is (K/128, R) in row-list order (entry [kb][p] belongs to list position p; row_ids is not
 * applied to it): a K step of a 256-row tile then reads its row scales from 8 cache lines instead of 256, which
 * is worth 2-3 % of the GEMM time at prefill sizes.  moe_gather_scales makes the block-major array from the
 * row-major one; moe_forward does this by itself for batches of more than 2048 routed rows. */
#define MOE_SCALES_ROW_MAJOR 0
#define MOE_SCALES_BLOCK_MAJOR 1
MOE_API int moe_gather_scales(const float* sx, const int32_t* row_ids, int R, int KB, float* out,
                              moe_stream_t stream);
/* moe_gemm_gateup_swiglu_fp8 with the layout of sx (read) and of sh (written) chosen by the caller. */
MOE_API int moe_gemm_gateup_swiglu_fp8_layout(const uint8_t* xq, const float* sx, const int32_t* row_ids,
                                      const uint8_t* w_gate, const float* sw_gate,
                                      const uint8_t* w_up, const float* sw_up,
                                      const int32_t* group_offsets, int E, int R, int D, int I,
                                      uint8_t* hq, float* sh, void* ws, size_t ws_bytes,
                                      int sx_layout, int sh_layout, moe_stream_t stream);

/* moe.py:87 (the third ragged_dot): y = h . Wdown[e]^T, bf16 out (R, D). */
MOE_API int moe_gemm_down_fp8(const uint8_t* hq, const float* sh, const uint8_t* w_down,
                      const float* sw_down, const int32_t* group_offsets, int E, int R, int I,
                      int D, void* y_bf16, void* ws, size_t ws_bytes, moe_stream_t stream);
/* The same with sh in the given layout (MOE_SCALES_*). */
MOE_API int moe_gemm_down_fp8_layout(const uint8_t* hq, const float* sh, const uint8_t* w_down,
                      const float* sw_down, const int32_t* group_offsets, int E, int R, int I,
                      int D, void* y_bf16, void* ws, size_t ws_bytes, int sh_layout, moe_stream_t stream);

/* moe.py:90-94 (_scatter_back) as a deterministic gather: out[t] = sum_s w[t,s] *
 * y[inv_perm[t*k+s]] (+ shared_gate[t] * shared[t]) in f32, one bf16 rounding.  shared may be
 * NULL (moe.py:281 adds the shared expert's output); shared_gate may be NULL (= 1; moe.py:278-279
 * multiplies the shared expert's output by sigmoid(x @ shared_expert_gate_weight)); residual
 * (M, D) bf16 or NULL is the layer's input added last (x = x + moe_out, block.py:58 and :91). */
MOE_API int moe_combine(const void* y_bf16, const float* w, const int32_t* inv_perm,
                const void* shared_bf16, const float* shared_gate, const void* residual_bf16, int M, int k,
                int D, void* out_bf16, moe_stream_t stream);

/* moe.py:50 (logits = matmul_maybe_fp8(x, gate_weight), a bf16 matmul widened to f32 by :51) and
 * moe.py:278 (sigmoid(x @ shared_expert_gate_weight)).  w_router is (E, D) bf16, K-contiguous (the
 * checkpoint layout of mlp.gate.weight; the reference's in-memory array is its transpose (D, E));
 * w_shared_gate is (1, D) bf16 or NULL.  logits (M, E) f32 hold bf16-rounded values; shared_gate
 * (M) f32 holds bf16-rounded sigmoids (NULL iff w_shared_gate is NULL). */
MOE_API size_t moe_router_workspace_bytes(int M, int D, int E);
MOE_API int moe_router_logits(const void* x_bf16, int M, int D, const void* w_router_bf16, int E,
                      const void* w_shared_gate_bf16, float* logits, float* shared_gate, void* ws,
                      size_t ws_bytes, moe_stream_t stream);

/* primitives.py:16-32 (rms_norm, Qwen3.5 convention: x / sqrt(mean(x^2) + eps) * (1 + weight), result in
 * bf16) as called in front of the MoE layer (block.py:54, :88), fused with the 1x128 quantisation of the
 * normalised row.  weight (D) f32; normed_bf16 (M, D) may be NULL when only the fp8 form is needed.
 * D <= 8192. */
MOE_API int moe_rmsnorm_quant(const void* x_bf16, const float* weight, float eps, int M, int D, void* normed_bf16,
                      uint8_t* xq, float* sx, moe_stream_t stream);

/* moe.py:282 (`.astype(x.dtype)`) and the widening in front of the layer: elementwise f32 <-> bf16 conversion of n
 * values (round-to-nearest-even towards bf16), so that a caller holding f32 activations needs no other library. */
MOE_API int moe_convert(const void* src, int src_is_f32, void* dst, int dst_is_f32, long long n, moe_stream_t stream);

/* The whole path (moe.py:97-114 + 225-232 + 281): router logits in, combined hidden
 * states out -- or, with w_router set, hidden states in (moe.py:235-282, moe_layer). */
typedef struct MoeForwardArgs {
  int M, D, E, k, I;       /* tokens, hidden, routed experts, top-k, expert intermediate */
  int SI;                  /* shared-expert intermediate, 0 = no shared expert */
  int routing;             /* MOE_ROUTING_* */
  int n_group, topk_group; /* sigmoid_grouped only */
  int renorm;
  float routed_scale;
  const void* x;           /* (M, D) bf16 */
  const float* logits;     /* (M, E); ignored (may be NULL) when w_router is set */
  const float* bias;       /* (E) or NULL */
  const uint8_t *w_gate, *w_up, *w_down;    /* (E,I,D) (E,I,D) (E,D,I) */
  const float *sw_gate, *sw_up, *sw_down;
  const uint8_t *ws_gate, *ws_up, *ws_down; /* shared expert (1,SI,D) (1,SI,D) (1,D,SI) or NULL */
  const float *sws_gate, *sws_up, *sws_down;
  void* out;               /* (M, D) bf16 */
  /* optional debug outputs (NULL to skip): the integer results the parity tests check */
  int32_t* out_idx;        /* (M, k) */
  float* out_w;            /* (M, k) */
  int32_t* out_group_sizes;      /* (E) */
  int32_t* out_sorted_token_ids; /* (R) */
  int32_t* out_inv_perm;         /* (R) */
  uint8_t* out_hq;               /* (R, I) e4m3 codes of the SwiGLU output, rows in sorted order */
  float* out_sh;                 /* (R, I/128) their 1x128 scales */
  uint8_t* out_hsq;              /* (M, SI) the same for the shared expert (needs SI > 0) */
  float* out_shs;                /* (M, SI/128) */
  void* out_y;                   /* (R, D) bf16 rows of the down GEMM, sorted order (what the combine gathers) */
  void* out_ys;                  /* (M, D) bf16 rows of the shared expert's down GEMM (needs SI > 0) */
  /* router in front of the path (NULL = the caller supplies logits) */
  const void* w_router;          /* (E, D) bf16: logits = bf16(x . w_router^T), moe.py:50 */
  const void* w_shared_gate;     /* (1, D) bf16 or NULL: shared expert's output is scaled by
                                    sigmoid(x . w_shared_gate^T), moe.py:278-279; needs w_router and SI > 0 */
  float* out_logits;             /* (M, E) optional copy of the logits the router computed (else never stored) */
  float* out_shared_gate;        /* (M) optional copy of the shared expert's gate values (needs w_shared_gate) */
  /* the steps either side of the layer (block.py:54-58, :88-91); NULL / 0 = off */
  const float* norm_weight;      /* (D) f32: x is RMS-normalised first (rms_norm with 1 + weight, in bf16) */
  float norm_eps;
  int add_residual;              /* out = x + moe_out, added in f32 before the one bf16 rounding */
} MoeForwardArgs;

/* Host-side objects moe_forward creates.  No device memory is ever allocated.  With a shared expert (SI > 0) the
 * call (a) creates, on the first such call on a device, ONE side stream for that device (default priority, kept until
 * the process ends, shared by every caller stream and host thread) and (b) creates two or three hipEvents per call and
 * destroys them before returning (quantised activations ready, shared expert done, and for large batches a fork
 * at the call's start), so that calls on different streams share no event state.  Consequences: if the caller's
 * stream is being captured into a HIP graph, the side stream joins that capture through the first of these events
 * for the length of the call; a second host thread that makes an
 * eager moe_forward call on the same device while another thread is inside a capturing call would enqueue onto a
 * capturing stream -- that combination is unsupported (serialise such calls, or capture on one thread only).  Without
 * a shared expert no stream or event is created. */
MOE_API size_t moe_forward_workspace_bytes(int M, int D, int E, int k, int I, int SI);
MOE_API int moe_forward(const MoeForwardArgs* args, void* ws, size_t ws_bytes, moe_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* MOE_HIP_H */
