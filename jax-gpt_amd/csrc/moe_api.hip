// Error reporting and the whole-path entry point of the C ABI.
//
// moe_forward = jax_gpt/models/qwen35/moe.py:97-114 (expert_forward_single) fed by
// router logits, plus the shared expert of moe.py:225-232 and the add of :281.
#include <stdarg.h>
#include <stdio.h>

#include <mutex>

#include "moe_common.h"

static thread_local char g_err[512] = "";

int moe_set_error(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

int moe_check_hip(hipError_t e, const char* what) {
  if (e == hipSuccess) return MOE_OK;
  return moe_set_error(MOE_ERR_HIP, "%s: %s", what, hipGetErrorString(e));
}

extern "C" int moe_abi_version(void) { return 6; }
extern "C" const char* moe_last_error(void) { return g_err; }

namespace {

// One side stream per device, default priority, created on first use and kept for the life of the process.
int side_stream(hipStream_t* out) {
  static std::mutex mu;
  static hipStream_t streams[64] = {};
  int dev = 0;
  int rc = moe_check_hip(hipGetDevice(&dev), "forward: hipGetDevice");
  if (rc) return rc;
  if (dev < 0 || dev >= 64) return moe_set_error(MOE_ERR_HIP, "forward: device index %d out of range", dev);
  std::lock_guard<std::mutex> lock(mu);
  if (!streams[dev]) {
    if ((rc = moe_check_hip(hipStreamCreateWithFlags(&streams[dev], hipStreamNonBlocking), "forward: side stream")))
      return rc;
  }
  *out = streams[dev];
  return MOE_OK;
}

// The events of a call with a shared expert (fork, activations quantised, join), kept per host thread and device
// and created on first use: a call enqueues and returns on one thread, and a wait that is already enqueued keeps
// the record it was enqueued after, so the thread's next call may record the same events again (calls of other
// threads have their own).  They are never destroyed: the runtime may be gone by the time a thread ends.
struct CallEvents {
  hipEvent_t fork, quant, join;
};
int call_events(CallEvents** out) {
  static thread_local CallEvents events[64] = {};
  int dev = 0;
  int rc = moe_check_hip(hipGetDevice(&dev), "forward: hipGetDevice");
  if (rc) return rc;
  if (dev < 0 || dev >= 64) return moe_set_error(MOE_ERR_HIP, "forward: device index %d out of range", dev);
  CallEvents& ev = events[dev];
  if (!ev.join) {
    hipEvent_t made[3] = {};
    for (int i = 0; i < 3; ++i) {
      const hipError_t e = hipEventCreateWithFlags(&made[i], hipEventDisableTiming);
      if (e != hipSuccess) {
        for (int j = 0; j < i; ++j) (void)hipEventDestroy(made[j]);
        return moe_check_hip(e, "forward: creating the fork/join events");
      }
    }
    ev = CallEvents{made[0], made[1], made[2]};
  }
  *out = &ev;
  return MOE_OK;
}

struct Carver {
  char* base;
  size_t used;
  void* take(size_t bytes) {
    void* p = base ? base + used : nullptr;
    used += (bytes + 255) & ~(size_t)255;
    return p;
  }
};

struct ForwardBuffers {
  int32_t *idx, *group_sizes, *group_offsets, *sorted_token_ids, *inv_perm, *dense_off;
  float *w, *sx, *sh, *shs, *shared_gate, *sx_listed, *sx_blocked;
  uint8_t *xq, *hq, *hsq;
  void *y, *ys, *permute_ws, *gemm_ws, *gemm_ws_shared, *router_ws, *normed;
  size_t permute_ws_bytes, gemm_ws_bytes, gemm_ws_shared_bytes, router_ws_bytes, total;
};

ForwardBuffers carve(void* ws, int M, int D, int E, int k, int I, int SI, bool router) {
  ForwardBuffers b;
  Carver c{(char*)ws, 0};
  const size_t R = (size_t)M * k;
  b.idx = (int32_t*)c.take(R * 4);
  b.w = (float*)c.take(R * 4);
  b.group_sizes = (int32_t*)c.take((size_t)E * 4);
  b.group_offsets = (int32_t*)c.take((size_t)(E + 1) * 4);
  b.sorted_token_ids = (int32_t*)c.take(R * 4);
  b.inv_perm = (int32_t*)c.take(R * 4);
  b.dense_off = (int32_t*)c.take(8);   // (stands in for the shared expert's group offsets, which its pre-built tile list makes unread)
  b.permute_ws_bytes = moe_permute_workspace_bytes(M, k, E);
  b.permute_ws = c.take(b.permute_ws_bytes);
  b.gemm_ws_bytes = moe_gemm_workspace_bytes((int)R, E, I > D ? I : D);
  b.gemm_ws = c.take(b.gemm_ws_bytes);        // tile list of the routed GEMMs (gate/up and down share it)
  // the shared expert runs beside the routed ones on its own stream: its launches need their own work lists
  b.gemm_ws_shared_bytes = SI ? moe_gemm_workspace_bytes(M, 1, SI > D ? SI : D) : 0;
  b.gemm_ws_shared = SI ? c.take(b.gemm_ws_shared_bytes) : nullptr;
  b.xq = (uint8_t*)c.take((size_t)M * D);
  b.sx = (float*)c.take((size_t)M * (D / 128) * 4);
  // block-major copies of the activation scales for large batches (GemmScales): routed rows in sorted order,
  // and the tokens in their own order for the shared expert
  b.sx_listed = (float*)c.take(R * (D / 128) * 4);
  b.sx_blocked = SI ? (float*)c.take((size_t)M * (D / 128) * 4) : nullptr;
  b.hq = (uint8_t*)c.take(R * I);
  b.sh = (float*)c.take(R * (I / 128) * 4);
  b.y = c.take(R * D * 2);
  b.hsq = SI ? (uint8_t*)c.take((size_t)M * SI) : nullptr;
  b.shs = SI ? (float*)c.take((size_t)M * (SI / 128) * 4) : nullptr;
  b.ys = SI ? c.take((size_t)M * D * 2) : nullptr;
  b.shared_gate = router ? (float*)c.take((size_t)M * 4) : nullptr;
  b.router_ws_bytes = router ? moe_router_workspace_bytes(M, D, E) : 0;
  b.router_ws = router ? c.take(b.router_ws_bytes) : nullptr;
  b.normed = router ? c.take((size_t)M * D * 2) : nullptr;   // RMS-normalised activations (norm_weight)
  b.total = c.used;
  return b;
}

}  // namespace

namespace {
// the activations the layer computes from: x itself, or its RMS-normalised form (kept in bf16 for the router)
// (sx_blocked: an optional second copy of the scales, block-major in token order, for the shared expert of a large batch)
int quantise(const MoeForwardArgs* a, const ForwardBuffers& b, float* sx_blocked, moe_stream_t stream) {
  if (a->norm_weight)
    return moe_rmsnorm_quant_impl(a->x, a->norm_weight, a->norm_eps, a->M, a->D, b.normed, b.xq, b.sx, sx_blocked, stream);
  return moe_quant_act_impl(a->x, a->M, a->D, b.xq, b.sx, sx_blocked, stream);
}
}  // namespace

extern "C" size_t moe_forward_workspace_bytes(int M, int D, int E, int k, int I, int SI) {
  if (M < 0 || D <= 0 || E <= 0 || k <= 0 || I <= 0 || SI < 0) return 0;
  return carve(nullptr, M, D, E, k, I, SI, true).total;   // room for the router whether or not a call uses it
}

extern "C" int moe_forward(const MoeForwardArgs* a, void* ws, size_t ws_bytes, moe_stream_t stream) {
  MOE_REQUIRE(a && ws, MOE_ERR_NULL, "forward: null args or workspace");
  MOE_REQUIRE(a->M >= 0 && a->D > 0 && a->E >= 1 && a->k >= 1 && a->I > 0 && a->SI >= 0, MOE_ERR_BAD_SHAPE,
              "forward: bad dims M=%d D=%d E=%d k=%d I=%d SI=%d", a->M, a->D, a->E, a->k, a->I, a->SI);
  MOE_REQUIRE(a->D % 128 == 0 && a->I % 128 == 0 && a->SI % 128 == 0, MOE_ERR_BAD_SHAPE,
              "forward: D=%d, I=%d and SI=%d must be multiples of 128", a->D, a->I, a->SI);
  MOE_REQUIRE((a->M == 0 || (a->x && (a->logits || a->w_router) && a->out)) && a->w_gate && a->w_up && a->w_down && a->sw_gate && a->sw_up && a->sw_down,
              MOE_ERR_NULL, "forward: null tensor pointer");
  if (a->SI)
    MOE_REQUIRE(a->ws_gate && a->ws_up && a->ws_down && a->sws_gate && a->sws_up && a->sws_down, MOE_ERR_NULL,
                "forward: SI > 0 but a shared-expert pointer is null");
  MOE_REQUIRE(MOE_ALIGNED16(ws), MOE_ERR_BAD_ALIGN, "forward: workspace must be 16-byte aligned");
  const size_t need = moe_forward_workspace_bytes(a->M, a->D, a->E, a->k, a->I, a->SI);
  MOE_REQUIRE(ws_bytes >= need, MOE_ERR_WORKSPACE_TOO_SMALL, "forward: workspace %zu < %zu", ws_bytes, need);
  if (a->M == 0) return MOE_OK;

  MOE_REQUIRE(!a->w_shared_gate || (a->w_router && a->SI), MOE_ERR_NULL,
              "forward: w_shared_gate needs w_router and a shared expert");
  MOE_REQUIRE(a->w_router || !a->out_logits, MOE_ERR_NULL, "forward: out_logits is an output of the router (w_router)");
  MOE_REQUIRE(a->w_shared_gate || !a->out_shared_gate, MOE_ERR_NULL, "forward: out_shared_gate needs w_shared_gate");
  ForwardBuffers b = carve(ws, a->M, a->D, a->E, a->k, a->I, a->SI, true);
  int32_t* idx = a->out_idx ? a->out_idx : b.idx;
  float* w = a->out_w ? a->out_w : b.w;
  int32_t* gsz = a->out_group_sizes ? a->out_group_sizes : b.group_sizes;
  int32_t* stid = a->out_sorted_token_ids ? a->out_sorted_token_ids : b.sorted_token_ids;
  int32_t* inv = a->out_inv_perm ? a->out_inv_perm : b.inv_perm;
  // the intermediate h is written straight into the caller's debug arrays when both are given
  MOE_REQUIRE((a->out_hq == nullptr) == (a->out_sh == nullptr), MOE_ERR_NULL, "forward: out_hq and out_sh come together");
  MOE_REQUIRE(MOE_ALIGNED16(a->out_hq), MOE_ERR_BAD_ALIGN, "forward: out_hq must be 16-byte aligned");
  uint8_t* hq = a->out_hq ? a->out_hq : b.hq;
  float* sh = a->out_sh ? a->out_sh : b.sh;
  MOE_REQUIRE((a->out_hsq == nullptr) == (a->out_shs == nullptr) && (!a->out_hsq || a->SI), MOE_ERR_NULL,
              "forward: out_hsq and out_shs come together and need a shared expert");
  MOE_REQUIRE(MOE_ALIGNED16(a->out_hsq), MOE_ERR_BAD_ALIGN, "forward: out_hsq must be 16-byte aligned");
  uint8_t* hsq = a->out_hsq ? a->out_hsq : b.hsq;
  float* shs = a->out_shs ? a->out_shs : b.shs;
  MOE_REQUIRE(!a->out_ys || a->SI, MOE_ERR_NULL, "forward: out_ys needs a shared expert");
  MOE_REQUIRE(MOE_ALIGNED16(a->out_y) && MOE_ALIGNED16(a->out_ys), MOE_ERR_BAD_ALIGN, "forward: out_y / out_ys must be 16-byte aligned");
  void* y = a->out_y ? a->out_y : b.y;
  void* ys = a->out_ys ? a->out_ys : b.ys;
  const int R = a->M * a->k;
  // large batches read their activation scales from block-major arrays (GemmScales); a decode-sized batch touches
  // few scale lines either way and is spared the extra launch
  const bool blocked_scales = R > 2048;
  hipStream_t main_s = (hipStream_t)stream;
  MOE_REQUIRE(a->routing == MOE_ROUTING_SOFTMAX || a->routing == MOE_ROUTING_SIGMOID_GROUPED, MOE_ERR_BAD_SHAPE,
              "forward: unknown routing %d", a->routing);
  int rc;

  // With a shared expert the call forks: the side stream runs the shared expert while the caller's stream routes,
  // permutes and runs the routed experts; the combine waits for the shared expert's output.  (Event record / wait
  // is also the pattern a capturing caller's graph turns into forks and joins.)
  //   Large batches fork at once: the side stream quantises the activations and starts the shared expert while the
  // caller's stream routes and permutes; the routed gate/up GEMM waits for the quantised activations.
  //   Small batches are bound by launch latency, so nothing may stand between the caller's stream and the routed
  // GEMMs: the activations are quantised on the caller's stream, the side stream waits for them, and the shared
  // expert's launches are enqueued after the routed ones (they still run beside them: the routed GEMMs take far longer).
  const bool small_batch = (long long)a->M * a->D <= (1ll << 21);
  hipStream_t side = nullptr;
  hipEvent_t ev_fork = nullptr, ev_quant = nullptr, ev_join = nullptr;
  int rc_shared = MOE_OK;
  bool quant_joined = true;
  bool side_forked = false;   // the side stream has been made to wait for work of this call on the caller's stream
  // the shared expert's one group and its tile list (they depend on M alone: enqueued ahead of the quantiser where
  // the side stream runs it, so that nothing stands between the quantiser and the shared gate/up GEMM)
  auto list_shared = [&]() {
    if (!rc_shared)
      rc_shared = moe_gemm_build_dense_tile_list(a->M, b.gemm_ws_shared, b.gemm_ws_shared_bytes, (moe_stream_t)side);
  };
  auto launch_shared = [&]() {
    GemmScales sc = moe_row_major_scales(a->D, a->SI);
    const float* sx_shared = b.sx;
    if (blocked_scales) {   // (block-major scales in token order: written by the quantiser itself)
      sx_shared = b.sx_blocked;
      sc.in_row = 1, sc.in_kb = a->M, sc.in_listed = true;
      if (!a->out_shs) sc.out_row = 1, sc.out_cb = a->M;   // (a debug copy of the h scales keeps the documented layout)
    }
    if (!rc_shared)
      rc_shared = moe_gemm_gateup_impl(b.xq, sx_shared, nullptr, a->ws_gate, a->sws_gate, a->ws_up, a->sws_up, b.dense_off,
                                       1, a->M, a->D, a->SI, hsq, shs, b.gemm_ws_shared, b.gemm_ws_shared_bytes, true, sc,
                                       (moe_stream_t)side);
    if (!rc_shared)   // same rows, same tile height: the list the gate/up launch built serves the down launch too
      rc_shared = moe_gemm_down_impl(hsq, shs, a->ws_down, a->sws_down, b.dense_off, 1, a->M, a->SI, a->D, ys,
                                     b.gemm_ws_shared, b.gemm_ws_shared_bytes, true,
                                     GemmScales{sc.out_row, sc.out_cb, true, 0, 0}, (moe_stream_t)side);
  };
  bool shared_pending = false;
  // Where the quantiser would run on the caller's stream just ahead of the routing kernel, the routing launch
  // carries its blocks instead (QuantJob: the two are independent; one launch less and they overlap).  Not with
  // an RMSNorm in front: the router then reads what the quantiser writes.
  const bool quant_in_route = (!a->SI || small_batch) && !a->norm_weight && a->M > 0;
  QuantJob quant_job{};
  if (quant_in_route &&
      (rc = moe_quant_act_job(a->x, a->M, a->D, b.xq, b.sx, (a->SI && blocked_scales) ? b.sx_blocked : nullptr, &quant_job)))
    return rc;
  if (a->SI) {
    if ((rc = side_stream(&side))) return rc;
    CallEvents* ev = nullptr;
    if ((rc = call_events(&ev))) return rc;
    ev_fork = ev->fork, ev_quant = ev->quant, ev_join = ev->join;
    if (!small_batch) {
      hipError_t e = hipEventRecord(ev_fork, main_s);
      if (e == hipSuccess) e = hipStreamWaitEvent(side, ev_fork, 0);
      if (e != hipSuccess) return moe_check_hip(e, "forward: fork");
      side_forked = true;
    }
    if (small_batch) {
      if (!quant_in_route) {
        rc_shared = quantise(a, b, blocked_scales ? b.sx_blocked : nullptr, stream);
        if (!rc_shared) rc_shared = moe_check_hip(hipEventRecord(ev_quant, main_s), "forward: quant event");
        if (!rc_shared) {
          rc_shared = moe_check_hip(hipStreamWaitEvent(side, ev_quant, 0), "forward: fork");
          side_forked = !rc_shared;
        }
      }   // (else: the same record and wait follow the routing launch, below)
      shared_pending = true;
    } else {
      quant_joined = false;
      list_shared();
      if (!rc_shared) rc_shared = quantise(a, b, blocked_scales ? b.sx_blocked : nullptr, (moe_stream_t)side);
      if (!rc_shared) rc_shared = moe_check_hip(hipEventRecord(ev_quant, side), "forward: quant event");
      launch_shared();
    }
  } else if (!quant_in_route) {
    if ((rc = quantise(a, b, nullptr, stream))) return rc;
  }
  // Once the side stream has been forked off this call, the join is enqueued on every path out of here, so that the
  // caller's stream (or the graph it is being captured into) never loses track of the side stream.  Before the
  // fork the side stream holds nothing of this call, and a wait on it would tie the caller's stream -- under
  // capture: the caller's graph -- to work that does not belong to it.
  auto join = [&](int code) {
    if (!a->SI) return code;
    if (shared_pending && side_forked && !code && !rc_shared) {
      list_shared();
      launch_shared();
    }
    shared_pending = false;
    if (!side_forked) return code ? code : rc_shared;
    hipError_t e1 = hipEventRecord(ev_join, side);
    hipError_t e2 = hipStreamWaitEvent(main_s, ev_join, 0);
    if (code) return code;
    if (rc_shared) return rc_shared;
    if (e1 != hipSuccess) return moe_check_hip(e1, "forward: join");
    return moe_check_hip(e2, "forward: join");
  };

  if (small_batch && rc_shared) return join(rc_shared);
  // With a router weight the routing kernel adds the matmul's split-K partial sums itself: the (M, E) logits
  // are written only when out_logits asks for them.
  LogitSource src{a->logits, nullptr, 0, a->E, nullptr, nullptr};
  const float* shared_gate = nullptr;
  if (a->w_router) {
    // the router reads the normalised activations, which the (possibly forked) quantiser writes
    if (a->norm_weight && !quant_joined) {
      if (rc_shared) return join(rc_shared);
      if ((rc = moe_check_hip(hipStreamWaitEvent(main_s, ev_quant, 0), "forward: quant join"))) return join(rc);
      quant_joined = true;
    }
    int splits = 0, n_cols = 0;
    if ((rc = moe_router_partials(a->norm_weight ? b.normed : a->x, a->M, a->D, a->w_router, a->E, a->w_shared_gate,
                                  b.router_ws, b.router_ws_bytes, &splits, &n_cols, stream)))
      return join(rc);
    float* gate_out = a->out_shared_gate ? a->out_shared_gate : b.shared_gate;   // (written by the routing kernel)
    if (a->w_shared_gate) shared_gate = gate_out;
    src = LogitSource{nullptr, (const float*)b.router_ws, splits, n_cols, a->out_logits, gate_out};
  }
  const QuantJob* carried = quant_in_route ? &quant_job : nullptr;
  if (a->routing == MOE_ROUTING_SOFTMAX)
    rc = moe_route_softmax_impl(src, a->M, a->E, a->k, a->renorm, idx, w, stream, carried);
  else
    rc = moe_route_sigmoid_grouped_impl(src, a->bias, a->M, a->E, a->n_group, a->topk_group, a->k, a->renorm,
                                        a->routed_scale, idx, w, stream, carried);
  if (rc) return join(rc);
  if (quant_in_route && a->SI) {   // the side stream's shared expert waits for the activations quantised above
    hipError_t e = hipEventRecord(ev_quant, main_s);
    if (e == hipSuccess) e = hipStreamWaitEvent(side, ev_quant, 0);
    if (e != hipSuccess) return join(moe_check_hip(e, "forward: quant event"));
    side_forked = true;
  }
  // the permutation kernels also list the routed GEMMs' row tiles (they hold every expert's row range anyway)
  TileList tiles;
  if ((rc = moe_gemm_tile_list(R, a->E, b.gemm_ws, b.gemm_ws_bytes, &tiles))) return join(rc);
  if ((rc = moe_permute_impl(idx, a->M, a->k, a->E, gsz, b.group_offsets, stid, nullptr, inv, b.permute_ws,
                             b.permute_ws_bytes, tiles, stream)))
    return join(rc);
  if (!quant_joined) {
    if (rc_shared) return join(rc_shared);
    if ((rc = moe_check_hip(hipStreamWaitEvent(main_s, ev_quant, 0), "forward: quant join"))) return join(rc);
  }
  GemmScales sc = moe_row_major_scales(a->D, a->I);
  const float* sx_routed = b.sx;
  if (blocked_scales) {
    if ((rc = moe_gather_scales(b.sx, stid, R, a->D / 128, b.sx_listed, stream))) return join(rc);
    sx_routed = b.sx_listed;
    sc.in_row = 1, sc.in_kb = R, sc.in_listed = true;
    if (!a->out_sh) sc.out_row = 1, sc.out_cb = R;
  }
  if ((rc = moe_gemm_gateup_impl(b.xq, sx_routed, stid, a->w_gate, a->sw_gate, a->w_up, a->sw_up, b.group_offsets, a->E,
                                 R, a->D, a->I, hq, sh, b.gemm_ws, b.gemm_ws_bytes, true, sc, stream)))
    return join(rc);
  if ((rc = moe_gemm_down_impl(hq, sh, a->w_down, a->sw_down, b.group_offsets, a->E, R, a->I, a->D, y,
                               b.gemm_ws, b.gemm_ws_bytes, true, GemmScales{sc.out_row, sc.out_cb, true, 0, 0}, stream)))
    return join(rc);
  if ((rc = join(MOE_OK))) return rc;
  return moe_combine(y, w, inv, a->SI ? ys : nullptr, shared_gate, a->add_residual ? a->x : nullptr, a->M, a->k,
                     a->D, a->out, stream);
}
