// C ABI of libfa2_gfx950.so: argument validation, the gfx950 tile/wave table and kernel launches.
// Declarations and the reference interfaces they replace are in include/fa2_gfx950.h.

#include "fa2_gfx950.h"

#include <hip/hip_runtime.h>

#include <algorithm>
#include <atomic>
#include <cmath>
#include <cstdarg>
#include <cstdio>

#include "fa2_launch.hpp"

namespace {

thread_local char g_error[512] = "";

int fail(int status, const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
  return status;
}

// ---- gfx950 tile/wave table -----------------------------------------------------------------
// One row per padded head dimension.  All rows use 4 waves of 64 lanes per workgroup and the
// 32x32x16 MFMA; a wave always owns 32 sequence positions of the operand it keeps in registers.
// What differs between rows is what the register file and LDS leave room for: whether the
// LDS-direct ("fast") kernels exist for the row, how many workgroups share a CU, how many LDS
// stages the streamed operand gets and in how many passes the dK/dV kernel covers the head dimension.
using fa2::kDkvBlockKV;
using fa2::kDkvBlockQ;
using fa2::kDqBlockKV;
using fa2::kDqBlockQ;
using fa2::kFwdBlockKV;
using fa2::kFwdBlockQ;
// (batch, head) pairs dispatched together: 8 per XCD, or 4 at head dimension 128, where a head's K and
// V rows are twice as large (C3, 64 heads: forward -0.9 %, dQ -1.3 % with 32 against 64; 16 costs
// 2-4 %; at head dimension 64 a group of 32 costs 5-10 %).
constexpr int kHeadGroup = 64;
constexpr int kHeadGroup128 = 32;

const fa2_config_info kTable[] = {
    // id DP  fwd:BQ       BKV        waves dK/dV:BQ   BKV       waves dQ:BQ    BKV      waves fast fwd/CU dq/CU dkdv/CU stages passes group atomic folded
    {0, 32, kFwdBlockQ, kFwdBlockKV, 4, kDkvBlockQ, kDkvBlockKV, 4, kDqBlockQ, kDqBlockKV, 4, 1, 4, 4, 3, 3, 1, kHeadGroup, 0, 0},
    {1, 64, kFwdBlockQ, kFwdBlockKV, 4, kDkvBlockQ, kDkvBlockKV, 4, kDqBlockQ, kDqBlockKV, 4, 1, 3, 3, 2, 3, 1, kHeadGroup, 0, 0},
    {2, 96, kFwdBlockQ, kFwdBlockKV, 4, kDkvBlockQ, kDkvBlockKV, 4, kDqBlockQ, kDqBlockKV, 4, 1, 2, 2, 1, 3, 1, kHeadGroup, 0, 0},
    {3, 128, kFwdBlockQ, kFwdBlockKV, 4, kDkvBlockQ, kDkvBlockKV, 4, kDqBlockQ, kDqBlockKV, 4, 1, 2, 2, 1, 3, 1, kHeadGroup128, 0, 0},
    {4, 192, kFwdBlockQ, kFwdBlockKV, 4, kDkvBlockQ, kDkvBlockKV, 4, kDqBlockQ, kDqBlockKV, 4, 2, 1, 1, 1, 2, 1, kHeadGroup, 0, 0},
    {5, 256, kFwdBlockQ, kFwdBlockKV, 4, kDkvBlockQ, kDkvBlockKV, 4, kDqBlockQ, kDqBlockKV, 4, 2, 1, 1, 1, 2, 2, kHeadGroup, 0, 0},
    // Sequence-parallel rows (dq_atomic = 1): the backward is one key-tile-parallel kernel that adds its
    // dQ contributions into an fp32 workspace with global atomics, the reference's non-deterministic
    // formulation (_triton_kernels_v2.py:336-339).  Never picked automatically: on MI355X the atomics
    // alone take longer than the whole two-kernel backward (profiles/bwd_sequence_parallel_atomic_*.txt);
    // a caller selects them by id.  Forward columns as in the row of the same head dimension.
    {6, 32, kFwdBlockQ, kFwdBlockKV, 4, kDkvBlockQ, kDkvBlockKV, 4, kDqBlockQ, kDqBlockKV, 4, 1, 4, 0, 1, 3, 1, kHeadGroup, 1, 0},
    {7, 64, kFwdBlockQ, kFwdBlockKV, 4, kDkvBlockQ, kDkvBlockKV, 4, kDqBlockQ, kDqBlockKV, 4, 1, 3, 0, 1, 3, 1, kHeadGroup, 1, 0},
    {8, 128, kFwdBlockQ, kFwdBlockKV, 4, kDkvBlockQ, kDkvBlockKV, 4, kDqBlockQ, kDqBlockKV, 4, 1, 2, 0, 1, 3, 1, kHeadGroup128, 1, 0},
    // Forward-only rows (fwd_exp_folded = 1): as rows 0-3, with the LDS-direct forward taking its exponents
    // straight from the score MFMAs (Q fragments multiplied by scale * log2(e) and rounded once).  Forward
    // -4 % on B=2 H=32 N=4096 D=128, -5 % at N=16384, -3.7 % at D=64.  Never picked by FA2_CONFIG_AUTO and
    // refused by the backward, which recomputes the probabilities from Q itself and needs the log-sum-exp
    // of exactly those scores; fa2_pick_config_forward_only returns them for bf16, where the extra half
    // unit in the last place of Q is of the size of the rounding the inputs already carry.
    {9, 32, kFwdBlockQ, kFwdBlockKV, 4, kDkvBlockQ, kDkvBlockKV, 4, kDqBlockQ, kDqBlockKV, 4, 1, 4, 4, 3, 3, 1, kHeadGroup, 0, 1},
    {10, 64, kFwdBlockQ, kFwdBlockKV, 4, kDkvBlockQ, kDkvBlockKV, 4, kDqBlockQ, kDqBlockKV, 4, 1, 3, 3, 2, 3, 1, kHeadGroup, 0, 1},
    {11, 96, kFwdBlockQ, kFwdBlockKV, 4, kDkvBlockQ, kDkvBlockKV, 4, kDqBlockQ, kDqBlockKV, 4, 1, 2, 2, 1, 3, 1, kHeadGroup, 0, 1},
    {12, 128, kFwdBlockQ, kFwdBlockKV, 4, kDkvBlockQ, kDkvBlockKV, 4, kDqBlockQ, kDqBlockKV, 4, 1, 2, 2, 1, 3, 1, kHeadGroup128, 0, 1},
};
constexpr int kTableRows = sizeof(kTable) / sizeof(kTable[0]);

// Heads dispatched together by the forward and dQ kernels: the table's group size, evened out over
// the heads there are (fa2::equal_head_groups).
int head_group(int cfg, int64_t heads) { return fa2::equal_head_groups(kTable[cfg].head_group, heads); }

// The row FA2_CONFIG_AUTO stands for: the first plain row wide enough for the head dimension.
int pick_config(int headdim) {
  for (int i = 0; i < kTableRows; i++)
    if (!kTable[i].dq_atomic && !kTable[i].fwd_exp_folded && headdim <= kTable[i].headdim_padded) return i;
  return -1;
}

// The row for a forward whose log-sum-exp no backward will read: for bf16 the folded row of the
// head dimension when there is one, else the plain row.
int pick_config_forward_only(int dtype, int headdim) {
  const int plain = pick_config(headdim);
  if (plain < 0 || dtype != FA2_DTYPE_BF16) return plain;
  for (int i = 0; i < kTableRows; i++)
    if (kTable[i].fwd_exp_folded && kTable[i].headdim_padded == kTable[plain].headdim_padded) return i;
  return plain;
}

// Query rows of the fp32 dQ accumulator of a sequence-parallel row: whole 64-row query tiles.
int64_t dq_accum_rows(int seqlen_q) { return ((int64_t)seqlen_q + kDkvBlockQ - 1) / kDkvBlockQ * kDkvBlockQ; }

int resolve_config(int config_id, int headdim, int *out) {
  if (config_id == FA2_CONFIG_AUTO) {
    *out = pick_config(headdim);
    return FA2_OK;
  }
  if (config_id < 0 || config_id >= kTableRows)
    return fail(FA2_ERR_BAD_CONFIG, "config id %d outside the table [0, %d)", config_id, kTableRows);
  if (kTable[config_id].headdim_padded < headdim)
    return fail(FA2_ERR_BAD_CONFIG, "config %d is built for headdim <= %d, got %d", config_id,
                kTable[config_id].headdim_padded, headdim);
  if (kTable[config_id].dq_atomic && kTable[config_id].headdim_padded != headdim)
    return fail(FA2_ERR_BAD_CONFIG, "sequence-parallel config %d is built for headdim == %d, got %d", config_id,
                kTable[config_id].headdim_padded, headdim);
  *out = config_id;
  return FA2_OK;
}

int check_common(int batch, int nheads, int seqlen_q, int seqlen_k, int headdim,
                 int seqlen_q_rounded, int dtype) {
  if (batch <= 0 || nheads <= 0 || seqlen_q <= 0 || seqlen_k <= 0 || headdim <= 0)
    return fail(FA2_ERR_BAD_SHAPE, "sizes must be positive: batch=%d nheads=%d seqlen_q=%d seqlen_k=%d headdim=%d",
                batch, nheads, seqlen_q, seqlen_k, headdim);
  if (seqlen_q_rounded < seqlen_q)
    return fail(FA2_ERR_BAD_SHAPE, "seqlen_q_rounded=%d < seqlen_q=%d", seqlen_q_rounded, seqlen_q);
  if (headdim > FA2_MAX_HEADDIM)
    return fail(FA2_ERR_HEADDIM, "Supports head dimensions only up to %d, got %d", FA2_MAX_HEADDIM, headdim);
  if (dtype != FA2_DTYPE_F16 && dtype != FA2_DTYPE_BF16)
    return fail(FA2_ERR_BAD_DTYPE, "dtype %d is neither FA2_DTYPE_F16 nor FA2_DTYPE_BF16", dtype);
  if ((int64_t)batch * nheads > 0x7fffffff / 64)
    return fail(FA2_ERR_TOO_LARGE, "batch*nheads=%lld too large", (long long)batch * nheads);
  return FA2_OK;
}

fa2::Tensor4 tensor(const fa2_tensor &t) {
  return fa2::Tensor4{const_cast<void *>(t.ptr), t.stride_batch, t.stride_head, t.stride_seq};
}

int check_tensor(const char *name, const fa2::Tensor4 &t) {
  if (t.ptr == nullptr) return fail(FA2_ERR_NULL_POINTER, "%s is NULL", name);
  if (t.stride_batch < 0 || t.stride_head < 0 || t.stride_seq < 0)
    return fail(FA2_ERR_BAD_STRIDE, "%s has a negative stride", name);
  return FA2_OK;
}

// 16-byte accesses need headdim % 8 == 0, 16-byte aligned bases and strides that keep rows aligned.
bool vec_ok(const fa2::Tensor4 &t, int headdim) {
  return headdim % 8 == 0 && (reinterpret_cast<uintptr_t>(t.ptr) % 16 == 0) &&
         t.stride_batch % 8 == 0 && t.stride_head % 8 == 0 && t.stride_seq % 8 == 0;
}

int launch_status(const char *what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(FA2_ERR_LAUNCH, "%s: %s", what, hipGetErrorString(e));
  return FA2_OK;
}

bool good_scale(float s) { return s > 0.f && std::isfinite(s); }

int fwd_impl(const fa2_fwd_args &a, void *stream) {
  int rc = check_common(a.batch, a.nheads, a.seqlen_q, a.seqlen_k, a.headdim, a.seqlen_q_rounded, a.dtype);
  if (rc) return rc;
  fa2::FwdParams p;
  p.q = tensor(a.q);
  p.k = tensor(a.k);
  p.v = tensor(a.v);
  p.o = tensor(a.o);
  if ((rc = check_tensor("q", p.q)) || (rc = check_tensor("k", p.k)) ||
      (rc = check_tensor("v", p.v)) || (rc = check_tensor("o", p.o)))
    return rc;
  if (a.lse == nullptr) return fail(FA2_ERR_NULL_POINTER, "lse is NULL");
  if (!good_scale(a.softmax_scale))
    return fail(FA2_ERR_BAD_SHAPE, "softmax_scale must be positive and finite, got %g", (double)a.softmax_scale);
  int cfg;
  if ((rc = resolve_config(a.config_id, a.headdim, &cfg))) return rc;

  p.lse = a.lse;
  p.batch = a.batch;
  p.nheads = a.nheads;
  p.seqlen_q = a.seqlen_q;
  p.seqlen_k = a.seqlen_k;
  p.headdim = a.headdim;
  p.seqlen_q_rounded = a.seqlen_q_rounded;
  p.n_qtiles = (a.seqlen_q + kFwdBlockQ - 1) / kFwdBlockQ;
  p.head_group = head_group(cfg, (int64_t)a.batch * a.nheads);
  p.scale = a.softmax_scale;
  p.scale_log2 = a.softmax_scale * fa2::kLog2e;
  p.vec = vec_ok(p.q, a.headdim) && vec_ok(p.k, a.headdim) && vec_ok(p.v, a.headdim) && vec_ok(p.o, a.headdim);

  const int64_t nwg = (int64_t)p.n_qtiles * a.batch * a.nheads;
  if (nwg > 0x7fffffff) return fail(FA2_ERR_TOO_LARGE, "grid of %lld workgroups too large", (long long)nwg);
  fa2::launch_fwd(a.dtype == FA2_DTYPE_BF16, kTable[cfg].headdim_padded, kTable[cfg].fwd_exp_folded != 0, p,
                  dim3((unsigned)nwg), reinterpret_cast<hipStream_t>(stream));
  return launch_status("fa2_fwd launch");
}

int preprocess_impl(const fa2_tensor &o, const fa2_tensor &d_o, float *delta, int batch, int nheads,
                    int seqlen_q, int headdim, int seqlen_q_rounded, int dtype, void *stream) {
  int rc = check_common(batch, nheads, seqlen_q, 1, headdim, seqlen_q_rounded, dtype);
  if (rc) return rc;
  fa2::PreParams p;
  p.o = tensor(o);
  p.d_o = tensor(d_o);
  if ((rc = check_tensor("o", p.o)) || (rc = check_tensor("d_o", p.d_o))) return rc;
  if (delta == nullptr) return fail(FA2_ERR_NULL_POINTER, "delta is NULL");
  p.delta = delta;
  p.batch = batch;
  p.nheads = nheads;
  p.seqlen_q = seqlen_q;
  p.headdim = headdim;
  p.seqlen_q_rounded = seqlen_q_rounded;
  p.vec = vec_ok(p.o, headdim) && vec_ok(p.d_o, headdim);
  const int64_t nwg = (int64_t)((seqlen_q_rounded + 15) / 16) * batch * nheads;
  if (nwg > 0x7fffffff) return fail(FA2_ERR_TOO_LARGE, "grid of %lld workgroups too large", (long long)nwg);
  fa2::launch_preprocess(dtype == FA2_DTYPE_BF16, p, dim3((unsigned)nwg), reinterpret_cast<hipStream_t>(stream));
  return launch_status("fa2_bwd_preprocess launch");
}

// Backward behind fa2_bwd, fa2_bwd_fused and fa2_bwd_packed.  With a.o given, delta is an
// output: it is formed by the dQ kernel when the fast dQ kernel applies (and the dK/dV kernel then
// runs second), otherwise by the preprocess kernel launched from here.  With the rows the table
// picks by itself `deterministic` and `workspace` are accepted and not needed: dQ is written once,
// in a fixed order, in both modes.  The sequence-parallel rows (dq_atomic) take the workspace.
int bwd_impl(const fa2_bwd_args &a, void *stream) {
  int rc = check_common(a.batch, a.nheads, a.seqlen_q, a.seqlen_k, a.headdim, a.seqlen_q_rounded, a.dtype);
  if (rc) return rc;
  const bool fused = a.o.ptr != nullptr;
  fa2::BwdParams p;
  p.q = tensor(a.q);
  p.k = tensor(a.k);
  p.v = tensor(a.v);
  p.d_o = tensor(a.d_o);
  p.dq = tensor(a.dq);
  p.dk = tensor(a.dk);
  p.dv = tensor(a.dv);
  p.o = fused ? tensor(a.o) : fa2::Tensor4{nullptr, 0, 0, 0};
  // A caller that needs only part of the gradient passes NULL for the rest: dq == NULL skips the
  // dQ kernel, dk == dv == NULL skips the dK/dV kernel.  dk and dv come from one kernel, so they
  // are given or omitted together.
  const bool want_dq = a.dq.ptr != nullptr;
  const bool want_dkdv = a.dk.ptr != nullptr || a.dv.ptr != nullptr;
  if (!want_dq && !want_dkdv) return fail(FA2_ERR_NULL_POINTER, "dq, dk and dv are all NULL");
  if (fused && !(want_dq && want_dkdv))
    return fail(FA2_ERR_NULL_POINTER, "with o given (delta formed on the way) none of dq, dk, dv may be NULL");
  if ((rc = check_tensor("q", p.q)) || (rc = check_tensor("k", p.k)) ||
      (rc = check_tensor("v", p.v)) || (rc = check_tensor("d_o", p.d_o)))
    return rc;
  if (fused && (rc = check_tensor("o", p.o))) return rc;
  if (want_dq && (rc = check_tensor("dq", p.dq))) return rc;
  if (want_dkdv && ((rc = check_tensor("dk", p.dk)) || (rc = check_tensor("dv", p.dv)))) return rc;
  if (a.lse == nullptr) return fail(FA2_ERR_NULL_POINTER, "lse is NULL");
  if (a.delta == nullptr) return fail(FA2_ERR_NULL_POINTER, "delta is NULL");
  if (!good_scale(a.softmax_scale))
    return fail(FA2_ERR_BAD_SHAPE, "softmax_scale must be positive and finite, got %g", (double)a.softmax_scale);
  int cfg;
  if ((rc = resolve_config(a.config_id, a.headdim, &cfg))) return rc;
  if (kTable[cfg].fwd_exp_folded)
    return fail(FA2_ERR_BAD_CONFIG, "config %d is a forward-only row: its forward rounds Q * scale, and the "
                                    "backward recomputes the probabilities from Q itself", cfg);

  p.lse = a.lse;
  p.delta = a.delta;
  p.delta_out = a.delta;
  p.batch = a.batch;
  p.nheads = a.nheads;
  p.seqlen_q = a.seqlen_q;
  p.seqlen_k = a.seqlen_k;
  p.headdim = a.headdim;
  p.seqlen_q_rounded = a.seqlen_q_rounded;
  p.head_group = head_group(cfg, (int64_t)a.batch * a.nheads);
  p.scale = a.softmax_scale;
  p.scale_log2 = a.softmax_scale * fa2::kLog2e;
  p.vec = vec_ok(p.q, a.headdim) && vec_ok(p.k, a.headdim) && vec_ok(p.v, a.headdim) &&
          vec_ok(p.d_o, a.headdim) && (!want_dq || vec_ok(p.dq, a.headdim)) &&
          (!want_dkdv || (vec_ok(p.dk, a.headdim) && vec_ok(p.dv, a.headdim)));

  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  const bool bf16 = a.dtype == FA2_DTYPE_BF16;
  const int dp = kTable[cfg].headdim_padded;
  const int64_t bh = (int64_t)a.batch * a.nheads;
  p.dq_accum = nullptr;
  p.dq_accum_rows = 0;

  fa2::BwdParams pk = p, pq = p;
  // The dK/dV kernel keeps the table's group size at every head count: with one or two workgroups
  // per CU its drain is short either way, and measured at 96 heads the single group is 1-2 % slower.
  pk.head_group = kTable[cfg].head_group;
  pk.n_tiles = (a.seqlen_k + kDkvBlockKV - 1) / kDkvBlockKV;
  pq.n_tiles = (a.seqlen_q + kDqBlockQ - 1) / kDqBlockQ;
  const int64_t nwg_k = pk.n_tiles * bh, nwg_q = pq.n_tiles * bh;
  if (nwg_k > 0x7fffffff || nwg_q > 0x7fffffff)
    return fail(FA2_ERR_TOO_LARGE, "grid of %lld workgroups too large", (long long)std::max(nwg_k, nwg_q));

  auto run_dkdv = [&]() {
    fa2::launch_dkdv(bf16, dp, pk, dim3((unsigned)nwg_k), s);
    return launch_status("backward dK/dV launch");
  };

  if (kTable[cfg].dq_atomic) {
    // Sequence-parallel mode: clear the accumulator, (form delta), one key-tile-parallel kernel for
    // dK, dV and the atomic dQ contributions, then dq = scale * accumulator.
    if (a.deterministic)
      return fail(FA2_ERR_BAD_CONFIG, "config %d accumulates dQ with atomics: not available with deterministic=1", cfg);
    if (!(want_dq && want_dkdv))
      return fail(FA2_ERR_NULL_POINTER, "the sequence-parallel backward produces dq, dk and dv together");
    if (a.workspace == nullptr)
      return fail(FA2_ERR_WORKSPACE, "config %d needs fa2_bwd_workspace_bytes() bytes of workspace", cfg);
    if (reinterpret_cast<uintptr_t>(a.workspace) % 16 != 0)
      return fail(FA2_ERR_WORKSPACE, "workspace must be 16-byte aligned");
    if (!fa2::seqpar_atomic_ok(dp, pk))
      return fail(FA2_ERR_BAD_CONFIG, "the sequence-parallel kernels need 16-byte aligned tensors and strides "
                                      "and a head dimension of 32, 64 or 128");
    pk.dq_accum = static_cast<float *>(a.workspace);
    pk.dq_accum_rows = (int)dq_accum_rows(a.seqlen_q);
    fa2::launch_dq_accum_zero(pk.dq_accum, bh * pk.dq_accum_rows * a.headdim, s);
    if ((rc = launch_status("dQ accumulator clear"))) return rc;
    if (fused) {
      rc = preprocess_impl(a.o, a.d_o, a.delta, a.batch, a.nheads, a.seqlen_q, a.headdim, a.seqlen_q_rounded,
                           a.dtype, stream);
      if (rc) return rc;
    }
    if ((rc = run_dkdv())) return rc;
    fa2::launch_dq_accum_convert(bf16, pk, s);
    return launch_status("dQ accumulator convert");
  }

  if (fused && fa2::dq_direct_ok(dp, pq) && vec_ok(p.o, a.headdim)) {
    // dQ first: it writes delta, which the dK/dV kernel reads.
    fa2::launch_dq(bf16, dp, pq, dim3((unsigned)nwg_q), true, s);
    if ((rc = launch_status("backward dQ launch (delta fused)"))) return rc;
    return run_dkdv();
  }
  if (fused) {
    rc = preprocess_impl(a.o, a.d_o, a.delta, a.batch, a.nheads, a.seqlen_q, a.headdim, a.seqlen_q_rounded,
                         a.dtype, stream);
    if (rc) return rc;
  }
  if (want_dkdv && (rc = run_dkdv())) return rc;
  if (want_dq) {
    fa2::launch_dq(bf16, dp, pq, dim3((unsigned)nwg_q), false, s);
    if ((rc = launch_status("backward dQ launch"))) return rc;
  }
  return FA2_OK;
}

fa2_tensor make_tensor(const void *ptr, int64_t sb, int64_t sh, int64_t ss) { return fa2_tensor{ptr, sb, sh, ss}; }

// ---- delta scratch of fa2_bwd_fused_noalloc ---------------------------------------------------
// fa2_bwd_fused needs batch * nheads * seqlen_q_rounded floats of scratch (delta) from its caller.
// The variant for callers that cannot allocate keeps that scratch here, in a device array that
// every GPU the library runs on holds until the process ends.  In host code `scratch` is only a
// handle for hipGetSymbolAddress: the device address differs per GPU and is looked up once per
// device (with that device current) and kept in g_scratch_addr.
constexpr size_t kScratchFloats = FA2_NOALLOC_MAX_ROWS;
static __device__ __align__(256) float scratch[kScratchFloats];
constexpr int kMaxDevices = 64;
std::atomic<float *> g_scratch_addr[kMaxDevices];

int scratch_on_current_device(float **out) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return fail(FA2_ERR_LAUNCH, "hipGetDevice: %s", hipGetErrorString(e));
  if (dev < 0 || dev >= kMaxDevices)
    return fail(FA2_ERR_TOO_LARGE, "device ordinal %d outside [0, %d)", dev, kMaxDevices);
  float *addr = g_scratch_addr[dev].load(std::memory_order_acquire);
  if (addr == nullptr) {
    // Two threads may both get here the first time; they find the same address.
    void *sym = nullptr;
    e = hipGetSymbolAddress(&sym, HIP_SYMBOL(scratch));
    if (e != hipSuccess || sym == nullptr)
      return fail(FA2_ERR_LAUNCH, "hipGetSymbolAddress(scratch) on device %d: %s", dev, hipGetErrorString(e));
    addr = static_cast<float *>(sym);
    g_scratch_addr[dev].store(addr, std::memory_order_release);
  }
  *out = addr;
  return FA2_OK;
}

}  // namespace

extern "C" {

int fa2_abi_version(void) { return FA2_ABI_VERSION; }

const char *fa2_last_error_string(void) { return g_error; }

const char *fa2_status_string(int status) {
  switch (status) {
    case FA2_OK: return "FA2_OK";
    case FA2_ERR_NULL_POINTER: return "FA2_ERR_NULL_POINTER";
    case FA2_ERR_BAD_SHAPE: return "FA2_ERR_BAD_SHAPE";
    case FA2_ERR_BAD_DTYPE: return "FA2_ERR_BAD_DTYPE";
    case FA2_ERR_HEADDIM: return "FA2_ERR_HEADDIM";
    case FA2_ERR_BAD_STRIDE: return "FA2_ERR_BAD_STRIDE";
    case FA2_ERR_BAD_CONFIG: return "FA2_ERR_BAD_CONFIG";
    case FA2_ERR_WORKSPACE: return "FA2_ERR_WORKSPACE";
    case FA2_ERR_LAUNCH: return "FA2_ERR_LAUNCH";
    case FA2_ERR_TOO_LARGE: return "FA2_ERR_TOO_LARGE";
    default: return "FA2_ERR_UNKNOWN";
  }
}

int fa2_config_count(void) { return kTableRows; }

int fa2_config_get(int config_id, fa2_config_info *out) {
  if (out == nullptr) return fail(FA2_ERR_NULL_POINTER, "out is NULL");
  if (config_id < 0 || config_id >= kTableRows)
    return fail(FA2_ERR_BAD_CONFIG, "config id %d outside the table [0, %d)", config_id, kTableRows);
  *out = kTable[config_id];
  return FA2_OK;
}

int fa2_pick_config(int dtype, int headdim, int seqlen_q, int seqlen_k, int deterministic) {
  (void)deterministic;  // both backward modes use the same row; sequence lengths are validated only
  if (dtype != FA2_DTYPE_F16 && dtype != FA2_DTYPE_BF16)
    return -fail(FA2_ERR_BAD_DTYPE, "dtype %d is neither FA2_DTYPE_F16 nor FA2_DTYPE_BF16", dtype);
  if (headdim <= 0 || seqlen_q <= 0 || seqlen_k <= 0)
    return -fail(FA2_ERR_BAD_SHAPE, "sizes must be positive: headdim=%d seqlen_q=%d seqlen_k=%d",
                 headdim, seqlen_q, seqlen_k);
  int id = pick_config(headdim);
  if (id < 0)
    return -fail(FA2_ERR_HEADDIM, "Supports head dimensions only up to %d, got %d", FA2_MAX_HEADDIM, headdim);
  return id;
}

int fa2_pick_config_forward_only(int dtype, int headdim, int seqlen_q, int seqlen_k) {
  const int id = fa2_pick_config(dtype, headdim, seqlen_q, seqlen_k, 0);  // validates
  return id < 0 ? id : pick_config_forward_only(dtype, headdim);
}

int fa2_fwd_packed(const fa2_fwd_args *args, void *stream) {
  if (args == nullptr) return fail(FA2_ERR_NULL_POINTER, "args is NULL");
  return fwd_impl(*args, stream);
}

int fa2_bwd_packed(const fa2_bwd_args *args, void *stream) {
  if (args == nullptr) return fail(FA2_ERR_NULL_POINTER, "args is NULL");
  return bwd_impl(*args, stream);
}

int fa2_fwd(const void *q, const void *k, const void *v, void *o, float *lse, int batch, int nheads,
            int seqlen_q, int seqlen_k, int headdim, int seqlen_q_rounded, int64_t q_sb,
            int64_t q_sh, int64_t q_ss, int64_t k_sb, int64_t k_sh, int64_t k_ss, int64_t v_sb,
            int64_t v_sh, int64_t v_ss, int64_t o_sb, int64_t o_sh, int64_t o_ss,
            float softmax_scale, int dtype, int config_id, void *stream) {
  fa2_fwd_args a;
  a.q = make_tensor(q, q_sb, q_sh, q_ss);
  a.k = make_tensor(k, k_sb, k_sh, k_ss);
  a.v = make_tensor(v, v_sb, v_sh, v_ss);
  a.o = make_tensor(o, o_sb, o_sh, o_ss);
  a.lse = lse;
  a.batch = batch;
  a.nheads = nheads;
  a.seqlen_q = seqlen_q;
  a.seqlen_k = seqlen_k;
  a.headdim = headdim;
  a.seqlen_q_rounded = seqlen_q_rounded;
  a.softmax_scale = softmax_scale;
  a.dtype = dtype;
  a.config_id = config_id;
  return fwd_impl(a, stream);
}

int fa2_bwd_preprocess(const void *o, const void *d_o, float *delta, int batch, int nheads,
                       int seqlen_q, int headdim, int seqlen_q_rounded, int64_t o_sb, int64_t o_sh,
                       int64_t o_ss, int64_t do_sb, int64_t do_sh, int64_t do_ss, int dtype,
                       void *stream) {
  return preprocess_impl(make_tensor(o, o_sb, o_sh, o_ss), make_tensor(d_o, do_sb, do_sh, do_ss), delta, batch,
                         nheads, seqlen_q, headdim, seqlen_q_rounded, dtype, stream);
}

size_t fa2_bwd_workspace_bytes(int batch, int nheads, int seqlen_q, int seqlen_k, int headdim,
                               int deterministic, int config_id) {
  (void)seqlen_k; (void)deterministic;
  // The two-kernel backward writes dQ exactly once from registers: no accumulation buffer.  A
  // sequence-parallel row accumulates dQ in fp32: batch * nheads * (seqlen_q rounded up to 64) * headdim floats.
  if (config_id < 0 || config_id >= kTableRows || !kTable[config_id].dq_atomic) return 0;
  if (batch <= 0 || nheads <= 0 || seqlen_q <= 0 || headdim <= 0) return 0;
  return (size_t)batch * (size_t)nheads * (size_t)dq_accum_rows(seqlen_q) * (size_t)headdim * sizeof(float);
}

int fa2_bwd(const void *q, const void *k, const void *v, const void *d_o, const float *lse,
            const float *delta, void *workspace, void *dq, void *dk, void *dv, int batch,
            int nheads, int seqlen_q, int seqlen_k, int headdim, int seqlen_q_rounded, int64_t q_sb,
            int64_t q_sh, int64_t q_ss, int64_t k_sb, int64_t k_sh, int64_t k_ss, int64_t v_sb,
            int64_t v_sh, int64_t v_ss, int64_t do_sb, int64_t do_sh, int64_t do_ss, int64_t dq_sb,
            int64_t dq_sh, int64_t dq_ss, int64_t dk_sb, int64_t dk_sh, int64_t dk_ss,
            int64_t dv_sb, int64_t dv_sh, int64_t dv_ss, float softmax_scale, int dtype,
            int deterministic, int config_id, void *stream) {
  fa2_bwd_args a;
  a.q = make_tensor(q, q_sb, q_sh, q_ss);
  a.k = make_tensor(k, k_sb, k_sh, k_ss);
  a.v = make_tensor(v, v_sb, v_sh, v_ss);
  a.o = make_tensor(nullptr, 0, 0, 0);
  a.d_o = make_tensor(d_o, do_sb, do_sh, do_ss);
  a.dq = make_tensor(dq, dq_sb, dq_sh, dq_ss);
  a.dk = make_tensor(dk, dk_sb, dk_sh, dk_ss);
  a.dv = make_tensor(dv, dv_sb, dv_sh, dv_ss);
  a.lse = lse;
  a.delta = const_cast<float *>(delta);  // only read when o is not given
  a.workspace = workspace;
  a.batch = batch;
  a.nheads = nheads;
  a.seqlen_q = seqlen_q;
  a.seqlen_k = seqlen_k;
  a.headdim = headdim;
  a.seqlen_q_rounded = seqlen_q_rounded;
  a.softmax_scale = softmax_scale;
  a.dtype = dtype;
  a.deterministic = deterministic;
  a.config_id = config_id;
  return bwd_impl(a, stream);
}

int fa2_bwd_fused(const void *q, const void *k, const void *v, const void *o, const void *d_o,
                  const float *lse, float *delta, void *workspace, void *dq, void *dk, void *dv,
                  int batch, int nheads, int seqlen_q, int seqlen_k, int headdim,
                  int seqlen_q_rounded, int64_t q_sb, int64_t q_sh, int64_t q_ss, int64_t k_sb,
                  int64_t k_sh, int64_t k_ss, int64_t v_sb, int64_t v_sh, int64_t v_ss, int64_t o_sb,
                  int64_t o_sh, int64_t o_ss, int64_t do_sb, int64_t do_sh, int64_t do_ss,
                  int64_t dq_sb, int64_t dq_sh, int64_t dq_ss, int64_t dk_sb, int64_t dk_sh,
                  int64_t dk_ss, int64_t dv_sb, int64_t dv_sh, int64_t dv_ss, float softmax_scale,
                  int dtype, int deterministic, int config_id, void *stream) {
  if (o == nullptr) return fail(FA2_ERR_NULL_POINTER, "o is NULL");
  fa2_bwd_args a;
  a.q = make_tensor(q, q_sb, q_sh, q_ss);
  a.k = make_tensor(k, k_sb, k_sh, k_ss);
  a.v = make_tensor(v, v_sb, v_sh, v_ss);
  a.o = make_tensor(o, o_sb, o_sh, o_ss);
  a.d_o = make_tensor(d_o, do_sb, do_sh, do_ss);
  a.dq = make_tensor(dq, dq_sb, dq_sh, dq_ss);
  a.dk = make_tensor(dk, dk_sb, dk_sh, dk_ss);
  a.dv = make_tensor(dv, dv_sb, dv_sh, dv_ss);
  a.lse = lse;
  a.delta = delta;
  a.workspace = workspace;
  a.batch = batch;
  a.nheads = nheads;
  a.seqlen_q = seqlen_q;
  a.seqlen_k = seqlen_k;
  a.headdim = headdim;
  a.seqlen_q_rounded = seqlen_q_rounded;
  a.softmax_scale = softmax_scale;
  a.dtype = dtype;
  a.deterministic = deterministic;
  a.config_id = config_id;
  return bwd_impl(a, stream);
}

int fa2_bwd_fused_noalloc(const void *q, const void *k, const void *v, const void *o, const void *d_o,
                          const float *lse, void *dq, void *dk, void *dv, int batch, int nheads,
                          int seqlen_q, int seqlen_k, int headdim, int seqlen_q_rounded, int64_t q_sb,
                          int64_t q_sh, int64_t q_ss, int64_t k_sb, int64_t k_sh, int64_t k_ss,
                          int64_t v_sb, int64_t v_sh, int64_t v_ss, int64_t o_sb, int64_t o_sh,
                          int64_t o_ss, int64_t do_sb, int64_t do_sh, int64_t do_ss, int64_t dq_sb,
                          int64_t dq_sh, int64_t dq_ss, int64_t dk_sb, int64_t dk_sh, int64_t dk_ss,
                          int64_t dv_sb, int64_t dv_sh, int64_t dv_ss, float softmax_scale, int dtype,
                          int deterministic, int config_id, void *stream) {
  if (o == nullptr) return fail(FA2_ERR_NULL_POINTER, "o is NULL");
  if (batch <= 0 || nheads <= 0 || seqlen_q_rounded <= 0)
    return fail(FA2_ERR_BAD_SHAPE, "sizes must be positive: batch=%d nheads=%d seqlen_q_rounded=%d", batch,
                nheads, seqlen_q_rounded);
  const uint64_t rows = (uint64_t)batch * (uint64_t)nheads * (uint64_t)seqlen_q_rounded;
  if (rows > kScratchFloats)
    return fail(FA2_ERR_TOO_LARGE,
                "batch*nheads*seqlen_q_rounded = %llu rows exceed the %llu rows of built-in scratch "
                "(FA2_NOALLOC_MAX_ROWS); use fa2_bwd_fused with a caller-supplied delta buffer",
                (unsigned long long)rows, (unsigned long long)kScratchFloats);
  float *delta = nullptr;
  if (int rc = scratch_on_current_device(&delta)) return rc;
  // Every row of delta the kernels read is written earlier in the same call (by the dQ kernel or
  // the preprocess kernel), so nothing left over from an earlier call has to be cleared.
  return fa2_bwd_fused(q, k, v, o, d_o, lse, delta, nullptr, dq, dk, dv, batch, nheads, seqlen_q, seqlen_k,
                       headdim, seqlen_q_rounded, q_sb, q_sh, q_ss, k_sb, k_sh, k_ss, v_sb, v_sh, v_ss, o_sb,
                       o_sh, o_ss, do_sb, do_sh, do_ss, dq_sb, dq_sh, dq_ss, dk_sb, dk_sh, dk_ss, dv_sb,
                       dv_sh, dv_ss, softmax_scale, dtype, deterministic, config_id, stream);
}

}  // extern "C"
