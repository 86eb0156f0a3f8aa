// C ABI of libfa2_gfx950.so: argument validation, the gfx950 tile table and kernel launches.
// Declarations and the reference interfaces they replace are in include/fa2_gfx950.h.

#include "fa2_gfx950.h"

#include <hip/hip_runtime.h>

#include <algorithm>
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
using fa2::kDkvBlockQ;
using fa2::kDqBlockKV;
using fa2::kFwdBlockKV;

const fa2_config_info kTable[] = {
    // id  DP   fwd: BQ   BKV waves   dK/dV: BQ  BKV  waves   dQ: BQ  BKV  waves
    {0, 32, fa2::kFwdBlockQ, kFwdBlockKV, 4, kDkvBlockQ, fa2::kDkvBlockKV, 4, fa2::kDqBlockQ, kDqBlockKV, 4},
    {1, 64, fa2::kFwdBlockQ, kFwdBlockKV, 4, kDkvBlockQ, fa2::kDkvBlockKV, 4, fa2::kDqBlockQ, kDqBlockKV, 4},
    {2, 96, fa2::kFwdBlockQ, kFwdBlockKV, 4, kDkvBlockQ, fa2::kDkvBlockKV, 4, fa2::kDqBlockQ, kDqBlockKV, 4},
    {3, 128, fa2::kFwdBlockQ, kFwdBlockKV, 4, kDkvBlockQ, fa2::kDkvBlockKV, 4, fa2::kDqBlockQ, kDqBlockKV, 4},
    {4, 192, fa2::kFwdBlockQ, kFwdBlockKV, 4, kDkvBlockQ, fa2::kDkvBlockKV, 4, fa2::kDqBlockQ, kDqBlockKV, 4},
    {5, 256, fa2::kFwdBlockQ, kFwdBlockKV, 4, kDkvBlockQ, fa2::kDkvBlockKV, 4, fa2::kDqBlockQ, kDqBlockKV, 4},
};
constexpr int kTableRows = sizeof(kTable) / sizeof(kTable[0]);

int pick_config(int headdim) {
  for (int i = 0; i < kTableRows; i++)
    if (headdim <= kTable[i].headdim_padded) return i;
  return -1;
}

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

fa2::Tensor4 tensor(const void *ptr, int64_t sb, int64_t sh, int64_t ss) {
  return fa2::Tensor4{const_cast<void *>(ptr), sb, sh, ss};
}

int launch_status(const char *what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(FA2_ERR_LAUNCH, "%s: %s", what, hipGetErrorString(e));
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
  (void)deterministic;
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

int fa2_fwd(const void *q, const void *k, const void *v, void *o, float *lse, int batch, int nheads,
            int seqlen_q, int seqlen_k, int headdim, int seqlen_q_rounded, int64_t q_sb,
            int64_t q_sh, int64_t q_ss, int64_t k_sb, int64_t k_sh, int64_t k_ss, int64_t v_sb,
            int64_t v_sh, int64_t v_ss, int64_t o_sb, int64_t o_sh, int64_t o_ss,
            float softmax_scale, int dtype, int config_id, void *stream) {
  int rc = check_common(batch, nheads, seqlen_q, seqlen_k, headdim, seqlen_q_rounded, dtype);
  if (rc) return rc;
  fa2::FwdParams p;
  p.q = tensor(q, q_sb, q_sh, q_ss);
  p.k = tensor(k, k_sb, k_sh, k_ss);
  p.v = tensor(v, v_sb, v_sh, v_ss);
  p.o = tensor(o, o_sb, o_sh, o_ss);
  if ((rc = check_tensor("q", p.q)) || (rc = check_tensor("k", p.k)) ||
      (rc = check_tensor("v", p.v)) || (rc = check_tensor("o", p.o)))
    return rc;
  if (lse == nullptr) return fail(FA2_ERR_NULL_POINTER, "lse is NULL");
  if (!(softmax_scale > 0.f) || !std::isfinite(softmax_scale))
    return fail(FA2_ERR_BAD_SHAPE, "softmax_scale must be positive and finite, got %g", (double)softmax_scale);
  int cfg;
  if ((rc = resolve_config(config_id, headdim, &cfg))) return rc;

  p.lse = lse;
  p.batch = batch;
  p.nheads = nheads;
  p.seqlen_q = seqlen_q;
  p.seqlen_k = seqlen_k;
  p.headdim = headdim;
  p.seqlen_q_rounded = seqlen_q_rounded;
  p.n_qtiles = (seqlen_q + fa2::kFwdBlockQ - 1) / fa2::kFwdBlockQ;
  p.scale = softmax_scale;
  p.scale_log2 = softmax_scale * fa2::kLog2e;
  p.vec = vec_ok(p.q, headdim) && vec_ok(p.k, headdim) && vec_ok(p.v, headdim) && vec_ok(p.o, headdim);

  const int64_t nwg = (int64_t)p.n_qtiles * batch * nheads;
  if (nwg > 0x7fffffff) return fail(FA2_ERR_TOO_LARGE, "grid of %lld workgroups too large", (long long)nwg);
  dim3 grid((unsigned)nwg);
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  const int dp = kTable[cfg].headdim_padded;
  fa2::launch_fwd(dtype == FA2_DTYPE_BF16, dp, p, grid, s);
  return launch_status("fa2_fwd launch");
}

int fa2_bwd_preprocess(const void *o, const void *d_o, float *delta, int batch, int nheads,
                       int seqlen_q, int headdim, int seqlen_q_rounded, int64_t o_sb, int64_t o_sh,
                       int64_t o_ss, int64_t do_sb, int64_t do_sh, int64_t do_ss, int dtype,
                       void *stream) {
  int rc = check_common(batch, nheads, seqlen_q, 1, headdim, seqlen_q_rounded, dtype);
  if (rc) return rc;
  fa2::PreParams p;
  p.o = tensor(o, o_sb, o_sh, o_ss);
  p.d_o = tensor(d_o, do_sb, do_sh, do_ss);
  if ((rc = check_tensor("o", p.o)) || (rc = check_tensor("d_o", p.d_o))) return rc;
  if (delta == nullptr) return fail(FA2_ERR_NULL_POINTER, "delta is NULL");
  p.delta = delta;
  p.batch = batch;
  p.nheads = nheads;
  p.seqlen_q = seqlen_q;
  p.headdim = headdim;
  p.seqlen_q_rounded = seqlen_q_rounded;
  p.vec = vec_ok(p.o, headdim) && vec_ok(p.d_o, headdim);
  const int64_t bh = (int64_t)batch * nheads;
  if (bh > 65535) return fail(FA2_ERR_TOO_LARGE, "batch*nheads=%lld exceeds the grid's second dimension", (long long)bh);
  dim3 grid((seqlen_q_rounded + 15) / 16, (unsigned)bh);
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  fa2::launch_preprocess(dtype == FA2_DTYPE_BF16, p, grid, s);
  return launch_status("fa2_bwd_preprocess launch");
}

size_t fa2_bwd_workspace_bytes(int batch, int nheads, int seqlen_q, int seqlen_k, int headdim,
                               int deterministic, int config_id) {
  (void)batch; (void)nheads; (void)seqlen_q; (void)seqlen_k; (void)headdim;
  (void)deterministic; (void)config_id;
  // Both modes currently write dQ exactly once from registers: no accumulation buffer.
  return 0;
}

namespace {

// Shared by fa2_bwd and fa2_bwd_fused.  With `o` given, delta is an output: it is formed by the dQ
// kernel when the fast dQ kernel applies (and the dK/dV kernel then runs second), otherwise by the
// preprocess kernel launched from here.
int bwd_impl(const void *q, const void *k, const void *v, const void *o, const void *d_o,
             const float *lse, float *delta, void *dq, void *dk, void *dv, int batch, int nheads,
             int seqlen_q, int seqlen_k, int headdim, int seqlen_q_rounded, const int64_t *st,
             const int64_t *o_st, float softmax_scale, int dtype, int config_id, void *stream) {
  int rc = check_common(batch, nheads, seqlen_q, seqlen_k, headdim, seqlen_q_rounded, dtype);
  if (rc) return rc;
  const bool fused = o != nullptr;
  fa2::BwdParams p;
  p.q = tensor(q, st[0], st[1], st[2]);
  p.k = tensor(k, st[3], st[4], st[5]);
  p.v = tensor(v, st[6], st[7], st[8]);
  p.d_o = tensor(d_o, st[9], st[10], st[11]);
  p.dq = tensor(dq, st[12], st[13], st[14]);
  p.dk = tensor(dk, st[15], st[16], st[17]);
  p.dv = tensor(dv, st[18], st[19], st[20]);
  p.o = fused ? tensor(o, o_st[0], o_st[1], o_st[2]) : fa2::Tensor4{nullptr, 0, 0, 0};
  // A caller that needs only part of the gradient passes NULL for the rest: dq == NULL skips the
  // dQ kernel, dk == dv == NULL skips the dK/dV kernel.  dk and dv come from one kernel, so they
  // are given or omitted together.
  const bool want_dq = dq != nullptr;
  const bool want_dkdv = dk != nullptr || dv != nullptr;
  if (!want_dq && !want_dkdv) return fail(FA2_ERR_NULL_POINTER, "dq, dk and dv are all NULL");
  if (fused && !(want_dq && want_dkdv))
    return fail(FA2_ERR_NULL_POINTER, "fa2_bwd_fused computes all of dq, dk and dv: none may be NULL");
  if ((rc = check_tensor("q", p.q)) || (rc = check_tensor("k", p.k)) ||
      (rc = check_tensor("v", p.v)) || (rc = check_tensor("d_o", p.d_o)))
    return rc;
  if (fused && (rc = check_tensor("o", p.o))) return rc;
  if (want_dq && (rc = check_tensor("dq", p.dq))) return rc;
  if (want_dkdv && ((rc = check_tensor("dk", p.dk)) || (rc = check_tensor("dv", p.dv)))) return rc;
  if (lse == nullptr) return fail(FA2_ERR_NULL_POINTER, "lse is NULL");
  if (delta == nullptr) return fail(FA2_ERR_NULL_POINTER, "delta is NULL");
  if (!(softmax_scale > 0.f) || !std::isfinite(softmax_scale))
    return fail(FA2_ERR_BAD_SHAPE, "softmax_scale must be positive and finite, got %g", (double)softmax_scale);
  int cfg;
  if ((rc = resolve_config(config_id, headdim, &cfg))) return rc;

  p.lse = lse;
  p.delta = delta;
  p.delta_out = delta;
  p.batch = batch;
  p.nheads = nheads;
  p.seqlen_q = seqlen_q;
  p.seqlen_k = seqlen_k;
  p.headdim = headdim;
  p.seqlen_q_rounded = seqlen_q_rounded;
  p.scale = softmax_scale;
  p.scale_log2 = softmax_scale * fa2::kLog2e;
  p.vec = vec_ok(p.q, headdim) && vec_ok(p.k, headdim) && vec_ok(p.v, headdim) &&
          vec_ok(p.d_o, headdim) && (!want_dq || vec_ok(p.dq, headdim)) &&
          (!want_dkdv || (vec_ok(p.dk, headdim) && vec_ok(p.dv, headdim)));

  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  const int dp = kTable[cfg].headdim_padded;
  const int64_t bh = (int64_t)batch * nheads;

  fa2::BwdParams pk = p, pq = p;
  pk.n_tiles = (seqlen_k + fa2::kDkvBlockKV - 1) / fa2::kDkvBlockKV;
  pq.n_tiles = (seqlen_q + fa2::kDqBlockQ - 1) / fa2::kDqBlockQ;
  const int64_t nwg_k = pk.n_tiles * bh, nwg_q = pq.n_tiles * bh;
  if (nwg_k > 0x7fffffff || nwg_q > 0x7fffffff)
    return fail(FA2_ERR_TOO_LARGE, "grid of %lld workgroups too large", (long long)std::max(nwg_k, nwg_q));

  auto run_dkdv = [&]() {
    dim3 grid((unsigned)nwg_k);
    fa2::launch_dkdv(dtype == FA2_DTYPE_BF16, dp, pk, grid, s);
    return launch_status("fa2_bwd dK/dV launch");
  };

  if (fused && fa2::dq_direct_ok(dp, pq) && vec_ok(p.o, headdim)) {
    // dQ first: it writes delta, which the dK/dV kernel reads.
    dim3 grid((unsigned)nwg_q);
    fa2::launch_dq(dtype == FA2_DTYPE_BF16, dp, pq, grid, true, s);
    if ((rc = launch_status("fa2_bwd_fused dQ launch"))) return rc;
    return run_dkdv();
  }
  if (fused) {
    rc = fa2_bwd_preprocess(o, d_o, delta, batch, nheads, seqlen_q, headdim, seqlen_q_rounded, o_st[0],
                            o_st[1], o_st[2], st[9], st[10], st[11], dtype, stream);
    if (rc) return rc;
  }
  if (want_dkdv && (rc = run_dkdv())) return rc;
  if (want_dq) {
    dim3 grid((unsigned)nwg_q);
    fa2::launch_dq(dtype == FA2_DTYPE_BF16, dp, pq, grid, false, s);
    if ((rc = launch_status("fa2_bwd dQ launch"))) return rc;
  }
  return FA2_OK;
}

}  // namespace

int fa2_bwd(const void *q, const void *k, const void *v, const void *d_o, const float *lse,
            const float *delta, void *workspace, void *dq, void *dk, void *dv, int batch,
            int nheads, int seqlen_q, int seqlen_k, int headdim, int seqlen_q_rounded, int64_t q_sb,
            int64_t q_sh, int64_t q_ss, int64_t k_sb, int64_t k_sh, int64_t k_ss, int64_t v_sb,
            int64_t v_sh, int64_t v_ss, int64_t do_sb, int64_t do_sh, int64_t do_ss, int64_t dq_sb,
            int64_t dq_sh, int64_t dq_ss, int64_t dk_sb, int64_t dk_sh, int64_t dk_ss,
            int64_t dv_sb, int64_t dv_sh, int64_t dv_ss, float softmax_scale, int dtype,
            int deterministic, int config_id, void *stream) {
  (void)workspace;
  (void)deterministic;  // both modes run the same atomic-free kernels
  const int64_t st[21] = {q_sb, q_sh, q_ss, k_sb, k_sh, k_ss, v_sb, v_sh, v_ss, do_sb, do_sh,
                          do_ss, dq_sb, dq_sh, dq_ss, dk_sb, dk_sh, dk_ss, dv_sb, dv_sh, dv_ss};
  return bwd_impl(q, k, v, nullptr, d_o, lse, const_cast<float *>(delta), dq, dk, dv, batch, nheads,
                  seqlen_q, seqlen_k, headdim, seqlen_q_rounded, st, nullptr, softmax_scale, dtype,
                  config_id, stream);
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
  (void)workspace;
  (void)deterministic;
  if (o == nullptr) return fail(FA2_ERR_NULL_POINTER, "o is NULL");
  const int64_t st[21] = {q_sb, q_sh, q_ss, k_sb, k_sh, k_ss, v_sb, v_sh, v_ss, do_sb, do_sh,
                          do_ss, dq_sb, dq_sh, dq_ss, dk_sb, dk_sh, dk_ss, dv_sb, dv_sh, dv_ss};
  const int64_t o_st[3] = {o_sb, o_sh, o_ss};
  return bwd_impl(q, k, v, o, d_o, lse, delta, dq, dk, dv, batch, nheads, seqlen_q, seqlen_k, headdim,
                  seqlen_q_rounded, st, o_st, softmax_scale, dtype, config_id, stream);
}


}  // extern "C"
