// C ABI of libbcattn: argument checks, workspace layout, dispatch.
#include <stdarg.h>
#include <stdio.h>
#include <string.h>

#include "bcattn_common.h"

namespace bcattn {

static thread_local char g_err[512] = "";

static int fail(int code, const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

// ---- key / query tile summaries ------------------------------------------------
__global__ __launch_bounds__(64) void summary_kernel(const int32_t *blk, const uint8_t *valid, int S,
                                                     int ntile, tile_summary_t *out) {
  const int t = blockIdx.x, b = blockIdx.y, lane = threadIdx.x;
  const int j = t * kSumTile + lane;
  const bool ok = j < S && valid[(int64_t)b * S + j] != 0;
  const int id = ok ? blk[(int64_t)b * S + j] : 0;
  const int mn = wave_min_i(ok ? id : kIntMax);
  const int mx = wave_max_i(ok ? id : kIntMin);
  const int cnt = wave_sum_i(ok ? 1 : 0);
  if (lane == 0) {
    tile_summary_t s;
    s.x = mn;
    s.y = mx;
    s.z = cnt == kSumTile ? 1 : 0;
    s.w = cnt;
    out[(int64_t)b * ntile + t] = s;
  }
}

int launch_summary(const int32_t *blk, const uint8_t *valid, int B, int S, tile_summary_t *out,
                   hipStream_t st) {
  const int ntile = (S + kSumTile - 1) / kSumTile;
  hipLaunchKernelGGL(summary_kernel, dim3(ntile, B), dim3(64), 0, st, blk, valid, S, ntile, out);
  return hipGetLastError() == hipSuccess ? BCATTN_OK : BCATTN_ERR_LAUNCH;
}

static size_t align256(size_t x) { return (x + 255) & ~(size_t)255; }
static size_t summary_bytes(int B, int S) {
  return align256((size_t)B * ((S + kSumTile - 1) / kSumTile) * sizeof(tile_summary_t));
}

static bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

static int check_tensor(const char *name, const bcattn_tensor &t, int vec, bool required) {
  if (t.ptr == nullptr) {
    if (required) return fail(BCATTN_ERR_INVALID, "%s: null pointer", name);
    return BCATTN_OK;
  }
  if (!aligned16(t.ptr)) return fail(BCATTN_ERR_INVALID, "%s: pointer not 16-byte aligned", name);
  if (t.stride_b % vec || t.stride_s % vec || t.stride_h % vec)
    return fail(BCATTN_ERR_INVALID, "%s: strides must be multiples of %d elements", name, vec);
  return BCATTN_OK;
}

static int check_common(int B, int Sq, int Sk, int H, int Hkv, int D, int dtype, float scale) {
  if (B < 0 || Sq <= 0 || Sk <= 0 || H <= 0 || Hkv <= 0)
    return fail(BCATTN_ERR_INVALID, "bad shape B=%d Sq=%d Sk=%d H=%d Hkv=%d", B, Sq, Sk, H, Hkv);
  if (H % Hkv) return fail(BCATTN_ERR_INVALID, "H=%d is not a multiple of Hkv=%d", H, Hkv);
  if (!(scale > 0.f)) return fail(BCATTN_ERR_INVALID, "scale must be positive");
  if (dtype == BCATTN_BF16) {
    if (D != 64 && D != 128 && D != 256)
      return fail(BCATTN_ERR_UNSUPPORTED, "bf16 kernels cover head_dim 64, 128, 256; got %d", D);
  } else if (dtype == BCATTN_F32) {
    if (D % 32 || D <= 0 || D > 256)
      return fail(BCATTN_ERR_UNSUPPORTED, "fp32 kernels need head_dim %% 32 == 0 and <= 256; got %d", D);
  } else {
    return fail(BCATTN_ERR_UNSUPPORTED, "dtype %d not supported (0 = fp32, 1 = bf16)", dtype);
  }
  if ((int64_t)(H / Hkv) * Sq > 0x3fffffff) return fail(BCATTN_ERR_INVALID, "G*Sq too large");
  return BCATTN_OK;
}

static TensorArg targ(const bcattn_tensor &t) {
  return TensorArg{t.ptr, t.stride_b, t.stride_s, t.stride_h};
}

static int check_fwd(const bcattn_fwd_params *p) {
  if (p == nullptr) return fail(BCATTN_ERR_INVALID, "null params");
  if (p->Sk0 < 0 || p->Sk1 < 0) return fail(BCATTN_ERR_INVALID, "negative key segment length");
  int rc = check_common(p->B, p->Sq, p->Sk0 + p->Sk1, p->H, p->Hkv, p->D, p->dtype, p->scale);
  if (rc) return rc;
  const int vec = p->dtype == BCATTN_BF16 ? 8 : 4;
  if ((rc = check_tensor("q", p->q, vec, true))) return rc;
  if ((rc = check_tensor("k", p->k, vec, p->Sk0 > 0))) return rc;
  if ((rc = check_tensor("v", p->v, vec, p->Sk0 > 0))) return rc;
  if ((rc = check_tensor("k1", p->k1, vec, p->Sk1 > 0))) return rc;
  if ((rc = check_tensor("v1", p->v1, vec, p->Sk1 > 0))) return rc;
  if ((rc = check_tensor("o", p->o, vec, true))) return rc;
  if (!p->q_blk || !p->k_blk || !p->q_valid || !p->k_valid)
    return fail(BCATTN_ERR_INVALID, "null block-id / valid pointer");
  return BCATTN_OK;
}

static FwdArgs fwd_args(const bcattn_fwd_params *p) {
  FwdArgs a;
  a.q = targ(p->q);
  a.k0 = targ(p->Sk0 > 0 ? p->k : p->k1);
  a.v0 = targ(p->Sk0 > 0 ? p->v : p->v1);
  a.k1 = targ(p->Sk1 > 0 ? p->k1 : p->k);
  a.v1 = targ(p->Sk1 > 0 ? p->v1 : p->v);
  a.o = p->o.ptr;
  a.o_sb = p->o.stride_b;
  a.o_ss = p->o.stride_s;
  a.o_sh = p->o.stride_h;
  a.lse = p->lse;
  a.q_blk = p->q_blk;
  a.k_blk = p->k_blk;
  a.q_valid = p->q_valid;
  a.k_valid = p->k_valid;
  a.ksum = nullptr;
  a.B = p->B;
  a.Sq = p->Sq;
  a.Sk0 = p->Sk0;
  a.Sk = p->Sk0 + p->Sk1;
  a.H = p->H;
  a.Hkv = p->Hkv;
  a.G = p->H / p->Hkv;
  a.scale = p->scale;
  return a;
}

}  // namespace bcattn

using namespace bcattn;

extern "C" {

int bcattn_abi_version(void) { return BCATTN_ABI_VERSION; }

const char *bcattn_last_error(void) { return g_err; }

size_t bcattn_fwd_workspace_bytes(const bcattn_fwd_params *p) {
  if (p == nullptr || p->B <= 0) return 0;
  return summary_bytes(p->B, p->Sk0 + p->Sk1);
}

size_t bcattn_fwd_kvcache_workspace_bytes(const bcattn_fwd_params *p) {
  if (p == nullptr || p->B <= 0) return 0;
  int ns = 0;
  return summary_bytes(p->B, p->Sk0 + p->Sk1) +
         kvcache_workspace_bytes(p->B, p->Sq, p->Sk0 + p->Sk1, p->H, p->Hkv, p->D, &ns);
}

size_t bcattn_bwd_workspace_bytes(const bcattn_bwd_params *p) {
  if (p == nullptr || p->B <= 0) return 0;
  return summary_bytes(p->B, p->Sk) + summary_bytes(p->B, p->Sq) +
         align256((size_t)p->B * p->H * p->Sq * sizeof(float));
}

int bcattn_fwd(const bcattn_fwd_params *p, void *stream) {
  int rc = check_fwd(p);
  if (rc) return rc;
  if (p->B == 0) return BCATTN_OK;
  const size_t need = bcattn_fwd_workspace_bytes(p);
  if (p->workspace == nullptr || p->workspace_bytes < need || !aligned16(p->workspace))
    return fail(BCATTN_ERR_WORKSPACE, "forward needs %zu bytes of 16-byte aligned workspace, got %zu",
                need, p->workspace ? p->workspace_bytes : (size_t)0);
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  FwdArgs a = fwd_args(p);
  tile_summary_t *ks = reinterpret_cast<tile_summary_t *>(p->workspace);
  if (!p->summary_ready) {
    rc = launch_summary(p->k_blk, p->k_valid, a.B, a.Sk, ks, st);
    if (rc) return fail(rc, "summary launch failed: %s", hipGetErrorString(hipGetLastError()));
  }
  a.ksum = ks;
  rc = p->dtype == BCATTN_BF16 ? launch_fwd_bf16(a, p->D, st) : launch_fwd_f32(a, p->D, st);
  if (rc) return fail(rc, "forward launch failed (D=%d dtype=%d)", p->D, p->dtype);
  return BCATTN_OK;
}

int bcattn_fwd_kvcache(const bcattn_fwd_params *p, void *stream) {
  int rc = check_fwd(p);
  if (rc) return rc;
  if (p->B == 0) return BCATTN_OK;
  if (p->dtype != BCATTN_BF16) return bcattn_fwd(p, stream);
  const size_t need = bcattn_fwd_kvcache_workspace_bytes(p);
  if (p->workspace == nullptr || p->workspace_bytes < need || !aligned16(p->workspace))
    return fail(BCATTN_ERR_WORKSPACE, "kvcache forward needs %zu bytes of 16-byte aligned workspace, got %zu",
                need, p->workspace ? p->workspace_bytes : (size_t)0);
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  FwdArgs a = fwd_args(p);
  char *ws = reinterpret_cast<char *>(p->workspace);
  tile_summary_t *ks = reinterpret_cast<tile_summary_t *>(ws);
  if (!p->summary_ready) {
    rc = launch_summary(p->k_blk, p->k_valid, a.B, a.Sk, ks, st);
    if (rc) return fail(rc, "summary launch failed: %s", hipGetErrorString(hipGetLastError()));
  }
  a.ksum = ks;
  ws += summary_bytes(a.B, a.Sk);
  SplitArgs s;
  const size_t part = kvcache_workspace_bytes(a.B, a.Sq, a.Sk, a.H, a.Hkv, p->D, &s.nsplit);
  const size_t R = (size_t)a.G * a.Sq;
  s.part_o = reinterpret_cast<float *>(ws);
  s.part_ml = s.part_o + (size_t)a.B * a.Hkv * s.nsplit * R * p->D;
  (void)part;
  rc = launch_fwd_kvcache_bf16(a, s, p->D, st);
  if (rc) return fail(rc, "kvcache forward launch failed (D=%d)", p->D);
  return BCATTN_OK;
}

int bcattn_bwd(const bcattn_bwd_params *p, void *stream) {
  if (p == nullptr) return fail(BCATTN_ERR_INVALID, "null params");
  int rc = check_common(p->B, p->Sq, p->Sk, p->H, p->Hkv, p->D, p->dtype, p->scale);
  if (rc) return rc;
  const int vec = p->dtype == BCATTN_BF16 ? 8 : 4;
  const struct {
    const char *n;
    const bcattn_tensor *t;
  } ts[] = {{"q", &p->q},   {"k", &p->k},   {"v", &p->v},   {"o", &p->o},
            {"d_o", &p->d_o}, {"dq", &p->dq}, {"dk", &p->dk}, {"dv", &p->dv}};
  for (auto &e : ts)
    if ((rc = check_tensor(e.n, *e.t, vec, true))) return rc;
  if (!p->lse || !p->q_blk || !p->k_blk || !p->q_valid || !p->k_valid)
    return fail(BCATTN_ERR_INVALID, "null lse / block-id / valid pointer");
  if (p->B == 0) return BCATTN_OK;
  const size_t need = bcattn_bwd_workspace_bytes(p);
  if (p->workspace == nullptr || p->workspace_bytes < need || !aligned16(p->workspace))
    return fail(BCATTN_ERR_WORKSPACE, "backward needs %zu bytes of 16-byte aligned workspace, got %zu",
                need, p->workspace ? p->workspace_bytes : (size_t)0);
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  BwdArgs a;
  a.q = targ(p->q);
  a.k = targ(p->k);
  a.v = targ(p->v);
  a.o = targ(p->o);
  a.d_o = targ(p->d_o);
  a.dq = p->dq.ptr;
  a.dq_sb = p->dq.stride_b, a.dq_ss = p->dq.stride_s, a.dq_sh = p->dq.stride_h;
  a.dk = p->dk.ptr;
  a.dk_sb = p->dk.stride_b, a.dk_ss = p->dk.stride_s, a.dk_sh = p->dk.stride_h;
  a.dv = p->dv.ptr;
  a.dv_sb = p->dv.stride_b, a.dv_ss = p->dv.stride_s, a.dv_sh = p->dv.stride_h;
  a.lse = p->lse;
  a.q_blk = p->q_blk, a.k_blk = p->k_blk, a.q_valid = p->q_valid, a.k_valid = p->k_valid;
  a.B = p->B, a.Sq = p->Sq, a.Sk = p->Sk, a.H = p->H, a.Hkv = p->Hkv, a.G = p->H / p->Hkv;
  a.scale = p->scale;
  a.stages = p->stages & (BCATTN_BWD_DELTA | BCATTN_BWD_DQ | BCATTN_BWD_DKV);
  if (a.stages == 0) a.stages = BCATTN_BWD_DELTA | BCATTN_BWD_DQ | BCATTN_BWD_DKV;
  char *ws = reinterpret_cast<char *>(p->workspace);
  tile_summary_t *ks = reinterpret_cast<tile_summary_t *>(ws);
  ws += summary_bytes(a.B, a.Sk);
  tile_summary_t *qs = reinterpret_cast<tile_summary_t *>(ws);
  ws += summary_bytes(a.B, a.Sq);
  a.delta = reinterpret_cast<float *>(ws);
  a.ksum = ks;
  a.qsum = qs;
  if (!p->summary_ready &&
      ((rc = launch_summary(p->k_blk, p->k_valid, a.B, a.Sk, ks, st)) ||
       (rc = launch_summary(p->q_blk, p->q_valid, a.B, a.Sq, qs, st))))
    return fail(rc, "summary launch failed");
  rc = p->dtype == BCATTN_BF16 ? launch_bwd_bf16(a, p->D, st) : launch_bwd_f32(a, p->D, st);
  if (rc) return fail(rc, "backward launch failed (D=%d dtype=%d)", p->D, p->dtype);
  return BCATTN_OK;
}

}  // extern "C"
