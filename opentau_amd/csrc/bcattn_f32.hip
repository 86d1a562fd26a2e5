// Exact fp32 block-causal attention (forward and backward) on the vector ALUs.
//
// This path exists for the fp32 acceptance configuration (relative L2 error of
// 1e-5 against an fp32 CPU evaluation), which no bf16 matrix instruction can
// meet.  It is a plain tiled implementation: a workgroup of 256 threads owns 16
// rows and streams 32-column tiles through LDS; thread (r, c) = (tid/16, tid%16)
// forms the dot products of row r with columns c and c+16, the softmax
// statistics of a row are reduced over its 16 lanes, and the second product is
// accumulated with every thread owning columns c, c+16, ... of the head
// dimension.  Same mask rule, same outputs (O, LSE) and the same zero rows as
// the MFMA kernels.
#include "bcattn_common.h"

namespace bcattn {

constexpr int F_BR = 16;  // rows per workgroup
constexpr int F_BC = 32;  // columns per tile
constexpr int F_MAXX = 16;  // head_dim / 16 <= 16

__device__ __forceinline__ float grp16_max(float v) {
#pragma unroll
  for (int o = 8; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
  return v;
}
__device__ __forceinline__ float grp16_sum(float v) {
#pragma unroll
  for (int o = 8; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}

// Copy `nrows` x D floats (rows row0.. of a (rows, D) strided operand, zero
// beyond `limit`) into LDS with the given pitch.
__device__ __forceinline__ void load_rows_f32(float *dst, int pitch, const float *base, int64_t stride,
                                              int row0, int nrows, int limit, int D, int tid) {
  const int n4 = D / 4;
  for (int idx = tid; idx < nrows * n4; idx += 256) {
    const int row = idx / n4, c4 = idx - row * n4;
    f32x4 v = {0.f, 0.f, 0.f, 0.f};
    if (row0 + row < limit) v = *reinterpret_cast<const f32x4 *>(base + (int64_t)(row0 + row) * stride + 4 * c4);
    float *d = dst + row * pitch + 4 * c4;
    d[0] = v[0], d[1] = v[1], d[2] = v[2], d[3] = v[3];
  }
}

__global__ __launch_bounds__(256) void fwd_f32_kernel(const FwdArgs a, const int D) {
  extern __shared__ __align__(16) float smf[];
  const int KP = D + 1;
  float *Qs = smf;                  // [16][D]
  float *Ks = Qs + F_BR * D;        // [32][D+1]
  float *Vs = Ks + F_BC * KP;       // [32][D]
  float *Ps = Vs + F_BC * D;        // [16][32]
  int *kb_s = reinterpret_cast<int *>(Ps + F_BR * F_BC);  // [32]
  int *red_s = kb_s + F_BC;         // [16]

  const int tid = threadIdx.x;
  const int ri = tid >> 4, cg = tid & 15;
  const int nx = D / 16;
  const int i0 = blockIdx.x * F_BR, h = blockIdx.y, b = blockIdx.z;
  const int hk = h / a.G;
  const int i = i0 + ri;
  const bool rowok = i < a.Sq;
  const bool qv = rowok && a.q_valid[(int64_t)b * a.Sq + (rowok ? i : 0)] != 0;
  const int qb = qv ? a.q_blk[(int64_t)b * a.Sq + i] : kIntMin;

  const float *qbase = reinterpret_cast<const float *>(a.q.ptr) + b * a.q.sb + h * a.q.sh;
  load_rows_f32(Qs, D, qbase, a.q.ss, i0, F_BR, a.Sq, D, tid);
  if (cg == 0) red_s[ri] = qv ? qb : kIntMin;
  __syncthreads();
  int qmax_g = kIntMin;
#pragma unroll
  for (int x = 0; x < F_BR; ++x) qmax_g = max(qmax_g, red_s[x]);

  const int Sk = a.Sk;
  const float *k0b = reinterpret_cast<const float *>(a.k0.ptr) + (b / a.kv_share) * a.k0.sb + hk * a.k0.sh;
  const float *v0b = reinterpret_cast<const float *>(a.v0.ptr) + (b / a.kv_share) * a.v0.sb + hk * a.v0.sh;
  const float *k1b = reinterpret_cast<const float *>(a.k1.ptr) + b * a.k1.sb + hk * a.k1.sh;
  const float *v1b = reinterpret_cast<const float *>(a.v1.ptr) + b * a.v1.sb + hk * a.v1.sh;
  const int nt0s = (a.Sk0 + kSumTile - 1) / kSumTile;  // summary tiles of segment 0
  const tile_summary_t *ksum =
      a.ksum + (int64_t)b * (nt0s + (Sk - a.Sk0 + kSumTile - 1) / kSumTile);

  float oacc[F_MAXX];
#pragma unroll
  for (int x = 0; x < F_MAXX; ++x) oacc[x] = 0.f;
  float m = -INFINITY, l = 0.f;
  const float c = a.scale * kLog2e;

  // The two key segments are walked one after the other; tiles do not straddle them.
  for (int seg = 0; seg < 2; ++seg) {
    const int len = seg ? Sk - a.Sk0 : a.Sk0;
    const int base = seg ? a.Sk0 : 0;
    const float *kseg = seg ? k1b : k0b, *vseg = seg ? v1b : v0b;
    const int64_t kss = seg ? a.k1.ss : a.k0.ss, vss = seg ? a.v1.ss : a.v0.ss;
    for (int j0 = 0; j0 < len; j0 += F_BC) {
      if (ksum[(seg ? nt0s : 0) + j0 / kSumTile].x > qmax_g) continue;  // uniform over the workgroup
      __syncthreads();
      load_rows_f32(Ks, KP, kseg, kss, j0, F_BC, len, D, tid);
      load_rows_f32(Vs, D, vseg, vss, j0, F_BC, len, D, tid);
      if (tid < F_BC) {
        const int j = j0 + tid;
        kb_s[tid] = (j < len && a.k_valid[(int64_t)b * Sk + base + j]) ? a.k_blk[(int64_t)b * Sk + base + j]
                                                                       : kIntMax;
      }
      __syncthreads();
      float s0 = 0.f, s1 = 0.f;
      const float *qr = Qs + ri * D, *kr0 = Ks + cg * KP, *kr1 = Ks + (cg + 16) * KP;
      for (int d = 0; d < D; ++d) {
        const float qd = qr[d];
        s0 = fmaf(qd, kr0[d], s0);
        s1 = fmaf(qd, kr1[d], s1);
      }
      if (!qv || kb_s[cg] > qb) s0 = -INFINITY;
      if (!qv || kb_s[cg + 16] > qb) s1 = -INFINITY;
      const float mloc = grp16_max(fmaxf(s0, s1));
      const float mnew = fmaxf(m, mloc);
      const float moff = (mnew == -INFINITY) ? 0.f : mnew * c;
      const float corr = fast_exp2(m * c - moff);
      const float p0 = fast_exp2(s0 * c - moff), p1 = fast_exp2(s1 * c - moff);
      l = l * corr + grp16_sum(p0 + p1);
      m = mnew;
      Ps[ri * F_BC + cg] = p0;
      Ps[ri * F_BC + cg + 16] = p1;
      __syncthreads();
#pragma unroll
      for (int x = 0; x < F_MAXX; ++x)
        if (x < nx) {
          float acc = oacc[x] * corr;
          const float *vcol = Vs + cg + 16 * x;
          const float *pr = Ps + ri * F_BC;
          for (int j = 0; j < F_BC; ++j) acc = fmaf(pr[j], vcol[j * D], acc);
          oacc[x] = acc;
        }
    }
  }

  if (rowok) {
    const bool has = qv && l > 0.f;
    const float inv = has ? 1.f / l : 0.f;
    float *optr = reinterpret_cast<float *>(a.o) + b * a.o_sb + (int64_t)i * a.o_ss + h * a.o_sh;
#pragma unroll
    for (int x = 0; x < F_MAXX; ++x)
      if (x < nx) optr[cg + 16 * x] = oacc[x] * inv;
    if (a.lse != nullptr && cg == 0)
      a.lse[((int64_t)b * a.H + h) * a.Sq + i] = has ? m * a.scale + logf(l) : 0.f;
  }
}

static size_t fwd_f32_smem(int D) {
  return sizeof(float) * ((size_t)F_BR * D + F_BC * (D + 1) + F_BC * D + F_BR * F_BC + F_BC + F_BR);
}

int launch_fwd_f32(const FwdArgs &a, int D, hipStream_t st) {
  const size_t smem = fwd_f32_smem(D);
  if (!allow_dynamic_lds<&fwd_f32_kernel>((int)fwd_f32_smem(256)))
    return BCATTN_ERR_LAUNCH;
  hipLaunchKernelGGL(fwd_f32_kernel, dim3((a.Sq + F_BR - 1) / F_BR, a.H, a.B), dim3(256), smem, st, a, D);
  return hipGetLastError() == hipSuccess ? BCATTN_OK : BCATTN_ERR_LAUNCH;
}

// ---- backward --------------------------------------------------------------------
__global__ __launch_bounds__(256) void bwd_delta_f32_kernel(const BwdArgs a, const int D) {
  const int64_t total = (int64_t)a.B * a.Sq * a.H;
  const int64_t row = (int64_t)blockIdx.x * 16 + (threadIdx.x >> 4);
  const int cg = threadIdx.x & 15;
  float acc = 0.f;
  int h = 0, i = 0, b = 0;
  if (row < total) {
    h = (int)(row % a.H);
    i = (int)((row / a.H) % a.Sq);
    b = (int)(row / ((int64_t)a.H * a.Sq));
    const float *op = reinterpret_cast<const float *>(a.o.ptr) + b * a.o.sb + (int64_t)i * a.o.ss + h * a.o.sh;
    const float *gp =
        reinterpret_cast<const float *>(a.d_o.ptr) + b * a.d_o.sb + (int64_t)i * a.d_o.ss + h * a.d_o.sh;
    for (int d = cg; d < D; d += 16) acc = fmaf(op[d], gp[d], acc);
  }
  acc = grp16_sum(acc);
  if (row < total && cg == 0) a.delta[((int64_t)b * a.H + h) * a.Sq + i] = acc;
}

__global__ __launch_bounds__(256) void bwd_dq_f32_kernel(const BwdArgs a, const int D) {
  extern __shared__ __align__(16) float smf[];
  const int KP = D + 1;
  float *Qs = smf;                 // [16][D]
  float *Gs = Qs + F_BR * D;       // [16][D]
  float *Ks = Gs + F_BR * D;       // [32][D+1]
  float *Vs = Ks + F_BC * KP;      // [32][D+1]
  float *Ss = Vs + F_BC * KP;      // [16][32] dS
  int *kb_s = reinterpret_cast<int *>(Ss + F_BR * F_BC);
  int *red_s = kb_s + F_BC;

  const int tid = threadIdx.x;
  const int ri = tid >> 4, cg = tid & 15;
  const int nx = D / 16;
  const int i0 = blockIdx.x * F_BR, h = blockIdx.y, b = blockIdx.z;
  const int hk = h / a.G;
  const int i = i0 + ri;
  const bool rowok = i < a.Sq;
  const bool qv = rowok && a.q_valid[(int64_t)b * a.Sq + (rowok ? i : 0)] != 0;
  const int qb = qv ? a.q_blk[(int64_t)b * a.Sq + i] : kIntMin;
  const int64_t stat = ((int64_t)b * a.H + h) * a.Sq + (rowok ? i : 0);
  const float lse2 = qv ? a.lse[stat] * kLog2e : INFINITY;
  const float delta = qv ? a.delta[stat] : 0.f;

  load_rows_f32(Qs, D, reinterpret_cast<const float *>(a.q.ptr) + b * a.q.sb + h * a.q.sh, a.q.ss, i0, F_BR,
                a.Sq, D, tid);
  load_rows_f32(Gs, D, reinterpret_cast<const float *>(a.d_o.ptr) + b * a.d_o.sb + h * a.d_o.sh, a.d_o.ss,
                i0, F_BR, a.Sq, D, tid);
  if (cg == 0) red_s[ri] = qv ? qb : kIntMin;
  __syncthreads();
  int qmax_g = kIntMin;
#pragma unroll
  for (int x = 0; x < F_BR; ++x) qmax_g = max(qmax_g, red_s[x]);

  const int Sk = a.Sk;
  const float *kb_ = reinterpret_cast<const float *>(a.k.ptr) + b * a.k.sb + hk * a.k.sh;
  const float *vb_ = reinterpret_cast<const float *>(a.v.ptr) + b * a.v.sb + hk * a.v.sh;
  const tile_summary_t *ksum = a.ksum + (int64_t)b * ((Sk + kSumTile - 1) / kSumTile);
  float acc[F_MAXX];
#pragma unroll
  for (int x = 0; x < F_MAXX; ++x) acc[x] = 0.f;
  const float c = a.scale * kLog2e;

  const int nt = (Sk + F_BC - 1) / F_BC;
  for (int t = 0; t < nt; ++t) {
    if (ksum[(t * F_BC) / kSumTile].x > qmax_g) continue;
    const int j0 = t * F_BC;
    __syncthreads();
    load_rows_f32(Ks, KP, kb_, a.k.ss, j0, F_BC, Sk, D, tid);
    load_rows_f32(Vs, KP, vb_, a.v.ss, j0, F_BC, Sk, D, tid);
    if (tid < F_BC) {
      const int j = j0 + tid;
      kb_s[tid] = (j < Sk && a.k_valid[(int64_t)b * Sk + j]) ? a.k_blk[(int64_t)b * Sk + j] : kIntMax;
    }
    __syncthreads();
    float s0 = 0.f, s1 = 0.f, d0 = 0.f, d1 = 0.f;
    const float *qr = Qs + ri * D, *gr = Gs + ri * D;
    const float *kr0 = Ks + cg * KP, *kr1 = Ks + (cg + 16) * KP;
    const float *vr0 = Vs + cg * KP, *vr1 = Vs + (cg + 16) * KP;
    for (int d = 0; d < D; ++d) {
      const float qd = qr[d], gd = gr[d];
      s0 = fmaf(qd, kr0[d], s0);
      s1 = fmaf(qd, kr1[d], s1);
      d0 = fmaf(gd, vr0[d], d0);
      d1 = fmaf(gd, vr1[d], d1);
    }
    float p0 = fast_exp2(s0 * c - lse2), p1 = fast_exp2(s1 * c - lse2);
    if (kb_s[cg] > qb) p0 = 0.f;
    if (kb_s[cg + 16] > qb) p1 = 0.f;
    Ss[ri * F_BC + cg] = p0 * (d0 - delta);
    Ss[ri * F_BC + cg + 16] = p1 * (d1 - delta);
    __syncthreads();
#pragma unroll
    for (int x = 0; x < F_MAXX; ++x)
      if (x < nx) {
        float v = acc[x];
        const float *kcol = Ks + cg + 16 * x;
        const float *sr = Ss + ri * F_BC;
        for (int j = 0; j < F_BC; ++j) v = fmaf(sr[j], kcol[j * KP], v);
        acc[x] = v;
      }
  }
  if (rowok) {
    float *optr = reinterpret_cast<float *>(a.dq) + b * a.dq_sb + (int64_t)i * a.dq_ss + h * a.dq_sh;
#pragma unroll
    for (int x = 0; x < F_MAXX; ++x)
      if (x < nx) optr[cg + 16 * x] = acc[x] * a.scale;
  }
}

__global__ __launch_bounds__(256) void bwd_dkv_f32_kernel(const BwdArgs a, const int D) {
  extern __shared__ __align__(16) float smf[];
  const int KP = D + 1;
  float *Ks = smf;                 // [16][D]
  float *Vs = Ks + F_BR * D;       // [16][D]
  float *Qs = Vs + F_BR * D;       // [32][D+1]
  float *Gs = Qs + F_BC * KP;      // [32][D+1]
  float *Ps = Gs + F_BC * KP;      // [16][32]
  float *Ss = Ps + F_BR * F_BC;    // [16][32]
  float *lse_s = Ss + F_BR * F_BC; // [32]
  float *del_s = lse_s + F_BC;     // [32]
  int *qb_s = reinterpret_cast<int *>(del_s + F_BC);  // [32]
  int *red_s = qb_s + F_BC;        // [16]

  const int tid = threadIdx.x;
  const int ki = tid >> 4, cg = tid & 15;
  const int nx = D / 16;
  const int j0 = blockIdx.x * F_BR, hk = blockIdx.y, b = blockIdx.z;
  const int Sk = a.Sk, Sq = a.Sq;
  const int j = j0 + ki;
  const bool jok = j < Sk;
  const bool kv = jok && a.k_valid[(int64_t)b * Sk + (jok ? j : 0)] != 0;
  const int kb = kv ? a.k_blk[(int64_t)b * Sk + j] : kIntMax;

  load_rows_f32(Ks, D, reinterpret_cast<const float *>(a.k.ptr) + b * a.k.sb + hk * a.k.sh, a.k.ss, j0, F_BR,
                Sk, D, tid);
  load_rows_f32(Vs, D, reinterpret_cast<const float *>(a.v.ptr) + b * a.v.sb + hk * a.v.sh, a.v.ss, j0, F_BR,
                Sk, D, tid);
  if (cg == 0) red_s[ki] = kb;
  __syncthreads();
  int kmin_g = kIntMax;
#pragma unroll
  for (int x = 0; x < F_BR; ++x) kmin_g = min(kmin_g, red_s[x]);

  const tile_summary_t *qsum = a.qsum + (int64_t)b * ((Sq + kSumTile - 1) / kSumTile);
  float dk[F_MAXX], dv[F_MAXX];
#pragma unroll
  for (int x = 0; x < F_MAXX; ++x) dk[x] = 0.f, dv[x] = 0.f;
  const float c = a.scale * kLog2e;
  const int nqt = (Sq + F_BC - 1) / F_BC;

  if (kmin_g != kIntMax) {
    for (int g = 0; g < a.G; ++g) {
      const int h = hk * a.G + g;
      const float *qb_ = reinterpret_cast<const float *>(a.q.ptr) + b * a.q.sb + h * a.q.sh;
      const float *gb_ = reinterpret_cast<const float *>(a.d_o.ptr) + b * a.d_o.sb + h * a.d_o.sh;
      for (int qt = 0; qt < nqt; ++qt) {
        const tile_summary_t sm = qsum[(qt * F_BC) / kSumTile];
        if (sm.w == 0 || sm.y < kmin_g) continue;
        const int i0 = qt * F_BC;
        __syncthreads();
        load_rows_f32(Qs, KP, qb_, a.q.ss, i0, F_BC, Sq, D, tid);
        load_rows_f32(Gs, KP, gb_, a.d_o.ss, i0, F_BC, Sq, D, tid);
        if (tid < F_BC) {
          const int i = i0 + tid;
          float lv = INFINITY, dl = 0.f;
          int qv = kIntMin;
          if (i < Sq && a.q_valid[(int64_t)b * Sq + i]) {
            const int64_t stat = ((int64_t)b * a.H + h) * Sq + i;
            lv = a.lse[stat] * kLog2e;
            dl = a.delta[stat];
            qv = a.q_blk[(int64_t)b * Sq + i];
          }
          lse_s[tid] = lv, del_s[tid] = dl, qb_s[tid] = qv;
        }
        __syncthreads();
        float s0 = 0.f, s1 = 0.f, d0 = 0.f, d1 = 0.f;
        const float *kr = Ks + ki * D, *vr = Vs + ki * D;
        const float *qr0 = Qs + cg * KP, *qr1 = Qs + (cg + 16) * KP;
        const float *gr0 = Gs + cg * KP, *gr1 = Gs + (cg + 16) * KP;
        for (int d = 0; d < D; ++d) {
          const float kd = kr[d], vd = vr[d];
          s0 = fmaf(kd, qr0[d], s0);
          s1 = fmaf(kd, qr1[d], s1);
          d0 = fmaf(vd, gr0[d], d0);
          d1 = fmaf(vd, gr1[d], d1);
        }
        float p0 = fast_exp2(s0 * c - lse_s[cg]), p1 = fast_exp2(s1 * c - lse_s[cg + 16]);
        if (kb > qb_s[cg]) p0 = 0.f;
        if (kb > qb_s[cg + 16]) p1 = 0.f;
        Ps[ki * F_BC + cg] = p0;
        Ps[ki * F_BC + cg + 16] = p1;
        Ss[ki * F_BC + cg] = p0 * (d0 - del_s[cg]);
        Ss[ki * F_BC + cg + 16] = p1 * (d1 - del_s[cg + 16]);
        __syncthreads();
#pragma unroll
        for (int x = 0; x < F_MAXX; ++x)
          if (x < nx) {
            float av = dv[x], ak = dk[x];
            const float *gcol = Gs + cg + 16 * x, *qcol = Qs + cg + 16 * x;
            const float *pr = Ps + ki * F_BC, *sr = Ss + ki * F_BC;
            for (int q = 0; q < F_BC; ++q) {
              av = fmaf(pr[q], gcol[q * KP], av);
              ak = fmaf(sr[q], qcol[q * KP], ak);
            }
            dv[x] = av, dk[x] = ak;
          }
      }
    }
  }
  if (jok) {
    float *dkp = reinterpret_cast<float *>(a.dk) + b * a.dk_sb + (int64_t)j * a.dk_ss + hk * a.dk_sh;
    float *dvp = reinterpret_cast<float *>(a.dv) + b * a.dv_sb + (int64_t)j * a.dv_ss + hk * a.dv_sh;
#pragma unroll
    for (int x = 0; x < F_MAXX; ++x)
      if (x < nx) {
        dkp[cg + 16 * x] = dk[x] * a.scale;
        dvp[cg + 16 * x] = dv[x];
      }
  }
}

static size_t dq_f32_smem(int D) {
  return sizeof(float) * ((size_t)2 * F_BR * D + 2 * F_BC * (D + 1) + F_BR * F_BC + F_BC + F_BR);
}
static size_t dkv_f32_smem(int D) {
  return sizeof(float) * ((size_t)2 * F_BR * D + 2 * F_BC * (D + 1) + 2 * F_BR * F_BC + 3 * F_BC + F_BR);
}

int launch_bwd_f32(const BwdArgs &a, int D, hipStream_t st) {
  if (!allow_dynamic_lds<&bwd_dq_f32_kernel>((int)dq_f32_smem(256)) ||
      !allow_dynamic_lds<&bwd_dkv_f32_kernel>((int)dkv_f32_smem(256)))
    return BCATTN_ERR_LAUNCH;
  const int64_t rows = (int64_t)a.B * a.Sq * a.H;
  if (a.stages & BCATTN_BWD_DELTA)
    hipLaunchKernelGGL(bwd_delta_f32_kernel, dim3((unsigned)((rows + 15) / 16)), dim3(256), 0, st, a, D);
  if (a.stages & BCATTN_BWD_DQ)
    hipLaunchKernelGGL(bwd_dq_f32_kernel, dim3((a.Sq + F_BR - 1) / F_BR, a.H, a.B), dim3(256), dq_f32_smem(D),
                     st, a, D);
  if (a.stages & BCATTN_BWD_DKV)
    hipLaunchKernelGGL(bwd_dkv_f32_kernel, dim3((a.Sk + F_BR - 1) / F_BR, a.Hkv, a.B), dim3(256),
                     dkv_f32_smem(D), st, a, D);
  return hipGetLastError() == hipSuccess ? BCATTN_OK : BCATTN_ERR_LAUNCH;
}

}  // namespace bcattn
