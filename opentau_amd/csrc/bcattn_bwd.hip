// Block-causal attention backward, bf16 in / fp32 accumulate, gfx950 MFMA.
//
// Three kernels, no atomics, so gradients are bit-repeatable:
//   delta   delta[b,h,i] = sum_d O*dO
//   dQ      a workgroup owns 128 packed query rows and streams key tiles;
//           dQ^T = K^T dS^T with dS^T = P^T o (dP^T - delta), all keys x queries
//   dK/dV   a workgroup owns 128 keys of one kv head and streams the query tiles
//           of every query head of its group, so the sum over the GQA group
//           happens in registers; dV^T = dO^T P, dK^T = Q^T dS (queries x keys)
// P is recomputed from the saved log-sum-exp: P = exp2(scale*log2e*S - log2e*LSE).
//
// As in the forward, the 32x32 accumulator of the first product is already the B
// operand of the second, so P / dS never leave registers; the operand that must
// be contracted over the sequence axis (K^T, Q^T, dO^T) is kept in LDS as a
// transposed tile next to the row tile.
#include "bcattn_common.h"

namespace bcattn {

// ---- tile movers -------------------------------------------------------------
// A 64 x D tile is moved as 16*(D/8) units of 4 rows x 8 columns: four 16-byte
// global loads per unit, then four 16-byte row stores and/or eight 8-byte
// transposed stores.
template <int D>
struct TileUnits {
  static constexpr int CPR = D / 8;
  static constexpr int UNITS = 16 * CPR;
  static constexpr int NU = (UNITS + 255) / 256;
};

template <int D>
__device__ __forceinline__ void load_units(bf16x8 (&reg)[TileUnits<D>::NU][4], const bf16_t *base,
                                           int64_t row_stride, int row0, int nrows, int tid) {
  using T = TileUnits<D>;
#pragma unroll
  for (int it = 0; it < T::NU; ++it) {
    const int u = min(tid + 256 * it, T::UNITS - 1);
    const int dch = u % T::CPR, kg = u / T::CPR;
#pragma unroll
    for (int x = 0; x < 4; ++x) {
      const int row = row0 + 4 * kg + x, rc = min(row, nrows - 1);
      const bf16x8 val = *reinterpret_cast<const bf16x8 *>(base + (int64_t)rc * row_stride + dch * 8);
      reg[it][x] = keep_if(row < nrows, val);
    }
  }
}

template <int D, bool ROWS, bool TRANS>
__device__ __forceinline__ void store_units(const bf16x8 (&reg)[TileUnits<D>::NU][4], bf16_t *rows,
                                            bf16_t *trans, int tid) {
  using T = TileUnits<D>;
  constexpr int KP = RowTile<D>::kPitch;
#pragma unroll
  for (int it = 0; it < T::NU; ++it) {
    const int u = tid + 256 * it;
    const int dch = u % T::CPR, kg = u / T::CPR;
    if (u < T::UNITS) {
      if (ROWS) {
#pragma unroll
        for (int x = 0; x < 4; ++x)
          *reinterpret_cast<bf16x8 *>(rows + (4 * kg + x) * KP + dch * 8) = reg[it][x];
      }
      if (TRANS) tr_store_4x8(trans, 8 * dch, kg, reg[it][0], reg[it][1], reg[it][2], reg[it][3]);
    }
  }
}

// ---- delta ---------------------------------------------------------------------
template <int D>
__global__ __launch_bounds__(256) void bwd_delta_kernel(const BwdArgs a) {
  constexpr int LPR = D / 8;
  constexpr int RPB = 256 / LPR;
  const int64_t total = (int64_t)a.B * a.Sq * a.H;
  const int64_t row = (int64_t)blockIdx.x * RPB + threadIdx.x / LPR;
  const int c = threadIdx.x % LPR;
  float acc = 0.f;
  int h = 0, i = 0, b = 0;
  if (row < total) {
    h = (int)(row % a.H);
    i = (int)((row / a.H) % a.Sq);
    b = (int)(row / ((int64_t)a.H * a.Sq));
    const bf16x8 ov = *reinterpret_cast<const bf16x8 *>(
        reinterpret_cast<const bf16_t *>(a.o.ptr) + b * a.o.sb + (int64_t)i * a.o.ss + h * a.o.sh + 8 * c);
    const bf16x8 gv = *reinterpret_cast<const bf16x8 *>(reinterpret_cast<const bf16_t *>(a.d_o.ptr) +
                                                        b * a.d_o.sb + (int64_t)i * a.d_o.ss +
                                                        h * a.d_o.sh + 8 * c);
#pragma unroll
    for (int e = 0; e < 8; ++e) acc += (float)ov[e] * (float)gv[e];
  }
#pragma unroll
  for (int o = LPR / 2; o > 0; o >>= 1) acc += __shfl_xor(acc, o, 64);
  if (row < total && c == 0) a.delta[((int64_t)b * a.H + h) * a.Sq + i] = acc;
}

// ---- dQ ------------------------------------------------------------------------
template <int D, bool PF>
__global__ __launch_bounds__(256) void bwd_dq_kernel(const BwdArgs a) {
  constexpr int BN = 64;
  constexpr int KP = RowTile<D>::kPitch;
  constexpr int DK = D / 16;
  constexpr int DB = D / 32;
  constexpr int CPR = D / 8;
  constexpr int VCH = (BN * CPR) / 256;
  constexpr int NU = TileUnits<D>::NU;

  extern __shared__ __align__(16) char smem_raw[];
  bf16_t *Ks = reinterpret_cast<bf16_t *>(smem_raw);
  bf16_t *Vs = Ks + BN * KP;
  bf16_t *Kt = Vs + BN * KP;
  int *kb_s = reinterpret_cast<int *>(Kt + D * BN);
  int *red_s = kb_s + BN;

  const int tid = threadIdx.x;
  const int wave = tid >> 6, lane = tid & 63;
  const int n = lane & 31, hh = lane >> 5;

  const int R = a.G * a.Sq;
  const int ntile_r = (R + 127) / 128;
  int bid = blockIdx.x;
  const int tile = bid % ntile_r;
  bid /= ntile_r;
  const int hk = bid % a.Hkv;
  const int b = bid / a.Hkv;

  const int r = tile * 128 + wave * 32 + n;
  const bool rowok = r < R;
  const int rr = rowok ? r : R - 1;
  const int g = rr / a.Sq;
  const int i = rr - g * a.Sq;
  const int h = hk * a.G + g;
  const bool qv = rowok && a.q_valid[(int64_t)b * a.Sq + i] != 0;
  const int qb = qv ? a.q_blk[(int64_t)b * a.Sq + i] : kIntMin;

  const bf16_t *qptr =
      reinterpret_cast<const bf16_t *>(a.q.ptr) + b * a.q.sb + (int64_t)i * a.q.ss + h * a.q.sh;
  const bf16_t *gptr =
      reinterpret_cast<const bf16_t *>(a.d_o.ptr) + b * a.d_o.sb + (int64_t)i * a.d_o.ss + h * a.d_o.sh;
  bf16x8 qf[DK], gof[DK];
#pragma unroll
  for (int ks = 0; ks < DK; ++ks) {
    qf[ks] = *reinterpret_cast<const bf16x8 *>(qptr + 16 * ks + 8 * hh);
    gof[ks] = *reinterpret_cast<const bf16x8 *>(gptr + 16 * ks + 8 * hh);
  }
  const int64_t stat = ((int64_t)b * a.H + h) * a.Sq + i;
  // Rows that take no part get +inf so that every probability comes out 0.
  const float lse2 = qv ? a.lse[stat] * kLog2e : INFINITY;
  const float delta = qv ? a.delta[stat] : 0.f;

  const int qmax_w = wave_max_i(qv ? qb : kIntMin);
  const int qmin_w = wave_min_i(qv ? qb : kIntMax);
  const int any_w = wave_max_i(qv ? 1 : 0);
  if (lane == 0) {
    red_s[wave] = qmax_w;
    red_s[4 + wave] = any_w;
  }
  __syncthreads();
  const int qmax_g = max(max(red_s[0], red_s[1]), max(red_s[2], red_s[3]));
  const int any_g = red_s[4] | red_s[5] | red_s[6] | red_s[7];

  const int Sk = a.Sk;
  const int nt = any_g ? (Sk + BN - 1) / BN : 0;
  const tile_summary_t *ksum = a.ksum + (int64_t)b * ((Sk + BN - 1) / BN);
  const bf16_t *kb_ = reinterpret_cast<const bf16_t *>(a.k.ptr) + b * a.k.sb + hk * a.k.sh;
  const bf16_t *vb_ = reinterpret_cast<const bf16_t *>(a.v.ptr) + b * a.v.sb + hk * a.v.sh;

  bf16x8 kreg[NU][4];
  bf16x8 vreg[VCH];
  int kbreg = kIntMax;

  auto next_needed = [&](int t) {
    while (t < nt && ksum[t].x > qmax_g) ++t;
    return t;
  };
  auto fetch = [&](int t) {
    const int j0 = t * BN;
    load_units<D>(kreg, kb_, a.k.ss, j0, Sk, tid);
#pragma unroll
    for (int it = 0; it < VCH; ++it) {
      const int c = tid + 256 * it;
      const int row = c / CPR, col = c % CPR;
      const int jc = min(j0 + row, Sk - 1);
      const bf16x8 val = *reinterpret_cast<const bf16x8 *>(vb_ + (int64_t)jc * a.v.ss + col * 8);
      vreg[it] = keep_if(j0 + row < Sk, val);
    }
    {
      const int j = j0 + (tid & (BN - 1)), jc = min(j, Sk - 1);
      const int id = a.k_blk[(int64_t)b * Sk + jc];
      const int ok = a.k_valid[(int64_t)b * Sk + jc];
      kbreg = (j < Sk && ok != 0) ? id : kIntMax;
    }
  };
  auto stage = [&]() {
    store_units<D, true, true>(kreg, Ks, Kt, tid);
#pragma unroll
    for (int it = 0; it < VCH; ++it) {
      const int c = tid + 256 * it;
      const int row = c / CPR, col = c % CPR;
      *reinterpret_cast<bf16x8 *>(Vs + row * KP + col * 8) = vreg[it];
    }
    if (tid < BN) kb_s[tid] = kbreg;
  };

  f32x16 dq[DB];
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int x = 0; x < 16; ++x) dq[db][x] = 0.f;
  const float c = a.scale * kLog2e;

  int t = next_needed(0);
  if (PF && t < nt) fetch(t);
  while (t < nt) {
    if (!PF) fetch(t);
    stage();
    __syncthreads();
    const tile_summary_t sm = ksum[t];
    const int tn = next_needed(t + 1);
    if (PF && tn < nt) fetch(tn);

    if (sm.x <= qmax_w) {
      const bool needmask = !(sm.z != 0 && sm.y <= qmin_w);
#pragma unroll
      for (int mb = 0; mb < 2; ++mb) {
        f32x16 s, dp;
#pragma unroll
        for (int x = 0; x < 16; ++x) s[x] = 0.f, dp[x] = 0.f;
        const bf16_t *kp = Ks + (32 * mb + n) * KP + 8 * hh;
        const bf16_t *vp = Vs + (32 * mb + n) * KP + 8 * hh;
        constexpr int KB = DK < 8 ? DK : 8;  // operand reads issued ahead of the products
#pragma unroll
        for (int k0 = 0; k0 < DK; k0 += KB) {
          bf16x8 fa[KB], fb[KB];
#pragma unroll
          for (int ks = 0; ks < KB; ++ks) {
            fa[ks] = *reinterpret_cast<const bf16x8 *>(kp + 16 * (k0 + ks));
            fb[ks] = *reinterpret_cast<const bf16x8 *>(vp + 16 * (k0 + ks));
          }
#pragma unroll
          for (int ks = 0; ks < KB; ++ks) {
            s = mfma32(fa[ks], qf[k0 + ks], s);
            dp = mfma32(fb[ks], gof[k0 + ks], dp);
          }
        }
        float ds[16];
#pragma unroll
        for (int r4 = 0; r4 < 4; ++r4) {
          i32x4 kb4 = {0, 0, 0, 0};
          if (needmask) kb4 = *reinterpret_cast<const i32x4 *>(kb_s + 32 * mb + 8 * r4 + 4 * hh);
#pragma unroll
          for (int x = 0; x < 4; ++x) {
            float p = fast_exp2(s[4 * r4 + x] * c - lse2);
            if (needmask && kb4[x] > qb) p = 0.f;
            ds[4 * r4 + x] = p * (dp[4 * r4 + x] - delta);
          }
        }
        bf16x8 dsb[2];
        dsb[0] = pack8(ds[0], ds[1], ds[2], ds[3], ds[4], ds[5], ds[6], ds[7]);
        dsb[1] = pack8(ds[8], ds[9], ds[10], ds[11], ds[12], ds[13], ds[14], ds[15]);
#pragma unroll
        for (int db = 0; db < DB; ++db) {
          const int d = 32 * db + n;
#pragma unroll
          for (int half = 0; half < 2; ++half) {
            const bf16x8 ka =
                *reinterpret_cast<const bf16x8 *>(Kt + tr_read_off(d, 2 * mb + half, hh));
            dq[db] = mfma32(ka, dsb[half], dq[db]);
          }
        }
      }
    }
    __syncthreads();
    t = tn;
  }

  if (rowok) {
    bf16_t *optr = reinterpret_cast<bf16_t *>(a.dq) + b * a.dq_sb + (int64_t)i * a.dq_ss + h * a.dq_sh;
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int r4 = 0; r4 < 4; ++r4) {
        bf16x4 w;
#pragma unroll
        for (int x = 0; x < 4; ++x) w[x] = (bf16_t)(dq[db][4 * r4 + x] * a.scale);
        *reinterpret_cast<bf16x4 *>(optr + 32 * db + 8 * r4 + 4 * hh) = w;
      }
  }
}

template <int D>
constexpr size_t dq_smem_bytes() {
  return (size_t)(2 * 64 * RowTile<D>::kPitch + D * 64) * 2 + 64 * 4 + 8 * 4;
}

// ---- dK / dV ---------------------------------------------------------------------
template <int D, bool PF>
__global__ __launch_bounds__(256) void bwd_dkv_kernel(const BwdArgs a) {
  constexpr int BQ = 64;
  constexpr int KP = RowTile<D>::kPitch;
  constexpr int DK = D / 16;
  constexpr int DB = D / 32;
  constexpr int NU = TileUnits<D>::NU;

  extern __shared__ __align__(16) char smem_raw[];
  bf16_t *Qs = reinterpret_cast<bf16_t *>(smem_raw);
  bf16_t *Gs = Qs + BQ * KP;
  bf16_t *Qt = Gs + BQ * KP;
  bf16_t *Gt = Qt + D * BQ;
  float *lse_s = reinterpret_cast<float *>(Gt + D * BQ);
  float *delta_s = lse_s + BQ;
  int *qb_s = reinterpret_cast<int *>(delta_s + BQ);
  int *red_s = qb_s + BQ;

  const int tid = threadIdx.x;
  const int wave = tid >> 6, lane = tid & 63;
  const int n = lane & 31, hh = lane >> 5;

  const int Sk = a.Sk, Sq = a.Sq;
  const int nkt = (Sk + 127) / 128;
  int bid = blockIdx.x;
  const int kt = bid % nkt;
  bid /= nkt;
  const int hk = bid % a.Hkv;
  const int b = bid / a.Hkv;

  // ---- this lane's key -----------------------------------------------------
  const int j = kt * 128 + wave * 32 + n;
  const bool jok = j < Sk;
  const int jj = jok ? j : Sk - 1;
  const bool kv = jok && a.k_valid[(int64_t)b * Sk + jj] != 0;
  const int kb = kv ? a.k_blk[(int64_t)b * Sk + jj] : kIntMax;
  const bf16_t *kptr =
      reinterpret_cast<const bf16_t *>(a.k.ptr) + b * a.k.sb + (int64_t)jj * a.k.ss + hk * a.k.sh;
  const bf16_t *vptr =
      reinterpret_cast<const bf16_t *>(a.v.ptr) + b * a.v.sb + (int64_t)jj * a.v.ss + hk * a.v.sh;
  bf16x8 kf[DK], vf[DK];
#pragma unroll
  for (int ks = 0; ks < DK; ++ks) {
    kf[ks] = *reinterpret_cast<const bf16x8 *>(kptr + 16 * ks + 8 * hh);
    vf[ks] = *reinterpret_cast<const bf16x8 *>(vptr + 16 * ks + 8 * hh);
  }
  const int kmin_w = wave_min_i(kb);
  const int kmax_w = wave_max_i(kv ? kb : kIntMin);
  const int allk_w = wave_min_i(kv ? 1 : 0);
  if (lane == 0) red_s[wave] = kmin_w;
  __syncthreads();
  const int kmin_g = min(min(red_s[0], red_s[1]), min(red_s[2], red_s[3]));

  const int nqt = (Sq + BQ - 1) / BQ;
  const tile_summary_t *qsum = a.qsum + (int64_t)b * nqt;
  const int nit = (kmin_g == kIntMax) ? 0 : a.G * nqt;

  bf16x8 qreg[NU][4], greg[NU][4];
  float lsereg = INFINITY, delreg = 0.f;
  int qbreg = kIntMin;

  auto next_needed = [&](int it) {
    while (it < nit) {
      const tile_summary_t s = qsum[it % nqt];
      if (s.w > 0 && s.y >= kmin_g) break;
      ++it;
    }
    return it;
  };
  auto fetch = [&](int it) {
    const int g = it / nqt, qt = it - g * nqt;
    const int h = hk * a.G + g;
    const int i0 = qt * BQ;
    const bf16_t *qb_ = reinterpret_cast<const bf16_t *>(a.q.ptr) + b * a.q.sb + h * a.q.sh;
    const bf16_t *gb_ = reinterpret_cast<const bf16_t *>(a.d_o.ptr) + b * a.d_o.sb + h * a.d_o.sh;
    load_units<D>(qreg, qb_, a.q.ss, i0, Sq, tid);
    load_units<D>(greg, gb_, a.d_o.ss, i0, Sq, tid);
    {
      const int i = i0 + (tid & (BQ - 1)), ic = min(i, Sq - 1);
      const int64_t stat = ((int64_t)b * a.H + h) * Sq + ic;
      const float lv = a.lse[stat], dl = a.delta[stat];
      const int id = a.q_blk[(int64_t)b * Sq + ic];
      const bool ok = i < Sq && a.q_valid[(int64_t)b * Sq + ic] != 0;
      lsereg = ok ? lv * kLog2e : INFINITY;
      delreg = ok ? dl : 0.f;
      qbreg = ok ? id : kIntMin;
    }
  };
  auto stage = [&]() {
    store_units<D, true, true>(qreg, Qs, Qt, tid);
    store_units<D, true, true>(greg, Gs, Gt, tid);
    if (tid < BQ) {
      lse_s[tid] = lsereg;
      delta_s[tid] = delreg;
      qb_s[tid] = qbreg;
    }
  };

  f32x16 dk[DB], dv[DB];
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int x = 0; x < 16; ++x) dk[db][x] = 0.f, dv[db][x] = 0.f;
  const float c = a.scale * kLog2e;

  int it = next_needed(0);
  if (PF && it < nit) fetch(it);
  while (it < nit) {
    if (!PF) fetch(it);
    stage();
    __syncthreads();
    const tile_summary_t sm = qsum[it % nqt];
    const int itn = next_needed(it + 1);
    if (PF && itn < nit) fetch(itn);

    if (sm.y >= kmin_w) {
      const bool needmask = !(sm.z != 0 && allk_w != 0 && kmax_w <= sm.x);
#pragma unroll
      for (int mb = 0; mb < 2; ++mb) {
        f32x16 s, dp;
#pragma unroll
        for (int x = 0; x < 16; ++x) s[x] = 0.f, dp[x] = 0.f;
        const bf16_t *qp = Qs + (32 * mb + n) * KP + 8 * hh;
        const bf16_t *gp = Gs + (32 * mb + n) * KP + 8 * hh;
        constexpr int KB = DK < 8 ? DK : 8;
#pragma unroll
        for (int k0 = 0; k0 < DK; k0 += KB) {
          bf16x8 fa[KB], fb[KB];
#pragma unroll
          for (int ks = 0; ks < KB; ++ks) {
            fa[ks] = *reinterpret_cast<const bf16x8 *>(qp + 16 * (k0 + ks));
            fb[ks] = *reinterpret_cast<const bf16x8 *>(gp + 16 * (k0 + ks));
          }
#pragma unroll
          for (int ks = 0; ks < KB; ++ks) {
            s = mfma32(fa[ks], kf[k0 + ks], s);
            dp = mfma32(fb[ks], vf[k0 + ks], dp);
          }
        }
        float p[16], ds[16];
#pragma unroll
        for (int r4 = 0; r4 < 4; ++r4) {
          const int q0 = 32 * mb + 8 * r4 + 4 * hh;
          const f32x4 lse4 = *reinterpret_cast<const f32x4 *>(lse_s + q0);
          const f32x4 del4 = *reinterpret_cast<const f32x4 *>(delta_s + q0);
          i32x4 qb4 = {0, 0, 0, 0};
          if (needmask) qb4 = *reinterpret_cast<const i32x4 *>(qb_s + q0);
#pragma unroll
          for (int x = 0; x < 4; ++x) {
            float pv = fast_exp2(s[4 * r4 + x] * c - lse4[x]);
            if (needmask && kb > qb4[x]) pv = 0.f;
            p[4 * r4 + x] = pv;
            ds[4 * r4 + x] = pv * (dp[4 * r4 + x] - del4[x]);
          }
        }
        bf16x8 pb[2], dsb[2];
        pb[0] = pack8(p[0], p[1], p[2], p[3], p[4], p[5], p[6], p[7]);
        pb[1] = pack8(p[8], p[9], p[10], p[11], p[12], p[13], p[14], p[15]);
        dsb[0] = pack8(ds[0], ds[1], ds[2], ds[3], ds[4], ds[5], ds[6], ds[7]);
        dsb[1] = pack8(ds[8], ds[9], ds[10], ds[11], ds[12], ds[13], ds[14], ds[15]);
#pragma unroll
        for (int db = 0; db < DB; ++db) {
          const int d = 32 * db + n;
#pragma unroll
          for (int half = 0; half < 2; ++half) {
            const int off = tr_read_off(d, 2 * mb + half, hh);
            dv[db] = mfma32(*reinterpret_cast<const bf16x8 *>(Gt + off), pb[half], dv[db]);
            dk[db] = mfma32(*reinterpret_cast<const bf16x8 *>(Qt + off), dsb[half], dk[db]);
          }
        }
      }
    }
    __syncthreads();
    it = itn;
  }

  if (jok) {
    bf16_t *dkp = reinterpret_cast<bf16_t *>(a.dk) + b * a.dk_sb + (int64_t)j * a.dk_ss + hk * a.dk_sh;
    bf16_t *dvp = reinterpret_cast<bf16_t *>(a.dv) + b * a.dv_sb + (int64_t)j * a.dv_ss + hk * a.dv_sh;
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int r4 = 0; r4 < 4; ++r4) {
        bf16x4 wk, wv;
#pragma unroll
        for (int x = 0; x < 4; ++x) {
          wk[x] = (bf16_t)(dk[db][4 * r4 + x] * a.scale);
          wv[x] = (bf16_t)dv[db][4 * r4 + x];
        }
        *reinterpret_cast<bf16x4 *>(dkp + 32 * db + 8 * r4 + 4 * hh) = wk;
        *reinterpret_cast<bf16x4 *>(dvp + 32 * db + 8 * r4 + 4 * hh) = wv;
      }
  }
}

template <int D>
constexpr size_t dkv_smem_bytes() {
  return (size_t)(2 * 64 * RowTile<D>::kPitch + 2 * D * 64) * 2 + 3 * 64 * 4 + 8 * 4;
}

template <int D, bool PF>
static int launch_bwd_d(const BwdArgs &a, hipStream_t st) {
  {
    if (hipFuncSetAttribute(reinterpret_cast<const void *>(&bwd_dq_kernel<D, PF>),
                            hipFuncAttributeMaxDynamicSharedMemorySize,
                            (int)dq_smem_bytes<D>()) != hipSuccess ||
        hipFuncSetAttribute(reinterpret_cast<const void *>(&bwd_dkv_kernel<D, PF>),
                            hipFuncAttributeMaxDynamicSharedMemorySize,
                            (int)dkv_smem_bytes<D>()) != hipSuccess)
      return BCATTN_ERR_LAUNCH;
  }
  constexpr int RPB = 256 / (D / 8);
  const int64_t rows = (int64_t)a.B * a.Sq * a.H;
  if (a.stages & BCATTN_BWD_DELTA)
    hipLaunchKernelGGL(bwd_delta_kernel<D>, dim3((unsigned)((rows + RPB - 1) / RPB)), dim3(256), 0, st, a);
  const int R = a.G * a.Sq;
  const int ntile_r = (R + 127) / 128;
  if (a.stages & BCATTN_BWD_DQ)
    hipLaunchKernelGGL((bwd_dq_kernel<D, PF>), dim3((unsigned)(ntile_r * a.Hkv * a.B)), dim3(256),
                     dq_smem_bytes<D>(), st, a);
  const int nkt = (a.Sk + 127) / 128;
  if (a.stages & BCATTN_BWD_DKV)
    hipLaunchKernelGGL((bwd_dkv_kernel<D, PF>), dim3((unsigned)(nkt * a.Hkv * a.B)), dim3(256),
                     dkv_smem_bytes<D>(), st, a);
  return hipGetLastError() == hipSuccess ? BCATTN_OK : BCATTN_ERR_LAUNCH;
}

int launch_bwd_bf16(const BwdArgs &a, int D, hipStream_t st) {
  switch (D) {
    case 64:
      return launch_bwd_d<64, true>(a, st);
    case 128:
      return launch_bwd_d<128, true>(a, st);
    case 256:
      return launch_bwd_d<256, false>(a, st);
    default:
      return BCATTN_ERR_UNSUPPORTED;
  }
}

}  // namespace bcattn
