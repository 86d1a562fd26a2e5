// Block-causal attention forward, bf16 in / fp32 accumulate, gfx950 MFMA.
//
// One workgroup = 4 waves = 128 "packed" query rows of one (batch, kv head):
// packed row r = g*Sq + i runs over the G = H/Hkv query heads that share the kv
// head, so MQA/GQA heads reuse the same K/V tile in LDS.  A wave owns 32 rows;
// lane l owns row l%32 (its running max / sum / block id live in scalars of the
// lane) and the two lane halves split the contraction index.
//
// Scores are computed transposed, S^T = K Q^T (keys x queries), so that the
// softmax reduction over keys is in-lane plus one exchange with lane^32, and so
// that the 32x32 accumulator of S^T is already laid out as the B operand of
// O^T = V^T P^T.  K tiles sit in LDS as rows, V tiles transposed.
#include "bcattn_common.h"

namespace bcattn {

//
// SPLIT: the key tiles are divided over `nsplit` workgroups per row tile; each
// writes its unnormalised fp32 partial (O, running max, sum) and
// `fwd_combine_kernel` merges them.  This is what lets a handful of
// (batch, kv head) problems with few query rows fill the chip.
template <int D, int NW, bool SPLIT>
__global__ __launch_bounds__(64 * NW) void fwd_bf16_kernel(const FwdArgs a, const SplitArgs sp) {
  constexpr int BN = 64;
  constexpr int NT = 64 * NW;   // threads
  constexpr int BM = 32 * NW;   // packed query rows per workgroup
  constexpr int KP = RowTile<D>::kPitch;
  constexpr int DK = D / 16;   // contraction steps of K Q^T
  constexpr int DB = D / 32;   // 32-row blocks of O^T
  constexpr int CPR = D / 8;   // 16-byte chunks per row
  constexpr int KCH = (BN * CPR) / NT;
  constexpr int VUNITS = 16 * CPR;  // 4x8 transposition units per V tile
  constexpr int VUN = (VUNITS + NT - 1) / NT;
  static_assert((BN * CPR) % NT == 0, "K tile must divide over the threads");

  __shared__ __align__(16) bf16_t Ks[BN * KP];
  __shared__ __align__(16) bf16_t Vt[D * BN];
  __shared__ __align__(16) int kb_s[BN];
  __shared__ int red_s[2 * NW];

  const int tid = threadIdx.x;
  const int wave = tid >> 6, lane = tid & 63;
  const int n = lane & 31, hh = lane >> 5;

  const int R = a.G * a.Sq;
  const int ntile_r = (R + BM - 1) / BM;
  int bid = blockIdx.x;
  const int tile = bid % ntile_r;
  bid /= ntile_r;
  const int split = SPLIT ? bid % sp.nsplit : 0;
  if (SPLIT) bid /= sp.nsplit;
  const int hk = bid % a.Hkv;
  const int b = bid / a.Hkv;

  // ---- this lane's query row ------------------------------------------------
  const int r = tile * BM + wave * 32 + n;
  const bool rowok = r < R;
  const int rr = rowok ? r : R - 1;
  const int g = rr / a.Sq;
  const int i = rr - g * a.Sq;
  const int h = hk * a.G + g;
  const bool qv = rowok && a.q_valid[(int64_t)b * a.Sq + i] != 0;
  const int qb = qv ? a.q_blk[(int64_t)b * a.Sq + i] : kIntMin;

  const bf16_t *qptr =
      reinterpret_cast<const bf16_t *>(a.q.ptr) + b * a.q.sb + (int64_t)i * a.q.ss + h * a.q.sh;
  bf16x8 qf[DK];
#pragma unroll
  for (int ks = 0; ks < DK; ++ks)
    qf[ks] = *reinterpret_cast<const bf16x8 *>(qptr + 16 * ks + 8 * hh);

  // ---- block-id range of the wave and of the workgroup ------------------------
  const int qmax_w = wave_max_i(qv ? qb : kIntMin);
  const int qmin_w = wave_min_i(qv ? qb : kIntMax);
  const int any_w = wave_max_i(qv ? 1 : 0);
  if (lane == 0) {
    red_s[wave] = qmax_w;
    red_s[NW + wave] = any_w;
  }
  __syncthreads();
  int qmax_g = kIntMin, any_g = 0;
#pragma unroll
  for (int x = 0; x < NW; ++x) {
    qmax_g = max(qmax_g, red_s[x]);
    any_g |= red_s[NW + x];
  }

  const int Sk = a.Sk;
  const int nt_all = (Sk + BN - 1) / BN;
  const int t_first = SPLIT ? split * sp.tiles_per_split : 0;
  const int nt = !any_g ? 0 : (SPLIT ? min(nt_all, t_first + sp.tiles_per_split) : nt_all);
  const tile_summary_t *ksum = a.ksum + (int64_t)b * nt_all;

  const bf16_t *k0b = reinterpret_cast<const bf16_t *>(a.k0.ptr) + b * a.k0.sb + hk * a.k0.sh;
  const bf16_t *v0b = reinterpret_cast<const bf16_t *>(a.v0.ptr) + b * a.v0.sb + hk * a.v0.sh;
  const bf16_t *k1b = reinterpret_cast<const bf16_t *>(a.k1.ptr) + b * a.k1.sb + hk * a.k1.sh;
  const bf16_t *v1b = reinterpret_cast<const bf16_t *>(a.v1.ptr) + b * a.v1.sb + hk * a.v1.sh;
  const int Sk0 = a.Sk0;
  const int32_t *kblk_b = a.k_blk + (int64_t)b * Sk;
  const uint8_t *kval_b = a.k_valid + (int64_t)b * Sk;

  bf16x8 kreg[KCH];
  bf16x8 vreg[VUN][4];
  int kbreg = kIntMax;

  auto next_needed = [&](int t) {
    while (t < nt && ksum[t].x > qmax_g) ++t;
    return t;
  };

  // Global loads of one tile into registers (consumed by stage() one iteration later).
  auto prefetch = [&](int t) {
    const int j0 = t * BN;
#pragma unroll
    for (int it = 0; it < KCH; ++it) {
      const int c = tid + NT * it;
      const int row = c / CPR, col = c % CPR;
      const int j = j0 + row, jc = min(j, Sk - 1);
      const bf16x8 val =
          *reinterpret_cast<const bf16x8 *>(seg_row(k0b, a.k0.ss, k1b, a.k1.ss, Sk0, jc) + col * 8);
      kreg[it] = keep_if(j < Sk, val);
    }
#pragma unroll
    for (int it = 0; it < VUN; ++it) {
      const int u = min(tid + NT * it, VUNITS - 1);
      const int dch = u % CPR, kg = u / CPR;
#pragma unroll
      for (int x = 0; x < 4; ++x) {
        const int j = j0 + 4 * kg + x, jc = min(j, Sk - 1);
        const bf16x8 val =
            *reinterpret_cast<const bf16x8 *>(seg_row(v0b, a.v0.ss, v1b, a.v1.ss, Sk0, jc) + dch * 8);
        vreg[it][x] = keep_if(j < Sk, val);
      }
    }
    {
      const int j = j0 + (tid & (BN - 1)), jc = min(j, Sk - 1);
      const int id = kblk_b[jc];
      const int ok = kval_b[jc];
      kbreg = (j < Sk && ok != 0) ? id : kIntMax;
    }
  };

  auto stage = [&]() {
#pragma unroll
    for (int it = 0; it < KCH; ++it) {
      const int c = tid + NT * it;
      const int row = c / CPR, col = c % CPR;
      *reinterpret_cast<bf16x8 *>(Ks + row * KP + col * 8) = kreg[it];
    }
#pragma unroll
    for (int it = 0; it < VUN; ++it) {
      const int u = tid + NT * it;
      const int dch = u % CPR, kg = u / CPR;
      if (u < VUNITS) tr_store_4x8(Vt, 8 * dch, kg, vreg[it][0], vreg[it][1], vreg[it][2], vreg[it][3]);
    }
    if (tid < BN) kb_s[tid] = kbreg;
  };

  // ---- running state ---------------------------------------------------------
  f32x16 o[DB];
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int x = 0; x < 16; ++x) o[db][x] = 0.f;
  float m = -INFINITY;  // running max of the raw (unscaled) scores
  float l = 0.f;        // this lane half's share of the running sum
  const float c = a.scale * kLog2e;

  int t = next_needed(t_first);
  if (t < nt) prefetch(t);
  while (t < nt) {
    stage();
    __syncthreads();
    const tile_summary_t sm = ksum[t];
    const int tn = next_needed(t + 1);
    if (tn < nt) prefetch(tn);

    if (sm.x <= qmax_w) {  // wave-uniform: some row of this wave sees some key of the tile
      f32x16 s[2];
#pragma unroll
      for (int mb = 0; mb < 2; ++mb) {
#pragma unroll
        for (int x = 0; x < 16; ++x) s[mb][x] = 0.f;
        const bf16_t *kp = Ks + (32 * mb + n) * KP + 8 * hh;
        bf16x8 ka[DK];
#pragma unroll
        for (int ks = 0; ks < DK; ++ks) ka[ks] = *reinterpret_cast<const bf16x8 *>(kp + 16 * ks);
#pragma unroll
        for (int ks = 0; ks < DK; ++ks) s[mb] = mfma32(ka[ks], qf[ks], s[mb]);
      }
      const bool needmask = !(sm.z != 0 && sm.y <= qmin_w);
      if (needmask) {
#pragma unroll
        for (int mb = 0; mb < 2; ++mb)
#pragma unroll
          for (int r4 = 0; r4 < 4; ++r4) {
            const i32x4 kb4 = *reinterpret_cast<const i32x4 *>(kb_s + 32 * mb + 8 * r4 + 4 * hh);
#pragma unroll
            for (int x = 0; x < 4; ++x)
              if (kb4[x] > qb) s[mb][4 * r4 + x] = -INFINITY;
          }
      }
      float mloc = s[0][0];
#pragma unroll
      for (int mb = 0; mb < 2; ++mb)
#pragma unroll
        for (int x = 0; x < 16; ++x) mloc = fmaxf(mloc, s[mb][x]);
      mloc = fmaxf(mloc, swap32(mloc));
      const float mnew = fmaxf(m, mloc);
      const float moff = (mnew == -INFINITY) ? 0.f : mnew * c;
      if (__any(mnew > m)) {
        const float corr = fast_exp2(m * c - moff);
        l *= corr;
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
          for (int x = 0; x < 16; ++x) o[db][x] *= corr;
      }
      m = mnew;
      bf16x8 pb[4];
#pragma unroll
      for (int mb = 0; mb < 2; ++mb) {
        float p[16];
#pragma unroll
        for (int x = 0; x < 16; ++x) {
          p[x] = fast_exp2(s[mb][x] * c - moff);
          l += p[x];
        }
        pb[2 * mb] = pack8(p[0], p[1], p[2], p[3], p[4], p[5], p[6], p[7]);
        pb[2 * mb + 1] = pack8(p[8], p[9], p[10], p[11], p[12], p[13], p[14], p[15]);
      }
#pragma unroll
      for (int db = 0; db < DB; ++db) {
        const int d = 32 * db + n;
        bf16x8 va[4];
#pragma unroll
        for (int kk = 0; kk < 4; ++kk)
          va[kk] = *reinterpret_cast<const bf16x8 *>(Vt + tr_read_off(d, kk, hh));
#pragma unroll
        for (int kk = 0; kk < 4; ++kk) o[db] = mfma32(va[kk], pb[kk], o[db]);
      }
    }
    __syncthreads();
    t = tn;
  }

  // ---- epilogue ----------------------------------------------------------------
  l += swap32(l);
  if (SPLIT) {
    if (rowok) {
      const int64_t prow = (((int64_t)b * a.Hkv + hk) * sp.nsplit + split) * R + r;
      if (hh == 0) {
        f32x2 ml;
        ml[0] = qv ? m : -INFINITY;
        ml[1] = qv ? l : 0.f;
        *reinterpret_cast<f32x2 *>(sp.part_ml + 2 * prow) = ml;
      }
      float *po = sp.part_o + prow * D;
#pragma unroll
      for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int r4 = 0; r4 < 4; ++r4) {
          f32x4 w;
#pragma unroll
          for (int x = 0; x < 4; ++x) w[x] = o[db][4 * r4 + x];
          *reinterpret_cast<f32x4 *>(po + 32 * db + 8 * r4 + 4 * hh) = w;
        }
    }
    return;
  }
  const bool has = qv && l > 0.f;
  const float inv = has ? 1.f / l : 0.f;
  if (rowok) {
    if (a.lse != nullptr && hh == 0)
      a.lse[((int64_t)b * a.H + h) * a.Sq + i] = has ? m * a.scale + __logf(l) : 0.f;
    bf16_t *optr = reinterpret_cast<bf16_t *>(a.o) + b * a.o_sb + (int64_t)i * a.o_ss + h * a.o_sh;
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int r4 = 0; r4 < 4; ++r4) {
        bf16x4 w;
#pragma unroll
        for (int x = 0; x < 4; ++x) w[x] = (bf16_t)(o[db][4 * r4 + x] * inv);
        *reinterpret_cast<bf16x4 *>(optr + 32 * db + 8 * r4 + 4 * hh) = w;
      }
  }
}

// Merge the per-split partials: one thread per (packed row, 4 head_dim columns).
template <int D>
__global__ __launch_bounds__(256) void fwd_combine_kernel(const FwdArgs a, const SplitArgs sp) {
  constexpr int TPR = D / 4;
  const int R = a.G * a.Sq;
  const int64_t total = (int64_t)a.B * a.Hkv * R;
  const int64_t idx = (int64_t)blockIdx.x * (256 / TPR) + threadIdx.x / TPR;
  const int c4 = threadIdx.x % TPR;
  if (idx >= total) return;
  const int r = (int)(idx % R);
  const int64_t bh = idx / R;
  const int hk = (int)(bh % a.Hkv);
  const int b = (int)(bh / a.Hkv);
  const int g = r / a.Sq, i = r - g * a.Sq, h = hk * a.G + g;
  const float c = a.scale * kLog2e;
  const int64_t p0 = bh * sp.nsplit * R + r;
  float mx = -INFINITY;
  for (int s = 0; s < sp.nsplit; ++s) mx = fmaxf(mx, sp.part_ml[2 * (p0 + (int64_t)s * R)]);
  f32x4 acc = {0.f, 0.f, 0.f, 0.f};
  float lsum = 0.f;
  if (mx != -INFINITY) {
    for (int s = 0; s < sp.nsplit; ++s) {
      const int64_t pr = p0 + (int64_t)s * R;
      const f32x2 ml = *reinterpret_cast<const f32x2 *>(sp.part_ml + 2 * pr);
      if (ml[0] == -INFINITY) continue;
      const float w = fast_exp2((ml[0] - mx) * c);
      lsum += w * ml[1];
      const f32x4 po = *reinterpret_cast<const f32x4 *>(sp.part_o + pr * D + 4 * c4);
#pragma unroll
      for (int x = 0; x < 4; ++x) acc[x] += w * po[x];
    }
  }
  const bool has = lsum > 0.f;
  const float inv = has ? 1.f / lsum : 0.f;
  bf16x4 w;
#pragma unroll
  for (int x = 0; x < 4; ++x) w[x] = (bf16_t)(acc[x] * inv);
  bf16_t *optr = reinterpret_cast<bf16_t *>(a.o) + b * a.o_sb + (int64_t)i * a.o_ss + h * a.o_sh;
  *reinterpret_cast<bf16x4 *>(optr + 4 * c4) = w;
  if (a.lse != nullptr && c4 == 0)
    a.lse[((int64_t)b * a.H + h) * a.Sq + i] = has ? mx * a.scale + __logf(lsum) : 0.f;
}

int launch_fwd_bf16(const FwdArgs &a, int D, hipStream_t st) {
  const int R = a.G * a.Sq;
  const SplitArgs sp{nullptr, nullptr, 1, 0};
  auto grid = [&](int bm) { return dim3((unsigned)(((R + bm - 1) / bm) * a.Hkv * a.B)); };
  switch (D) {
    case 64:
      hipLaunchKernelGGL((fwd_bf16_kernel<64, 4, false>), grid(128), dim3(256), 0, st, a, sp);
      break;
    case 128:
      if (R >= 1024)
        hipLaunchKernelGGL((fwd_bf16_kernel<128, 8, false>), grid(256), dim3(512), 0, st, a, sp);
      else
        hipLaunchKernelGGL((fwd_bf16_kernel<128, 4, false>), grid(128), dim3(256), 0, st, a, sp);
      break;
    case 256:
      hipLaunchKernelGGL((fwd_bf16_kernel<256, 4, false>), grid(128), dim3(256), 0, st, a, sp);
      break;
    default:
      return BCATTN_ERR_UNSUPPORTED;
  }
  return hipGetLastError() == hipSuccess ? BCATTN_OK : BCATTN_ERR_LAUNCH;
}

// How many ways to split the key axis so that about 1.5 workgroups per CU exist.
static void plan_split(int B, int Sq, int Sk, int H, int Hkv, int *nsplit, int *tps) {
  const int R = (H / Hkv) * Sq;
  const int base = B * Hkv * ((R + 127) / 128);
  const int ntiles = (Sk + 63) / 64;
  int want = (384 + base - 1) / base;
  if (want < 1) want = 1;
  if (want > ntiles) want = ntiles;
  *tps = (ntiles + want - 1) / want;
  *nsplit = (ntiles + *tps - 1) / *tps;
}

size_t kvcache_workspace_bytes(int B, int Sq, int Sk, int H, int Hkv, int D, int *nsplit_out) {
  int ns, tps;
  plan_split(B, Sq, Sk, H, Hkv, &ns, &tps);
  *nsplit_out = ns;
  if (ns <= 1) return 0;
  const size_t R = (size_t)(H / Hkv) * Sq;
  const size_t rows = (size_t)B * Hkv * ns * R;
  return ((rows * (D + 2) * sizeof(float)) + 255) & ~(size_t)255;
}

template <int D>
static int launch_split(const FwdArgs &a, const SplitArgs &sp, hipStream_t st) {
  const int R = a.G * a.Sq;
  const int ntile_r = (R + 127) / 128;
  hipLaunchKernelGGL((fwd_bf16_kernel<D, 4, true>), dim3((unsigned)(ntile_r * sp.nsplit * a.Hkv * a.B)),
                     dim3(256), 0, st, a, sp);
  constexpr int RPB = 256 / (D / 4);
  const int64_t rows = (int64_t)a.B * a.Hkv * R;
  hipLaunchKernelGGL(fwd_combine_kernel<D>, dim3((unsigned)((rows + RPB - 1) / RPB)), dim3(256), 0, st, a,
                     sp);
  return hipGetLastError() == hipSuccess ? BCATTN_OK : BCATTN_ERR_LAUNCH;
}

int launch_fwd_kvcache_bf16(const FwdArgs &a, const SplitArgs &sp_in, int D, hipStream_t st) {
  SplitArgs sp = sp_in;
  int ns, tps;
  plan_split(a.B, a.Sq, a.Sk, a.H, a.Hkv, &ns, &tps);
  if (ns <= 1) return launch_fwd_bf16(a, D, st);
  sp.nsplit = ns;
  sp.tiles_per_split = tps;
  switch (D) {
    case 64:
      return launch_split<64>(a, sp, st);
    case 128:
      return launch_split<128>(a, sp, st);
    case 256:
      return launch_split<256>(a, sp, st);
    default:
      return BCATTN_ERR_UNSUPPORTED;
  }
}

}  // namespace bcattn
