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
#include "bcattn_tiles.h"

namespace bcattn {

//
// SPLIT: the key tiles are divided over `nsplit` workgroups per row tile; each
// writes its unnormalised fp32 partial (O, running max, sum) and
// `fwd_combine_kernel` merges them.  This is what lets a handful of
// (batch, kv head) problems with few query rows fill the chip.
// LDS stages: three where they fit in the 160 KB of a CU, else two.
template <int D>
struct FwdStages {
  static constexpr int value = D <= 128 ? 3 : 2;
};

template <int D, int NW, bool SPLIT>
__global__ __launch_bounds__(64 * NW) void fwd_bf16_kernel(const FwdArgs a, const SplitArgs sp) {
  using T = Tile<D>;
  constexpr int NT = 64 * NW;   // threads
  constexpr int BM = 32 * NW;   // packed query rows per workgroup
  constexpr int DK = D / 16;    // contraction steps of K Q^T
  constexpr int DB = D / 32;    // 32-row blocks of O^T
  constexpr int STAGE = 2 * T::kBytes + 256;  // K tile, V tile, 64 key ids
  constexpr int NS = FwdStages<D>::value;

  extern __shared__ __align__(1024) char smem[];
  __shared__ int red_s[2 * NW];

  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
  const int n = lane & 31, hh = lane >> 5;

  const int R = a.G * a.Sq;
  const int ntile_r = (R + BM - 1) / BM;
  const int nitems = ntile_r * (SPLIT ? sp.nsplit : 1) * a.Hkv * a.B;
  int bid = xcd_item(blockIdx.x, nitems);
  if (bid >= nitems) return;
  const int tile = __builtin_amdgcn_readfirstlane(bid % ntile_r);
  bid /= ntile_r;
  const int split = SPLIT ? __builtin_amdgcn_readfirstlane(bid % sp.nsplit) : 0;
  if (SPLIT) bid /= sp.nsplit;
  // (division results live in vector registers; say that they are uniform)
  const int hk = __builtin_amdgcn_readfirstlane(bid % a.Hkv);
  const int b = __builtin_amdgcn_readfirstlane(bid / a.Hkv);

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

  // Key tiles never straddle the two key segments: tiles [0, nt0) cover segment 0,
  // tiles [nt0, nt0+nt1) segment 1, each padded (zero rows, invalid ids) at its end.
  const int nt0 = (a.Sk0 + 63) / 64;
  const int nt_all = nt0 + (a.Sk - a.Sk0 + 63) / 64;
  const int t_first = SPLIT ? split * sp.tiles_per_split : 0;
  const int nt = !any_g ? 0 : (SPLIT ? min(nt_all, t_first + sp.tiles_per_split) : nt_all);
  const tile_summary_t *ksum = a.ksum + (int64_t)b * nt_all;

  const bf16_t *k0b = reinterpret_cast<const bf16_t *>(a.k0.ptr) + b * a.k0.sb + hk * a.k0.sh;
  const bf16_t *v0b = reinterpret_cast<const bf16_t *>(a.v0.ptr) + b * a.v0.sb + hk * a.v0.sh;
  const bf16_t *k1b = reinterpret_cast<const bf16_t *>(a.k1.ptr) + b * a.k1.sb + hk * a.k1.sh;
  const bf16_t *v1b = reinterpret_cast<const bf16_t *>(a.v1.ptr) + b * a.v1.sb + hk * a.v1.sh;
  const int n0 = a.Sk0 > 0 ? a.Sk0 : 1, n1 = a.Sk - a.Sk0 > 0 ? a.Sk - a.Sk0 : 1;
  const buf_rsrc_t k0rs = make_rsrc(k0b, (uint32_t)(((int64_t)(n0 - 1) * a.k0.ss + D) * 2));
  const buf_rsrc_t v0rs = make_rsrc(v0b, (uint32_t)(((int64_t)(n0 - 1) * a.v0.ss + D) * 2));
  const buf_rsrc_t k1rs = make_rsrc(k1b, (uint32_t)(((int64_t)(n1 - 1) * a.k1.ss + D) * 2));
  const buf_rsrc_t v1rs = make_rsrc(v1b, (uint32_t)(((int64_t)(n1 - 1) * a.v1.ss + D) * 2));
  const buf_rsrc_t idrs =
      make_rsrc(a.kbm + (int64_t)b * nt_all * 64, (uint32_t)(nt_all * 64 * 4));
  TileLoad<D, NT> k0ld, v0ld, k1ld, v1ld;
  k0ld.init(tid, a.k0.ss);
  v0ld.init(tid, a.v0.ss);
  k1ld.init(tid, a.k1.ss);
  v1ld.init(tid, a.v1.ss);

  const_summary_t *ksum_s = scalar_view(ksum);
  // First tile at or after t that some row of the workgroup can see, with its summary.
  auto next_needed = [&](int t, tile_summary_t &sm) {
    while (t < nt) {
      sm = ksum_s[t];
      if (sm.x <= qmax_g) break;
      ++t;
    }
    return t;
  };
  auto issue = [&](int t, auto stage_c) {
    const char *st = smem + decltype(stage_c)::value * STAGE;
    if (t < nt0) {
      k0ld.issue(k0rs, st, (uint32_t)(t * 64 * a.k0.ss * 2), wave);
      v0ld.issue(v0rs, st + T::kBytes, (uint32_t)(t * 64 * a.v0.ss * 2), wave);
    } else {
      k1ld.issue(k1rs, st, (uint32_t)((t - nt0) * 64 * a.k1.ss * 2), wave);
      v1ld.issue(v1rs, st + T::kBytes, (uint32_t)((t - nt0) * 64 * a.v1.ss * 2), wave);
    }
    load_row64_dwords(idrs, st + 2 * T::kBytes, (uint32_t)t * 256, lane);  // every wave, same data
  };
  constexpr int LPT = 2 * TileLoad<D, NT>::kLoads + 1;  // loads per tile and wave

  RowAddr<D> rowa;
  rowa.init(lane);
  TrAddr<D> tra;
  tra.init(lane);

  // ---- running state ---------------------------------------------------------
  f32x16 o[DB];
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int x = 0; x < 16; ++x) o[db][x] = 0.f;
  float m = -INFINITY;  // running max of the raw (unscaled) scores
  float l = 0.f;        // this lane half's share of the running sum
  const float c = a.scale * kLog2e;

  auto compute = [&](auto stage_c, const tile_summary_t sm) {
    if (sm.x > qmax_w) return;  // wave-uniform: no row of this wave sees a key of the tile
#ifdef IGLP
    __builtin_amdgcn_iglp_opt(IGLP);
#endif
    const char *st = smem + decltype(stage_c)::value * STAGE;
    const char *Kt = st, *Vt = st + T::kBytes;
    const int *kb_s = reinterpret_cast<const int *>(st + 2 * T::kBytes);
    // Two independent accumulator chains (the two 32-key halves) are interleaved:
    // back-to-back products on one accumulator would each wait for the previous one.
    f32x16 s[2];
#pragma unroll
    for (int mb = 0; mb < 2; ++mb)
#pragma unroll
      for (int x = 0; x < 16; ++x) s[mb][x] = 0.f;
    {
      constexpr int KB = DK < 4 ? DK : 4;
#pragma unroll
      for (int k0 = 0; k0 < DK; k0 += KB) {
        bf16x8 ka0[KB], ka1[KB];
#pragma unroll
        for (int ks = 0; ks < KB; ++ks) {
          ka0[ks] = rowa.read(Kt, 0, k0 + ks);
          ka1[ks] = rowa.read(Kt, 32, k0 + ks);
        }
#pragma unroll
        for (int ks = 0; ks < KB; ++ks) {
          s[0] = mfma32(ka0[ks], qf[k0 + ks], s[0]);
          s[1] = mfma32(ka1[ks], qf[k0 + ks], s[1]);
        }
      }
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
    // O^T += V^T P^T: the DB accumulators are independent, so the key steps run outermost.
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) {
      constexpr int DBB = DB < 4 ? DB : 4;
#pragma unroll
      for (int d0 = 0; d0 < DB; d0 += DBB) {
        bf16x8 va[DBB];
#pragma unroll
        for (int db = 0; db < DBB; ++db) va[db] = tra.read(Vt, kk, d0 + db);
#pragma unroll
        for (int db = 0; db < DBB; ++db) o[d0 + db] = mfma32(va[db], pb[kk], o[d0 + db]);
      }
    }
  };

  // Two LDS stages: while tile t is being used, tile t+1 streams into the other one.
  tile_pipeline<NS, LPT>(t_first, nt, next_needed, issue, compute);

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

template <int D>
constexpr size_t fwd_smem_bytes() {
  return FwdStages<D>::value * (2 * (size_t)Tile<D>::kBytes + 256);
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

template <int D, int NW, bool SPLIT>
static int launch_fwd_t(const FwdArgs &a, const SplitArgs &sp, hipStream_t st) {
  if (hipFuncSetAttribute(reinterpret_cast<const void *>(&fwd_bf16_kernel<D, NW, SPLIT>),
                          hipFuncAttributeMaxDynamicSharedMemorySize, (int)fwd_smem_bytes<D>()) != hipSuccess)
    return BCATTN_ERR_LAUNCH;
  const int R = a.G * a.Sq;
  const int ntile_r = (R + 32 * NW - 1) / (32 * NW);
  hipLaunchKernelGGL((fwd_bf16_kernel<D, NW, SPLIT>),
                     dim3(xcd_grid((unsigned)(ntile_r * (SPLIT ? sp.nsplit : 1) * a.Hkv * a.B))), dim3(64 * NW),
                     fwd_smem_bytes<D>(), st, a, sp);
  return hipGetLastError() == hipSuccess ? BCATTN_OK : BCATTN_ERR_LAUNCH;
}

int launch_fwd_bf16(const FwdArgs &a, int D, hipStream_t st) {
  const int R = a.G * a.Sq;
  const SplitArgs sp{nullptr, nullptr, 1, 0};
  switch (D) {
    case 64:
      return launch_fwd_t<64, 4, false>(a, sp, st);
    case 128:
      return R >= 1024 ? launch_fwd_t<128, 8, false>(a, sp, st) : launch_fwd_t<128, 4, false>(a, sp, st);
    case 256:
      return launch_fwd_t<256, 4, false>(a, sp, st);
    default:
      return BCATTN_ERR_UNSUPPORTED;
  }
}

// How many ways to split the key axis so that about 1.5 workgroups per CU exist.
static void plan_split(int B, int Sq, int Sk0, int Sk, int H, int Hkv, int *nsplit, int *tps) {
  const int R = (H / Hkv) * Sq;
  const int base = B * Hkv * ((R + 127) / 128);
  const int ntiles = (Sk0 + 63) / 64 + (Sk - Sk0 + 63) / 64;
  int want = (384 + base - 1) / base;
  if (want < 1) want = 1;
  if (want > ntiles) want = ntiles;
  *tps = (ntiles + want - 1) / want;
  *nsplit = (ntiles + *tps - 1) / *tps;
}

size_t kvcache_workspace_bytes(int B, int Sq, int Sk0, int Sk, int H, int Hkv, int D, int *nsplit_out) {
  int ns, tps;
  plan_split(B, Sq, Sk0, Sk, H, Hkv, &ns, &tps);
  *nsplit_out = ns;
  if (ns <= 1) return 0;
  const size_t R = (size_t)(H / Hkv) * Sq;
  const size_t rows = (size_t)B * Hkv * ns * R;
  return ((rows * (D + 2) * sizeof(float)) + 255) & ~(size_t)255;
}

template <int D>
static int launch_split(const FwdArgs &a, const SplitArgs &sp, hipStream_t st) {
  const int R = a.G * a.Sq;
  const int rc = launch_fwd_t<D, 4, true>(a, sp, st);
  if (rc) return rc;
  constexpr int RPB = 256 / (D / 4);
  const int64_t rows = (int64_t)a.B * a.Hkv * R;
  hipLaunchKernelGGL(fwd_combine_kernel<D>, dim3((unsigned)((rows + RPB - 1) / RPB)), dim3(256), 0, st, a,
                     sp);
  return hipGetLastError() == hipSuccess ? BCATTN_OK : BCATTN_ERR_LAUNCH;
}

int launch_fwd_kvcache_bf16(const FwdArgs &a, const SplitArgs &sp_in, int D, hipStream_t st) {
  SplitArgs sp = sp_in;
  int ns, tps;
  plan_split(a.B, a.Sq, a.Sk0, a.Sk, a.H, a.Hkv, &ns, &tps);
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
