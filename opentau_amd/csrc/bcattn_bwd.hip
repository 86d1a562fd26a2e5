// Block-causal attention backward, bf16 in / fp32 accumulate, gfx950 MFMA.
//
// Three kernels, no atomics, so gradients are bit-repeatable:
//   prep    delta[b,h,i] = sum_d O*dO, and log2e*LSE (+inf on rows that take no
//           part), both padded to whole 64-row tiles so that the dK/dV kernel can
//           pull them into LDS with one buffer load
//   dQ      a workgroup owns 32*NW packed query rows and streams key tiles;
//           dQ^T = K^T dS^T with dS^T = P^T o (dP^T - delta), all keys x queries
//   dK/dV   a workgroup owns 128 keys of one kv head and streams the query tiles
//           of every query head of its group, so the sum over the GQA group
//           happens in registers; dV^T = dO^T P, dK^T = Q^T dS (queries x keys)
// P is recomputed from the saved log-sum-exp: P = exp2(scale*log2e*S - log2e*LSE).
//
// As in the forward, the 32x32 accumulator of the first product is already the B
// operand of the second, so P / dS never leave registers.  Streamed tiles go
// from global memory straight into swizzled LDS tiles (no registers, no LDS
// stores), double buffered; the operand that must be contracted over the
// sequence axis (K^T, Q^T, dO^T) is read from the same row-major tile with the
// transposing LDS read.
#include "bcattn_tiles.h"

namespace bcattn {

// ---- prep: delta and scaled LSE, padded -------------------------------------------
template <int D>
__global__ __launch_bounds__(256) void bwd_prep_kernel(const BwdArgs a) {
  constexpr int LPR = D / 8;
  constexpr int RPB = 256 / LPR;
  const int Sqp = a.Sq_pad;
  const int64_t total = (int64_t)a.B * a.H * Sqp;  // (b, h, i) with i fastest
  const int64_t row = (int64_t)blockIdx.x * RPB + threadIdx.x / LPR;
  const int c = threadIdx.x % LPR;
  float acc = 0.f;
  int h = 0, i = 0, b = 0;
  bool real = false;
  if (row < total) {
    i = (int)(row % Sqp);
    h = (int)((row / Sqp) % a.H);
    b = (int)(row / ((int64_t)Sqp * a.H));
    real = i < a.Sq;
    if (real) {
      const bf16x8 ov = *reinterpret_cast<const bf16x8 *>(reinterpret_cast<const bf16_t *>(a.o.ptr) +
                                                          b * a.o.sb + (int64_t)i * a.o.ss + h * a.o.sh + 8 * c);
      const bf16x8 gv = *reinterpret_cast<const bf16x8 *>(reinterpret_cast<const bf16_t *>(a.d_o.ptr) +
                                                          b * a.d_o.sb + (int64_t)i * a.d_o.ss +
                                                          h * a.d_o.sh + 8 * c);
#pragma unroll
      for (int e = 0; e < 8; ++e) acc += (float)ov[e] * (float)gv[e];
    }
  }
#pragma unroll
  for (int o = LPR / 2; o > 0; o >>= 1) acc += __shfl_xor(acc, o, 64);
  if (row < total && c == 0) {
    const bool ok = real && a.q_valid[(int64_t)b * a.Sq + i] != 0;
    a.delta[row] = ok ? acc : 0.f;
    a.lse2[row] = ok ? a.lse[((int64_t)b * a.H + h) * a.Sq + i] * kLog2e : INFINITY;
  }
}

// LDS stages: three where they fit in the 160 KB of a CU, else two.
template <int D>
struct BwdStages {
  static constexpr int value = D <= 128 ? 3 : 2;
};

// ---- dQ ------------------------------------------------------------------------
template <int D, int NW>
__global__ __launch_bounds__(64 * NW) void bwd_dq_kernel(const BwdArgs a) {
  using T = Tile<D>;
  constexpr int NT = 64 * NW, BM = 32 * NW;
  constexpr int DK = D / 16, DB = D / 32;
  constexpr int STAGE = 2 * T::kBytes + 256;  // K tile, V tile, 64 key ids
  constexpr int NS = BwdStages<D>::value;

  extern __shared__ __align__(1024) char smem[];
  __shared__ int red_s[2 * NW];

  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
  const int n = lane & 31, hh = lane >> 5;

  const int R = a.G * a.Sq;
  const int ntile_r = (R + BM - 1) / BM;
  const int nitems = ntile_r * a.Hkv * a.B;
  int bid = xcd_item(blockIdx.x, nitems);
  if (bid >= nitems) return;
  const int tile = __builtin_amdgcn_readfirstlane(bid % ntile_r);
  bid /= ntile_r;
  // (division results live in vector registers; say that they are uniform)
  const int hk = __builtin_amdgcn_readfirstlane(bid % a.Hkv);
  const int b = __builtin_amdgcn_readfirstlane(bid / a.Hkv);

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
  const bf16_t *gptr =
      reinterpret_cast<const bf16_t *>(a.d_o.ptr) + b * a.d_o.sb + (int64_t)i * a.d_o.ss + h * a.d_o.sh;
  bf16x8 qf[DK], gof[DK];
#pragma unroll
  for (int ks = 0; ks < DK; ++ks) {
    qf[ks] = *reinterpret_cast<const bf16x8 *>(qptr + 16 * ks + 8 * hh);
    gof[ks] = *reinterpret_cast<const bf16x8 *>(gptr + 16 * ks + 8 * hh);
  }
  const int64_t stat = ((int64_t)b * a.H + h) * a.Sq_pad + i;
  const float lse2 = rowok ? a.lse2[stat] : INFINITY;  // +inf on rows that take no part
  const float delta = rowok ? a.delta[stat] : 0.f;

  const int qmax_w = wave_max_i(qv ? qb : kIntMin);
  const int qmin_w = wave_min_i(qv ? qb : kIntMax);
  const int any_w = wave_max_i(qv ? 1 : 0);
  if (lane == 0) {
    red_s[wave] = qmax_w;
    red_s[NW + wave] = any_w;
  }
  const int nt_all = (a.Sk + 63) / 64;
  const tile_summary_t *ksum = a.ksum + (int64_t)b * nt_all;
  SummaryTable ktab;
  ktab.fill(ksum, reinterpret_cast<tile_summary_t *>(smem + NS * STAGE), nt_all, tid, NT);
  __syncthreads();
  int qmax_g = kIntMin, any_g = 0;
#pragma unroll
  for (int x = 0; x < NW; ++x) {
    qmax_g = max(qmax_g, red_s[x]);
    any_g |= red_s[NW + x];
  }
  // (values read from LDS count as per-lane; these are the same in every lane)
  qmax_g = __builtin_amdgcn_readfirstlane(qmax_g);
  any_g = __builtin_amdgcn_readfirstlane(any_g);

  const int Sk = a.Sk;
  const int nt = any_g ? nt_all : 0;

  const bf16_t *kbase = reinterpret_cast<const bf16_t *>(a.k.ptr) + b * a.k.sb + hk * a.k.sh;
  const bf16_t *vbase = reinterpret_cast<const bf16_t *>(a.v.ptr) + b * a.v.sb + hk * a.v.sh;
  const buf_rsrc_t krs = make_rsrc(kbase, (uint32_t)(((int64_t)(Sk - 1) * a.k.ss + D) * 2));
  const buf_rsrc_t vrs = make_rsrc(vbase, (uint32_t)(((int64_t)(Sk - 1) * a.v.ss + D) * 2));
  const buf_rsrc_t idrs =
      make_rsrc(a.kbm + (int64_t)b * nt_all * 64, (uint32_t)(nt_all * 64 * 4));
  TileLoad<D, NT> kld, vld;
  kld.init(tid, a.k.ss);
  vld.init(tid, a.v.ss);
  const uint32_t kstep = (uint32_t)(64 * a.k.ss * 2), vstep = (uint32_t)(64 * a.v.ss * 2);

  // A tile is needed if some row of the workgroup can see one of its keys.
  auto needed = [&](int t) { return ktab.at(t).x <= qmax_g; };
  const uint32_t smem0 = lds_addr(smem);
  auto issue = [&](int t, auto stage_c, auto, bool live) {
    const uint32_t st = smem0 + decltype(stage_c)::value * STAGE;
    kld.issue(rsrc_if(krs, live), st, (uint32_t)t * kstep, wave);
    vld.issue(rsrc_if(vrs, live), st + T::kBytes, (uint32_t)t * vstep, wave);
    load_row64_dwords(rsrc_if(idrs, live), st + 2 * T::kBytes, (uint32_t)t * 256, lane);  // every wave, same data
  };
  constexpr int LPT = 2 * TileLoad<D, NT>::kLoads + 1;  // loads per tile and wave

  RowAddr<D> rowa;
  rowa.init(lane);
  TrAddr<D> tra;
  tra.init(lane);

  f32x16 dq[DB];
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int x = 0; x < 16; ++x) dq[db][x] = 0.f;
  const float c = a.scale * kLog2e;

  auto compute = [&](auto stage_c, int t, auto bg) {
    const tile_summary_t sm = ktab.at(t);
    if (sm.x > qmax_w) return false;
    bg(StageC<0>{});  // wave-uniform: no row of this wave sees a key of the tile
    const char *st = smem + decltype(stage_c)::value * STAGE;
    const char *Kt = st, *Vt = st + T::kBytes;
    const int *kb_s = reinterpret_cast<const int *>(st + 2 * T::kBytes);
    const bool needmask = !(sm.z != 0 && sm.y <= qmin_w);
#pragma unroll
    for (int mb = 0; mb < 2; ++mb) {
      f32x16 s, dp;
#pragma unroll
      for (int x = 0; x < 16; ++x) s[x] = 0.f, dp[x] = 0.f;
      constexpr int KB = 2;  // operand reads issued ahead of the products
#pragma unroll
      for (int k0 = 0; k0 < DK; k0 += KB) {
        bf16x8 fa[KB], fb[KB];
#pragma unroll
        for (int ks = 0; ks < KB; ++ks) {
          fa[ks] = rowa.read(Kt, 32 * mb, k0 + ks);
          fb[ks] = rowa.read(Vt, 32 * mb, k0 + ks);
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
      for (int half = 0; half < 2; ++half) {
        bf16x8 ka[DB];
#pragma unroll
        for (int db = 0; db < DB; ++db) ka[db] = tra.read(Kt, 2 * mb + half, db);
#pragma unroll
        for (int db = 0; db < DB; ++db) dq[db] = mfma32(ka[db], dsb[half], dq[db]);
      }
    }
    return true;
  };

  // Two LDS stages: while tile t is being used, tile t+1 streams into the other one.
  settle_loads();
  tile_pipeline<NS, LPT, 1>(0, nt, needed, issue, compute);

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
  return BwdStages<D>::value * (2 * (size_t)Tile<D>::kBytes + 256);
}

// ---- dK / dV ---------------------------------------------------------------------
// MODE selects what a launch produces: both gradients (one pass, needs K and V
// fragments plus both accumulators in registers), or dV alone / dK alone (two
// launches that each recompute S; this is what fits the register file at
// head_dim 256, and at 128 it lets two waves share a SIMD).
constexpr int kModeBoth = 0, kModeDV = 1, kModeDK = 2;

// Spreads `parts` things over `slots` >= parts places in order: the part that belongs at
// slot s (part p sits at slot p*slots/parts), or -1.
constexpr int part_at_slot(int s, int slots, int parts) {
  for (int p = 0; p < parts; ++p)
    if (p * slots / parts == s) return p;
  return -1;
}

template <int D, int NW, int MODE>
__global__ __launch_bounds__(64 * NW) void bwd_dkv_kernel(const BwdArgs a) {
  using T = Tile<D>;
  constexpr bool WANT_DV = MODE != kModeDK, WANT_DK = MODE != kModeDV;
  constexpr int NT = 64 * NW, BK = 32 * NW;
  constexpr int DK = D / 16, DB = D / 32;
  constexpr int STAGE = 2 * T::kBytes + 3 * 256;  // Q tile, dO tile, lse2, delta, q ids
  constexpr int NS = BwdStages<D>::value;

  extern __shared__ __align__(1024) char smem[];
  __shared__ int red_s[NW];

  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
  const int n = lane & 31, hh = lane >> 5;

  const int Sk = a.Sk, Sq = a.Sq, Sqp = a.Sq_pad;
  const int nkt = (Sk + BK - 1) / BK;
  const int nitems = nkt * a.Hkv * a.B;
  int bid = xcd_item(blockIdx.x, nitems);
  if (bid >= nitems) return;
  const int kt = __builtin_amdgcn_readfirstlane(bid % nkt);
  bid /= nkt;
  // (division results live in vector registers; say that they are uniform)
  const int hk = __builtin_amdgcn_readfirstlane(bid % a.Hkv);
  const int b = __builtin_amdgcn_readfirstlane(bid / a.Hkv);

  // ---- this lane's key -----------------------------------------------------
  const int j = kt * BK + wave * 32 + n;
  const bool jok = j < Sk;
  const int jj = jok ? j : Sk - 1;
  const bool kv = jok && a.k_valid[(int64_t)b * Sk + jj] != 0;
  const int kb = kv ? a.k_blk[(int64_t)b * Sk + jj] : kIntMax;
  const bf16_t *kptr =
      reinterpret_cast<const bf16_t *>(a.k.ptr) + b * a.k.sb + (int64_t)jj * a.k.ss + hk * a.k.sh;
  const bf16_t *vptr =
      reinterpret_cast<const bf16_t *>(a.v.ptr) + b * a.v.sb + (int64_t)jj * a.v.ss + hk * a.v.sh;
  bf16x8 kf[DK], vf[WANT_DK ? DK : 1];
#pragma unroll
  for (int ks = 0; ks < DK; ++ks) {
    kf[ks] = *reinterpret_cast<const bf16x8 *>(kptr + 16 * ks + 8 * hh);
    if (WANT_DK) vf[ks] = *reinterpret_cast<const bf16x8 *>(vptr + 16 * ks + 8 * hh);
  }
  const int kmin_w = wave_min_i(kb);
  const int kmax_w = wave_max_i(kv ? kb : kIntMin);
  const int allk_w = wave_min_i(kv ? 1 : 0);
  if (lane == 0) red_s[wave] = kmin_w;
  const int nqt = a.Sq_pad / 64;
  const tile_summary_t *qsum = a.qsum + (int64_t)b * nqt;
  SummaryTable qtab;
  qtab.fill(qsum, reinterpret_cast<tile_summary_t *>(smem + NS * STAGE), nqt, tid, NT);
  __syncthreads();
  int kmin_g = kIntMax;
#pragma unroll
  for (int x = 0; x < NW; ++x) kmin_g = min(kmin_g, red_s[x]);
  // (values read from LDS count as per-lane; this one is the same in every lane)
  kmin_g = __builtin_amdgcn_readfirstlane(kmin_g);

  const int nit = (kmin_g == kIntMax) ? 0 : a.G * nqt;

  const bf16_t *qb0 = reinterpret_cast<const bf16_t *>(a.q.ptr) + b * a.q.sb + (int64_t)hk * a.G * a.q.sh;
  const bf16_t *gb0 =
      reinterpret_cast<const bf16_t *>(a.d_o.ptr) + b * a.d_o.sb + (int64_t)hk * a.G * a.d_o.sh;
  const uint32_t qbytes = (uint32_t)(((int64_t)(Sq - 1) * a.q.ss + D) * 2);
  const uint32_t gbytes = (uint32_t)(((int64_t)(Sq - 1) * a.d_o.ss + D) * 2);
  const int64_t stat0 = ((int64_t)b * a.H + (int64_t)hk * a.G) * Sqp;  // first row of (b, first head)
  // One statistics row of the tile per wave (lse, delta, query ids; further waves repeat
  // one): each wave keeps only the descriptor of the row it fetches.
  const int stat_kind = wave % 3;
  const buf_rsrc_t strs = stat_kind == 1   ? make_rsrc(a.delta + stat0, (uint32_t)(a.G * Sqp * 4))
                          : stat_kind == 2 ? make_rsrc(a.qbm + (int64_t)b * Sqp, (uint32_t)(Sqp * 4))
                                           : make_rsrc(a.lse2 + stat0, (uint32_t)(a.G * Sqp * 4));
  const uint32_t stat_dst = 2 * T::kBytes + 256 * stat_kind;
  TileLoad<D, NT> qld, gld;
  qld.init(tid, a.q.ss);
  gld.init(tid, a.d_o.ss);
  const uint32_t qstep = (uint32_t)(64 * a.q.ss * 2), gstep = (uint32_t)(64 * a.d_o.ss * 2);

  // Iterations run over (query head of the group, query tile), head-major.  The pipeline
  // asks about iterations in increasing order, so (head, tile) follow `it` by counting
  // instead of by division.
  int at_g = 0, at_base = 0;  // head of the iteration asked about last, and its first iteration
  auto seek = [&](int it) {
    int g = at_g, base = at_base;
    while (it >= base + nqt) base += nqt, ++g;
    at_g = __builtin_amdgcn_readfirstlane(g);
    at_base = __builtin_amdgcn_readfirstlane(base);
  };
  auto needed = [&](int it) {
    seek(it);
    const tile_summary_t sm = qtab.at(it - at_base);
    return sm.w > 0 && sm.y >= kmin_g;
  };
  const uint32_t smem0 = lds_addr(smem);
  // A tile is requested one load at a time (part p of LPT): the Q loads, the dO loads,
  // then the wave's statistics row.  Part 0 works out where the tile is.
  constexpr int KL = TileLoad<D, NT>::kLoads;
  constexpr int LPT = 2 * KL + 1;  // loads per tile and wave
  int req_g = 0, req_qt = 0;
  auto issue = [&](int it, auto stage_c, auto part_c, bool live) {
    constexpr int P = decltype(part_c)::value;
    const uint32_t st = smem0 + decltype(stage_c)::value * STAGE;
    if constexpr (P == 0) {
      // (the head asked about last is this tile's or a later one: count back)
      int g = at_g, qt = it - at_base;
      while (qt < 0) qt += nqt, --g;
      req_g = __builtin_amdgcn_readfirstlane(g), req_qt = __builtin_amdgcn_readfirstlane(qt);
    }
    // (descriptors are rebuilt where they are used: scalar registers are the scarce ones)
    if constexpr (P < KL) {
      qld.template issue_one<P>(make_rsrc(qb0 + (int64_t)req_g * a.q.sh, live ? qbytes : 0u), st,
                                (uint32_t)req_qt * qstep, wave);
    } else if constexpr (P < 2 * KL) {
      gld.template issue_one<P - KL>(make_rsrc(gb0 + (int64_t)req_g * a.d_o.sh, live ? gbytes : 0u), st + T::kBytes,
                                     (uint32_t)req_qt * gstep, wave);
    } else {
      const uint32_t row = stat_kind == 2 ? (uint32_t)(req_qt * 64) * 4 : (uint32_t)(req_g * Sqp + req_qt * 64) * 4;
      load_row64_dwords(rsrc_if(strs, live), st + stat_dst, row, lane);
    }
  };

  RowAddr<D> rowa;
  rowa.init(lane);
  TrAddr<D> tra;
  tra.init(lane);

  f32x16 dk[WANT_DK ? DB : 1], dv[WANT_DV ? DB : 1];
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int x = 0; x < 16; ++x) {
      if (WANT_DK) dk[db][x] = 0.f;
      if (WANT_DV) dv[db][x] = 0.f;
    }
  const float c = a.scale * kLog2e;

  // One query tile, software-pipelined inside the wave so that the vector ALU work
  // of one 32-query half runs in the shadow of the other half's matrix products:
  //   A0 | A1 + softmax0 | C0 + softmax1 | C1
  // A(mb): S = Q K^T and dP = dO V^T of queries 32mb.. (row operands from LDS)
  // softmax(mb): P = exp2(c S - log2e LSE), dS = P o (dP - delta), packed to bf16
  // C(mb): dV^T += dO^T P, dK^T += Q^T dS (transposed operands from LDS)
  // The scheduler is given the interleaving explicitly (sched_group_barrier:
  // 0x008 matrix, 0x100 LDS read, 0x002 vector ALU); MASKED is a compile-time copy
  // of "some pair of this tile may be masked", so the common case carries no
  // compare/select at all.
  auto compute_t = [&](auto stage_c, auto masked_c, auto bg) {
    constexpr bool MASKED = decltype(masked_c)::value != 0;
    const char *st = smem + decltype(stage_c)::value * STAGE;
    const char *Qt = st, *Gt = st + T::kBytes;
    const float *lse_s = reinterpret_cast<const float *>(st + 2 * T::kBytes);
    const float *delta_s = lse_s + 64;
    const int *qb_s = reinterpret_cast<const int *>(delta_s + 64);
    f32x16 s[2], dp[WANT_DK ? 2 : 1];
    bf16x8 pb[2][2], dsb[2][2];

    // The loads of the tile due in this step go out one at a time between the products
    // of the two A phases.
    auto phase_a = [&](auto mb_c) {
      constexpr int mb = decltype(mb_c)::value;
#pragma unroll
      for (int x = 0; x < 16; ++x) {
        s[mb][x] = 0.f;
        if (WANT_DK) dp[mb][x] = 0.f;
      }
      static_for<DK>([&](auto ks_c) {
        constexpr int ks = decltype(ks_c)::value;
        constexpr int part = part_at_slot(mb * DK + ks, 2 * DK, LPT);
        if constexpr (part >= 0) bg(StageC<part>{});
        s[mb] = mfma32(rowa.read(Qt, 32 * mb, ks), kf[ks], s[mb]);
        if (WANT_DK) dp[mb] = mfma32(rowa.read(Gt, 32 * mb, ks), vf[ks], dp[mb]);
      });
    };
    auto softmax = [&](int mb) {
#pragma unroll
      for (int half = 0; half < 2; ++half) {
        float p[8], ds[8];
#pragma unroll
        for (int r2 = 0; r2 < 2; ++r2) {
          const int r4 = 2 * half + r2;
          const int q0 = 32 * mb + 8 * r4 + 4 * hh;
          const f32x4 lse4 = *reinterpret_cast<const f32x4 *>(lse_s + q0);
          f32x4 del4 = {0.f, 0.f, 0.f, 0.f};
          if (WANT_DK) del4 = *reinterpret_cast<const f32x4 *>(delta_s + q0);
          i32x4 qb4 = {0, 0, 0, 0};
          if (MASKED) qb4 = *reinterpret_cast<const i32x4 *>(qb_s + q0);
#pragma unroll
          for (int x = 0; x < 4; ++x) {
            float pv = fast_exp2(s[mb][4 * r4 + x] * c - lse4[x]);
            if (MASKED && kb > qb4[x]) pv = 0.f;
            p[4 * r2 + x] = pv;
            if (WANT_DK) ds[4 * r2 + x] = pv * (dp[mb][4 * r4 + x] - del4[x]);
          }
        }
        if (WANT_DV) pb[mb][half] = pack8(p[0], p[1], p[2], p[3], p[4], p[5], p[6], p[7]);
        if (WANT_DK) dsb[mb][half] = pack8(ds[0], ds[1], ds[2], ds[3], ds[4], ds[5], ds[6], ds[7]);
      }
    };
    auto phase_c = [&](int mb) {
#pragma unroll
      for (int half = 0; half < 2; ++half)
#pragma unroll
        for (int db = 0; db < DB; ++db) {
          if (WANT_DV) dv[db] = mfma32(tra.read(Gt, 2 * mb + half, db), pb[mb][half], dv[db]);
          if (WANT_DK) dk[db] = mfma32(tra.read(Qt, 2 * mb + half, db), dsb[mb][half], dk[db]);
        }
    };
    constexpr int PER = (WANT_DV ? 1 : 0) + (WANT_DK ? 1 : 0);
    constexpr int NA = PER == 2 ? 2 * DK : (WANT_DK ? 2 * DK : DK);  // products of one A phase
    constexpr int NC = 2 * DB * PER;                                  // products of one C phase
    constexpr int VA = (MASKED ? 9 : 7) * 16 / (NA < NC ? NA : NC) + 1;  // vector ALU instr. per product

    phase_a(StageC<0>{});
    {
      constexpr int kAhead = NA < 6 ? NA : 6;
      __builtin_amdgcn_sched_group_barrier(0x100, kAhead, 0);
#pragma unroll
      for (int x = 0; x < NA - kAhead; ++x) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
      }
      __builtin_amdgcn_sched_group_barrier(0x008, kAhead, 0);
    }
    __builtin_amdgcn_sched_barrier(0);

    phase_a(StageC<1>{});
    softmax(0);
    {
      constexpr int kAhead = NA < 4 ? NA : 4;
      __builtin_amdgcn_sched_group_barrier(0x100, kAhead, 0);
#pragma unroll
      for (int x = 0; x < NA; ++x) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);  // next operand + statistics reads
        __builtin_amdgcn_sched_group_barrier(0x002, VA, 0);
      }
    }
    __builtin_amdgcn_sched_barrier(0);

    phase_c(0);
    softmax(1);
    {
      constexpr int kAhead = NC < 4 ? NC : 4;
      __builtin_amdgcn_sched_group_barrier(0x100, 2 * kAhead, 0);
#pragma unroll
      for (int x = 0; x < NC; ++x) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, 3, 0);
        __builtin_amdgcn_sched_group_barrier(0x002, VA, 0);
      }
    }
    __builtin_amdgcn_sched_barrier(0);

    phase_c(1);
    {
      constexpr int kAhead = NC < 4 ? NC : 4;
      __builtin_amdgcn_sched_group_barrier(0x100, 2 * kAhead, 0);
#pragma unroll
      for (int x = 0; x < NC - kAhead; ++x) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
      }
      __builtin_amdgcn_sched_group_barrier(0x008, kAhead, 0);
    }
    __builtin_amdgcn_sched_barrier(0);
  };
  auto compute = [&](auto stage_c, int it, auto bg) {
    // (the head of iteration `it` is at most the one asked about last: count its tiles back)
    int qt = it - at_base;
    while (qt < 0) qt += nqt;
    const tile_summary_t sm = qtab.at(__builtin_amdgcn_readfirstlane(qt));
    if (sm.y < kmin_w) return false;  // wave-uniform: no key of this wave is seen by the tile
    if (sm.z != 0 && allk_w != 0 && kmax_w <= sm.x)
      compute_t(stage_c, StageC<0>{}, bg);  // every pair of the tile attends
    else
      compute_t(stage_c, StageC<1>{}, bg);
    return true;
  };

  settle_loads();
  tile_pipeline<NS, LPT, LPT>(0, nit, needed, issue, compute);

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
          if (WANT_DK) wk[x] = (bf16_t)(dk[db][4 * r4 + x] * a.scale);
          if (WANT_DV) wv[x] = (bf16_t)dv[db][4 * r4 + x];
        }
        if (WANT_DK) *reinterpret_cast<bf16x4 *>(dkp + 32 * db + 8 * r4 + 4 * hh) = wk;
        if (WANT_DV) *reinterpret_cast<bf16x4 *>(dvp + 32 * db + 8 * r4 + 4 * hh) = wv;
      }
  }
}

template <int D>
constexpr size_t dkv_smem_bytes() {
  return BwdStages<D>::value * (2 * (size_t)Tile<D>::kBytes + 3 * 256);
}

template <int D, int NW, int MODE>
static int launch_dkv(const BwdArgs &a, hipStream_t st) {
  if (!allow_dynamic_lds<&bwd_dkv_kernel<D, NW, MODE>>((int)(kLdsBytes - 1024))) return BCATTN_ERR_LAUNCH;
  if (!summary_table_fits(dkv_smem_bytes<D>(), a.Sq_pad / 64)) return BCATTN_ERR_UNSUPPORTED;
  const size_t smem = dkv_smem_bytes<D>() + (size_t)(a.Sq_pad / 64) * sizeof(tile_summary_t);
  const int nkt = (a.Sk + 32 * NW - 1) / (32 * NW);
  hipLaunchKernelGGL((bwd_dkv_kernel<D, NW, MODE>), dim3(xcd_grid((unsigned)(nkt * a.Hkv * a.B))),
                     dim3(64 * NW), smem, st, a);
  return hipGetLastError() == hipSuccess ? BCATTN_OK : BCATTN_ERR_LAUNCH;
}

// NWQ: waves of the dQ kernel; NWK, SPLIT: waves of the dK/dV kernel and whether it
// runs as two launches (dV, then dK).
template <int D, int NWQ, int NWK, bool SPLIT>
static int launch_bwd_d(const BwdArgs &a, hipStream_t st) {
  if (!allow_dynamic_lds<&bwd_dq_kernel<D, NWQ>>((int)(kLdsBytes - 1024))) return BCATTN_ERR_LAUNCH;
  if (!summary_table_fits(dq_smem_bytes<D>(), (a.Sk + 63) / 64)) return BCATTN_ERR_UNSUPPORTED;
  if (a.stages & BCATTN_BWD_DELTA) {
    constexpr int RPB = 256 / (D / 8);
    const int64_t rows = (int64_t)a.B * a.H * a.Sq_pad;
    hipLaunchKernelGGL(bwd_prep_kernel<D>, dim3((unsigned)((rows + RPB - 1) / RPB)), dim3(256), 0, st, a);
  }
  if (a.stages & BCATTN_BWD_DQ) {
    const int R = a.G * a.Sq;
    const int ntile_r = (R + 32 * NWQ - 1) / (32 * NWQ);
    const size_t smem = dq_smem_bytes<D>() + (size_t)((a.Sk + 63) / 64) * sizeof(tile_summary_t);
    hipLaunchKernelGGL((bwd_dq_kernel<D, NWQ>), dim3(xcd_grid((unsigned)(ntile_r * a.Hkv * a.B))), dim3(64 * NWQ),
                       smem, st, a);
  }
  if (a.stages & BCATTN_BWD_DKV) {
    int rc;
    if (SPLIT) {
      if ((rc = launch_dkv<D, NWK, kModeDV>(a, st)) || (rc = launch_dkv<D, NWK, kModeDK>(a, st))) return rc;
    } else if ((rc = launch_dkv<D, NWK, kModeBoth>(a, st))) {
      return rc;
    }
  }
  return hipGetLastError() == hipSuccess ? BCATTN_OK : BCATTN_ERR_LAUNCH;
}

int launch_bwd_bf16(const BwdArgs &a, int D, hipStream_t st) {
  const int R = a.G * a.Sq;
  switch (D) {
    case 64:
      return launch_bwd_d<64, 4, 4, false>(a, st);
    case 128:
      return R >= 1024 ? launch_bwd_d<128, 8, 4, false>(a, st) : launch_bwd_d<128, 4, 4, false>(a, st);
    case 256:
      return launch_bwd_d<256, 4, 4, true>(a, st);
    default:
      return BCATTN_ERR_UNSUPPORTED;
  }
}

}  // namespace bcattn
