// LDS tiles of the MFMA kernels: 64 rows x D bf16, filled by buffer loads that
// write LDS directly, read either as row operands (16-byte reads) or as
// transposed operands (ds_read_b64_tr_b16), with one XOR swizzle that keeps both
// kinds of read free of bank conflicts.
#pragma once

#include "bcattn_common.h"

namespace bcattn {

typedef __attribute__((address_space(3))) void lds_void_t;
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) s16x4 lds_s16x4_t;

// A 64 x D tile.  Row r occupies bytes [r*2D, (r+1)*2D); inside the row the
// 16-byte slot that holds columns 8L..8L+7 sits at slot L ^ swz(r).
//
// Row reads: 16 lanes read the same logical slot of 16 consecutive rows; swz is
// a bijection of (r mod 16) [of (r/2 mod 8) for D=64, whose rows are 128 bytes],
// so they land in 16 different slots = all 64 banks.
// Transposed reads: 32 lanes read two adjacent slots of 4 consecutive rows (two
// 16-lane groups, the second two slots further); swz>>1 takes 4 different
// values on 4 consecutive rows, so the 8 slot pairs are again all 64 banks.
template <int D>
struct Tile {
  static constexpr int kSlotsPerRow = D / 8;
  static constexpr int kRowBytes = 2 * D;
  static constexpr int kBytes = 64 * kRowBytes;
  static constexpr int kSlots = 64 * kSlotsPerRow;

  __device__ __forceinline__ static int swz(int r) {
    if (D == 64) return (((r >> 1) & 1) << 2) | (((r >> 2) & 1) << 1) | ((r >> 3) & 1);
    return ((r & 3) << 2) | ((r >> 2) & 3);
  }
  // Byte offset of logical slot L of row r.
  __device__ __forceinline__ static int off(int r, int L) { return r * kRowBytes + 16 * (L ^ swz(r)); }
};

// Buffer descriptor over `bytes` bytes at p (loads past the end return zero), in
// scalar registers.  Base and size are the same in every lane; reading them from
// the first lane is what puts them in scalar registers.
typedef i32x4 buf_rsrc_t;
__device__ __forceinline__ buf_rsrc_t make_rsrc(const void *p, uint32_t bytes) {
  const uint64_t addr = reinterpret_cast<uint64_t>(p);
  buf_rsrc_t r;
  r[0] = __builtin_amdgcn_readfirstlane((int)(uint32_t)addr);
  r[1] = __builtin_amdgcn_readfirstlane((int)((uint32_t)(addr >> 32) & 0xffffu));
  r[2] = __builtin_amdgcn_readfirstlane((int)bytes);
  r[3] = 0x00020000;  // raw buffer, 32-bit data format
  return r;
}

// Byte address of an LDS location, as the hardware counts it.
__device__ __forceinline__ uint32_t lds_addr(const void *p) {
  return (uint32_t)(uintptr_t)((__attribute__((address_space(3))) const char *)p);
}

// Asynchronous global -> LDS copy, 16 (or 4) bytes per lane: lane l reads
// base + voff + soff and writes LDS byte lds_base + 16*l (4*l).  Issued as
// assembly so that the compiler does not order later LDS reads of the *other*
// stage behind it; completion is awaited explicitly with wait_async_loads().
__device__ __forceinline__ void dma16(buf_rsrc_t rsrc, uint32_t lds_base, uint32_t voff, uint32_t soff) {
  asm volatile(
      "s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
      :
      : "s"(lds_base), "v"(voff), "s"(rsrc), "s"(soff)
      : "memory", "m0");
}
__device__ __forceinline__ void dma4(buf_rsrc_t rsrc, uint32_t lds_base, uint32_t voff, uint32_t soff) {
  asm volatile(
      "s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dword %1, %2, %3 offen lds"
      :
      : "s"(lds_base), "v"(voff), "s"(rsrc), "s"(soff)
      : "memory", "m0");
}

// Per-thread source offsets of an asynchronous tile load.  The tile's kSlots
// 16-byte slots are covered by kSlots/NT loads per thread; load x of wave w
// fills the 64 consecutive LDS slots (x*NT + 64*w) .. +63, lane l the l-th, and
// fetches the matching (row, logical slot) of the source.
template <int D, int NT>
struct TileLoad {
  static constexpr int kLoads = Tile<D>::kSlots / NT;
  static_assert(Tile<D>::kSlots % NT == 0, "tile slots must divide over the threads");
  uint32_t voff[kLoads];

  __device__ __forceinline__ void init(int tid, int64_t row_stride_elems) {
#pragma unroll
    for (int x = 0; x < kLoads; ++x) {
      const int s = x * NT + tid;
      const int row = s / Tile<D>::kSlotsPerRow, P = s % Tile<D>::kSlotsPerRow;
      const int L = P ^ Tile<D>::swz(row);
      voff[x] = (uint32_t)(row * row_stride_elems * 2 + L * 16);
    }
  }
  // `tile` is the LDS tile base, `soff` the byte offset of the tile's first row.
  __device__ __forceinline__ void issue(buf_rsrc_t rsrc, const char *tile, uint32_t soff, int wave) const {
    const uint32_t base = __builtin_amdgcn_readfirstlane(lds_addr(tile) + 1024u * (uint32_t)wave);
    const uint32_t so = __builtin_amdgcn_readfirstlane(soff);
#pragma unroll
    for (int x = 0; x < kLoads; ++x) dma16(rsrc, base + (uint32_t)(x * NT * 16), voff[x], so);
  }
};

// 64 consecutive dwords -> LDS, one per lane (a whole wave must call it).
__device__ __forceinline__ void load_row64_dwords(buf_rsrc_t rsrc, const void *dst, uint32_t soff, int lane) {
  dma4(rsrc, __builtin_amdgcn_readfirstlane(lds_addr(dst)), (uint32_t)lane * 4,
       __builtin_amdgcn_readfirstlane(soff));
}

__device__ __forceinline__ void wait_async_loads() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }

// ---------------------------------------------------------------------------
// Operand reads.  The swizzle makes a read address a per-lane XOR pattern rather
// than base + constant, so each lane computes its offsets once, before the main
// loop; in the loop an address is (precomputed lane offset) + (compile-time
// tile / stage / block constant), which folds into the instruction's immediate.
// ---------------------------------------------------------------------------

// Row operand of a 32x32x16 product: row (rbase + lane%32), columns
// 16*ks + 8*(lane/32) .. +7.  rbase must be a multiple of 16 rows.
template <int D>
struct RowAddr {
  int a[D / 16];
  __device__ __forceinline__ void init(int lane) {
    const int n = lane & 31, hh = lane >> 5;
#pragma unroll
    for (int ks = 0; ks < D / 16; ++ks) a[ks] = Tile<D>::off(n, 2 * ks + hh);
  }
  __device__ __forceinline__ bf16x8 read(const char *tile, int rbase, int ks) const {
    return *reinterpret_cast<const bf16x8 *>(tile + rbase * Tile<D>::kRowBytes + a[ks]);
  }
};

// Transposed operand: for output row d = 32*db + lane%32 the 8 sequence positions
//   16*kk + 8*(e/4) + 4*(lane/32) + e%4,  e = 0..7
// of a row-major tile (positions are tile rows), i.e. exactly the positions whose
// values a lane holds in registers 8*half .. 8*half+7 of a 32x32 accumulator.
// Two ds_read_b64_tr_b16: within 16 lanes, lane i receives, from the 8-byte rows
// the 16 lanes point at, element (i%4) of rows 4e + i/4 -- a 4x16 transpose.  So
// lane i of a group points at row 4*(lane/32) + i/4 (+8 for the second read),
// columns 32*db + 16*(group%2) + 4*(i%4) .. +3.
template <int D>
struct TrAddr {
  int lo[D / 32], hi[D / 32];
  __device__ __forceinline__ void init(int lane) {
    const int i = lane & 15, grp = (lane >> 4) & 1, hh = lane >> 5;
    const int row = 4 * hh + (i >> 2);
    const int slot = 2 * grp + ((i & 3) >> 1);
    const int byte = 8 * (i & 1);
#pragma unroll
    for (int db = 0; db < D / 32; ++db) {
      lo[db] = Tile<D>::off(row, 4 * db + slot) + byte;
      hi[db] = Tile<D>::off(row + 8, 4 * db + slot) + byte;
    }
  }
  __device__ __forceinline__ bf16x8 read(const char *tile, int kk, int db) const {
    const char *base = tile + 16 * kk * Tile<D>::kRowBytes;
    const s16x4 l = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_t *)(base + lo[db]));
    const s16x4 h = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_t *)(base + hi[db]));
    typedef short s16x8 __attribute__((ext_vector_type(8)));
    const s16x8 both = __builtin_shufflevector(l, h, 0, 1, 2, 3, 4, 5, 6, 7);
    return __builtin_bit_cast(bf16x8, both);
  }
};

// Compile-time stage index, so that stage offsets fold into immediates.
template <int S>
struct StageC {
  static constexpr int value = S;
};

// Tile summaries are read with scalar loads (uniform address, memory that no
// kernel writes while this one runs): they come back through the scalar cache
// and do not queue behind the asynchronous tile loads.
typedef const __attribute__((address_space(4))) tile_summary_t const_summary_t;
__device__ __forceinline__ const_summary_t *scalar_view(const tile_summary_t *p) {
  return (const_summary_t *)reinterpret_cast<uintptr_t>(p);
}

// Wait until at most N of this wave's asynchronous loads are still in flight.
template <int N>
__device__ __forceinline__ void wait_async_loads_but() {
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}
// Workgroup barrier without the fence of __syncthreads(): the tile data it orders
// was already awaited by each wave (wait_async_loads*), and a fence would drain
// the loads that are meant to stay in flight.
__device__ __forceinline__ void tile_barrier() { asm volatile("s_barrier" ::: "memory"); }

// Walk the needed tiles of [first, end) with NS LDS stages, i.e. NS-1 tiles of
// asynchronous loads in flight while one is computed on.
//   next(t, sm)        first needed tile >= t (or end) and its summary
//   issue(t, StageC)   start the loads of tile t into that stage; every wave must
//                      issue exactly LPT loads
//   compute(StageC, sm)
// The loop is written out over the stages so that every LDS address inside
// compute() is a lane offset plus a compile-time constant.
template <int NS, int LPT, class Next, class Issue, class Compute>
__device__ __forceinline__ void tile_pipeline(int first, int end, Next next, Issue issue, Compute compute) {
  static_assert(NS == 2 || NS == 3, "two or three stages");
  tile_summary_t s0 = {0, 0, 0, 0}, s1 = s0, s2 = s0;
  int t0 = next(first, s0);
  if (t0 >= end) return;
  issue(t0, StageC<0>{});
  int t1 = end, t2 = end;
  if (NS == 3) {
    t1 = next(t0 + 1, s1);
    if (t1 < end) issue(t1, StageC<1>{});
  }
  auto step = [&](auto sc) {
    constexpr int S = decltype(sc)::value;
    if (NS == 2) {
      t1 = next(t0 + 1, s1);
      wait_async_loads_but<0>();
      tile_barrier();
      if (t1 < end) issue(t1, StageC<(S + 1) % 2>{});
      compute(sc, s0);
      t0 = t1, s0 = s1;
    } else {
      t2 = t1 < end ? next(t1 + 1, s2) : end;
      if (t1 < end)
        wait_async_loads_but<LPT>();  // the newer tile may still be in flight
      else
        wait_async_loads_but<0>();
      tile_barrier();
      if (t2 < end) issue(t2, StageC<(S + 2) % 3>{});
      compute(sc, s0);
      t0 = t1, s0 = s1, t1 = t2, s1 = s2;
    }
    return t0 >= end;
  };
  for (;;) {
    if (step(StageC<0>{})) break;
    if (step(StageC<1>{})) break;
    if (NS == 3)
      if (step(StageC<2>{})) break;
  }
}

// Short tile ranges (a split of the key axis): the tiles [first, end) are taken in
// order, none is skipped, and as many as there are LDS stages are requested at once,
// so that a range of at most NS tiles pays the memory latency once.  The caller has
// already requested the first min(NS, end - first) tiles into stages 0.. (it can do
// that before it knows anything else); tile_burst() requests the rest as stages
// free up.   issue(t, StageC) / compute(StageC, t) as for tile_pipeline.
template <int K, int LPT>
__device__ __forceinline__ void wait_async_tiles_but(int newer) {
  // wait until at most `newer` (0..K) whole tiles of this wave's loads are in flight
  if constexpr (K == 0) {
    wait_async_loads_but<0>();
  } else {
    if (newer >= K)
      wait_async_loads_but<K * LPT>();
    else
      wait_async_tiles_but<K - 1, LPT>(newer);
  }
}
template <int NS, int LPT, class Issue, class Compute>
__device__ __forceinline__ void tile_burst(int first, int end, Issue issue, Compute compute) {
  static_assert(NS >= 2 && NS * LPT <= 63 + LPT, "wait counts are 6-bit immediates");
  int t = first;
  auto step = [&](auto sc) {
    constexpr int S = decltype(sc)::value;
    // tiles requested after t so far: up to first+NS-1 at the start, t+NS-2 later
    const int last_req = min(end - 1, t == first ? first + NS - 1 : t + NS - 2);
    wait_async_tiles_but<NS - 1, LPT>(last_req - t);
    tile_barrier();  // tile t is in LDS for every wave, and every wave is done with tile t-1
    if (t > first && t - 1 + NS < end) issue(t - 1 + NS, StageC<(S + NS - 1) % NS>{});
    compute(sc, t);
    return ++t >= end;
  };
  if (t >= end) return;
  for (;;) {
    if (step(StageC<0>{})) break;
    if (step(StageC<1>{})) break;
    if constexpr (NS >= 3)
      if (step(StageC<2>{})) break;
    if constexpr (NS >= 4)
      if (step(StageC<3>{})) break;
    static_assert(NS <= 4, "at most four stages");
  }
}

}  // namespace bcattn
