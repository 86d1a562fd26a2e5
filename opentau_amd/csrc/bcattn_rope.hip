// Rotary position embedding of queries and keys (with an optional per-head RMS norm in
// front): an elementwise pass bound by HBM, read once and written once.
//
// A workgroup takes a few tokens.  Phase 1: one thread per (token, band) computes the sine
// and cosine of that band's angle, once for all heads, into LDS.  Phase 2: the threads walk
// over the (token, head, 16-byte piece) items; an item is a piece of the first half of a row
// and the matching piece of the second half.  Consecutive lanes take consecutive pieces of a
// row and then the next head, so with heads stored side by side a wave's loads and stores
// cover one contiguous span.  The first items are requested before phase 1, so the trigonometry
// runs under their latency.
#include "bcattn_common.h"

namespace bcattn {

template <typename T, int V>
struct Vec {
  T v[V];
} __attribute__((aligned(16)));

constexpr int kRopeThreads = 256;
constexpr int kRopeUnroll = 2;  // items a thread has in flight
// Tokens per workgroup: enough for about this many items (measured: 600 to 1200 items per
// workgroup run fastest at every shape tried; fewer leave the barrier and the trigonometry
// exposed, more leave the last workgroups of a CU running alone), within 32 KB of LDS.
constexpr int kRopeItems = 1024;
inline int rope_tokens(int D, int items_per_token) {
  const int want = (kRopeItems + items_per_token / 2) / items_per_token;
  const int fit = 8192 / D;
  return want < 1 ? 1 : (want > fit ? fit : want);
}

template <typename T, int V>
struct RopeItem {
  const T *src;
  T *dst;
  const T *wgt;  // norm weights of the row's tensor, or null
  int t;         // token slot in the workgroup
  bool live;
};

template <typename T, int V>
__device__ __forceinline__ RopeItem<T, V> rope_item(const RopeArgs &a, int item, int nitems, int tok0, int ntok,
                                                    int lpr) {
  // item = (token slot, row, piece), piece fastest; rows: the heads of q, then those of k
  const int rows = (a.q.ptr ? a.H : 0) + (a.k.ptr ? a.Hkv : 0);
  RopeItem<T, V> it;
  const int c = item % lpr;
  const int rest = item / lpr;
  const int row = rest % rows;
  it.t = rest / rows;
  const int64_t tok = (int64_t)tok0 + it.t;
  it.live = item < nitems && tok < ntok;
  const int b = it.live ? (int)(tok / a.L) : 0, l = it.live ? (int)(tok % a.L) : 0;
  const int nq = a.q.ptr ? a.H : 0;
  const bool is_k = row >= nq;
  const TensorArg &in = is_k ? a.k : a.q;
  const TensorArg &out = is_k ? a.k_out : a.q_out;
  const int h = is_k ? row - nq : row;
  it.src = reinterpret_cast<const T *>(in.ptr) + b * in.sb + (int64_t)l * in.ss + h * in.sh + c * V;
  it.dst = reinterpret_cast<T *>(const_cast<void *>(out.ptr)) + b * out.sb + (int64_t)l * out.ss + h * out.sh + c * V;
  const void *w = is_k ? a.k_w : a.q_w;
  it.wgt = w ? reinterpret_cast<const T *>(w) + c * V : nullptr;
  return it;
}

template <typename T, int V>
__global__ __launch_bounds__(kRopeThreads) void rope_kernel(const RopeArgs a, const int TB) {
#pragma clang fp contract(off)  // products and sums rounded one by one, as a framework's elementwise ops do
  extern __shared__ __align__(16) float trig[];  // [tokens][half] sines, then as many cosines
  const int tid = threadIdx.x;
  const int half = a.D / 2;
  const int lpr = half / V;  // lanes (pieces) per row
  const int ntok = a.B * a.L;
  const int tok0 = blockIdx.x * TB;
  const int rows = (a.q.ptr ? a.H : 0) + (a.k.ptr ? a.Hkv : 0);
  const int nitems = TB * rows * lpr;
  float *sin_s = trig, *cos_s = trig + TB * half;

  RopeItem<T, V> it[kRopeUnroll];
  Vec<T, V> x1[kRopeUnroll], x2[kRopeUnroll];
  auto request = [&](int first) __attribute__((always_inline)) {
#pragma unroll
    for (int u = 0; u < kRopeUnroll; ++u) {
      it[u] = rope_item<T, V>(a, first + u * kRopeThreads, nitems, tok0, ntok, lpr);
      if (it[u].live) {
        x1[u] = *reinterpret_cast<const Vec<T, V> *>(it[u].src);
        x2[u] = *reinterpret_cast<const Vec<T, V> *>(it[u].src + half);
      }
    }
  };
  request(tid);

  // ---- phase 1: one (token, band) pair per thread and step ----------------------------------
  for (int p = tid; p < TB * half; p += kRopeThreads) {
    const int t = p / half, band = p % half;
    const int64_t tok = (int64_t)tok0 + t;
    float sn = 0.f, cs = 1.f;
    if (tok < ntok) {
      const int b = (int)(tok / a.L), l = (int)(tok % a.L);
      const int axis = a.n_axes > 1 ? band % a.n_axes : 0;
      const float pos = (float)a.positions[((int64_t)axis * a.B + b) * a.L + l];
      const float ang = __fdiv_rn(pos, a.timescale[band]);
      sincosf(ang, &sn, &cs);
      if (a.inverse) sn = -sn;
    }
    sin_s[p] = sn;
    cos_s[p] = cs;
  }
  // LDS writes done, then the barrier; the requested rows stay in flight across it
  asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");

  // ---- phase 2 --------------------------------------------------------------------------------
  for (int first = tid; first < nitems; first += kRopeUnroll * kRopeThreads) {
    if (first != tid) request(first);
#pragma unroll
    for (int u = 0; u < kRopeUnroll; ++u) {
      if (!it[u].live) continue;
      float f1[V], f2[V];
#pragma unroll
      for (int e = 0; e < V; ++e) {
        f1[e] = (float)x1[u].v[e];
        f2[e] = (float)x2[u].v[e];
      }
      if (it[u].wgt != nullptr) {
        // The lpr lanes of a row are neighbours, aligned to lpr (a power of two here), and take
        // this branch together.
        float ss = 0.f;
#pragma unroll
        for (int e = 0; e < V; ++e) ss += f1[e] * f1[e] + f2[e] * f2[e];
        for (int o = 1; o < lpr; o <<= 1) ss += __shfl_xor(ss, o, 64);
        const float r = 1.0f / sqrtf(ss / (float)a.D + a.eps);
        const Vec<T, V> w1 = *reinterpret_cast<const Vec<T, V> *>(it[u].wgt);
        const Vec<T, V> w2 = *reinterpret_cast<const Vec<T, V> *>(it[u].wgt + half);
#pragma unroll
        for (int e = 0; e < V; ++e) {  // rounded to the element type, as the norm module returns it
          f1[e] = (float)(T)((f1[e] * r) * (1.0f + (float)w1.v[e]));
          f2[e] = (float)(T)((f2[e] * r) * (1.0f + (float)w2.v[e]));
        }
      }
      const int c = (first + u * kRopeThreads) % lpr;
      const float *sp = sin_s + it[u].t * half + c * V, *cp = cos_s + it[u].t * half + c * V;
      Vec<T, V> y1, y2;
#pragma unroll
      for (int e = 0; e < V; ++e) {
        const float sn = sp[e], cs = cp[e];
        y1.v[e] = (T)(f1[e] * cs - f2[e] * sn);
        y2.v[e] = (T)(f2[e] * cs + f1[e] * sn);
      }
      *reinterpret_cast<Vec<T, V> *>(it[u].dst) = y1;
      *reinterpret_cast<Vec<T, V> *>(it[u].dst + half) = y2;
    }
  }
}

int launch_rope(const RopeArgs &a, int dtype, hipStream_t st) {
  const int64_t ntok = (int64_t)a.B * a.L;
  const int rows = (a.q.ptr ? a.H : 0) + (a.k.ptr ? a.Hkv : 0);
  if (ntok == 0 || rows == 0) return BCATTN_OK;
  const int TB = rope_tokens(a.D, rows * (a.D / (dtype == BCATTN_F32 ? 8 : 16)));
  const dim3 grid((unsigned)((ntok + TB - 1) / TB)), block(kRopeThreads);
  const size_t lds = (size_t)TB * a.D * sizeof(float);
  if (dtype == BCATTN_F32)
    hipLaunchKernelGGL((rope_kernel<float, 4>), grid, block, lds, st, a, TB);
  else if (dtype == BCATTN_BF16)
    hipLaunchKernelGGL((rope_kernel<__bf16, 8>), grid, block, lds, st, a, TB);
  else
    hipLaunchKernelGGL((rope_kernel<_Float16, 8>), grid, block, lds, st, a, TB);
  return hipGetLastError() == hipSuccess ? BCATTN_OK : BCATTN_ERR_LAUNCH;
}

}  // namespace bcattn
