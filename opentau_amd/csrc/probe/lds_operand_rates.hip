// Two measurements behind the tile bodies of the attention kernels, on whatever GPU is present:
//  (1) the LDS read rate of a CU for the three read instructions the kernels use (ds_read_b128 for row
//      operands, ds_read_b64 and the transposing ds_read_b64_tr_b16), reads alone, eight waves per CU;
//  (2) the matrix rate of the pattern "one v_mfma_f32_32x32x16_bf16 per 16-byte-per-lane LDS operand read,
//      the read issued RING products ahead", with one wave per SIMD (the head_dim 256 kernels' occupancy),
//      alone and with a direct-to-LDS tile request (buffer_load ... lds, 1 KB per wave) every N products.
// Prints one JSON line.  A measurement aid: the library does not use it.
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef int i32x4 __attribute__((ext_vector_type(4)));

#define CHECK(x)                                              \
  do {                                                        \
    hipError_t e_ = (x);                                      \
    if (e_ != hipSuccess) {                                   \
      fprintf(stderr, "%s: %s\n", #x, hipGetErrorString(e_)); \
      exit(1);                                                \
    }                                                         \
  } while (0)

// (1) MODE 0: ds_read_b128, 1: ds_read_b64, 2: ds_read_b64_tr_b16.  Sixteen reads, then a wait for all of them.
template <int MODE>
__global__ __launch_bounds__(512) void lds_reads(float *out, int iters) {
  __shared__ __align__(16) char tile[65536];
  for (int i = threadIdx.x; i < 65536 / 4; i += 512) reinterpret_cast<float *>(tile)[i] = (float)i;
  __syncthreads();
  const int lane = threadIdx.x & 63;
  // consecutive lanes read consecutive 16 (8) bytes: no bank conflicts
  const unsigned base = (unsigned)(size_t)tile + lane * (MODE == 0 ? 16 : 8) + (threadIdx.x >> 6) * 2048;
  f32x4 sum = {0.f, 0.f, 0.f, 0.f};
  for (int it = 0; it < iters; ++it) {
    f32x4 r[16];
#pragma unroll
    for (int j = 0; j < 16; ++j) {
      if (MODE == 0) {
        asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(r[j]) : "v"(base), "n"(j * 1024));
      } else {
        f32x2 t;
        if (MODE == 1)
          asm volatile("ds_read_b64 %0, %1 offset:%2" : "=v"(t) : "v"(base), "n"(j * 512));
        else
          asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(t) : "v"(base), "n"(j * 512));
        r[j] = f32x4{t[0], t[1], 0.f, 0.f};
      }
    }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
    for (int j = 0; j < 16; ++j) sum += r[j];
  }
  out[blockIdx.x * 512 + threadIdx.x] = sum[0] + sum[1] + sum[2] + sum[3];
}

// (2) RING operand registers, each re-read right after the product that used it; DMA > 0: a tile request in
// front of every DMA-th product (1 KB per wave from a 64 KB source per workgroup into a part of the LDS that
// nothing reads), at most RING / DMA of them in flight.
template <int RING, int DMA>
__global__ __launch_bounds__(256) void product_per_read(float *out, int iters, const char *src) {
  __shared__ __align__(16) char tile[65536];
  for (int i = threadIdx.x; i < 65536 / 4; i += 256) reinterpret_cast<unsigned *>(tile)[i] = 0x3f803f80u;
  __syncthreads();
  bf16x8 b, r[RING];
  for (int e = 0; e < 8; ++e) b[e] = (__bf16)(e * 0.5f);
  for (int i = 0; i < RING; ++i)
    for (int e = 0; e < 8; ++e) r[i][e] = (__bf16)1.0f;
  f32x16 acc[2];
  for (int i = 0; i < 2; ++i)
    for (int x = 0; x < 16; ++x) acc[i][x] = 0.f;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const unsigned addr = (unsigned)(size_t)tile + lane * 16 + wave * 4096;
  i32x4 rsrc;
  {
    const unsigned long long a = (unsigned long long)(src + (size_t)blockIdx.x * 65536);
    rsrc[0] = __builtin_amdgcn_readfirstlane((int)(unsigned)a);
    rsrc[1] = __builtin_amdgcn_readfirstlane((int)((unsigned)(a >> 32) & 0xffffu));
    rsrc[2] = 65536;
    rsrc[3] = 0x00020000;
  }
  const unsigned dst = __builtin_amdgcn_readfirstlane((unsigned)(size_t)tile + 32768 + wave * 4096);
  const unsigned voff = lane * 16 + wave * 4096;
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int i = 0; i < RING; ++i) {
      if constexpr (DMA > 0) {
        if (i % DMA == 0)
          asm volatile("s_add_u32 m0, %0, %4\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
                       :
                       : "s"(dst), "v"(voff), "s"(rsrc), "s"(0), "n"((i % 4) * 1024)
                       : "m0", "scc");
        if (i == RING - 1) asm volatile("s_waitcnt vmcnt(%0)" : : "n"((RING + DMA - 1) / DMA));
      }
      asm volatile("s_waitcnt lgkmcnt(%4)\n\tv_mfma_f32_32x32x16_bf16 %0, %1, %2, %0\n\tds_read_b128 %1, %3 offset:%5"
                   : "+v"(acc[i % 2]), "+v"(r[i])
                   : "v"(b), "v"(addr), "n"(RING - 1), "n"((i % 4) * 1024));
    }
  }
  asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
  float s = 0.f;
  for (int i = 0; i < 2; ++i)
    for (int x = 0; x < 16; ++x) s += acc[i][x];
  out[blockIdx.x * 256 + threadIdx.x] = s;
}

static hipEvent_t e0, e1;
template <class Launch>
static float best_ms(Launch launch) {
  float best = 1e30f;
  for (int rep = 0; rep < 4; ++rep) {
    CHECK(hipEventRecord(e0));
    launch();
    CHECK(hipEventRecord(e1));
    CHECK(hipEventSynchronize(e1));
    float ms;
    CHECK(hipEventElapsedTime(&ms, e0, e1));
    if (ms < best) best = ms;
  }
  return best;
}

int main() {
  hipDeviceProp_t prop;
  CHECK(hipGetDeviceProperties(&prop, 0));
  const int cus = prop.multiProcessorCount;
  const double ghz = prop.clockRate * 1e-6;  // the highest shader clock; the rates per clock below are lower bounds
  float *out;
  char *src;
  CHECK(hipMalloc(&out, (size_t)cus * 512 * sizeof(float)));
  CHECK(hipMalloc(&src, (size_t)cus * 65536));
  CHECK(hipMemset(src, 0x3f, (size_t)cus * 65536));
  CHECK(hipEventCreate(&e0));
  CHECK(hipEventCreate(&e1));

  const int it1 = 20000;
  auto bytes_per_clk = [&](float ms, int bytes_per_read) {
    return (double)it1 * 16 * 8 * bytes_per_read / (ms * 1e-3 * ghz * 1e9);
  };
  const double b128 = bytes_per_clk(best_ms([&] { hipLaunchKernelGGL(lds_reads<0>, dim3(cus), dim3(512), 0, 0, out, it1); }), 1024);
  const double b64 = bytes_per_clk(best_ms([&] { hipLaunchKernelGGL(lds_reads<1>, dim3(cus), dim3(512), 0, 0, out, it1); }), 512);
  const double tr64 = bytes_per_clk(best_ms([&] { hipLaunchKernelGGL(lds_reads<2>, dim3(cus), dim3(512), 0, 0, out, it1); }), 512);

  const int products = 400000;  // per wave
  auto tflops = [&](float ms) { return (double)cus * 4 * products * 32768.0 / (ms * 1e-3) / 1e12; };
  const double ring3 = tflops(best_ms([&] { hipLaunchKernelGGL((product_per_read<3, 0>), dim3(cus), dim3(256), 0, 0, out, products / 3, src); }));
  const double ring6 = tflops(best_ms([&] { hipLaunchKernelGGL((product_per_read<6, 0>), dim3(cus), dim3(256), 0, 0, out, products / 6, src); }));
  const double dma3 = tflops(best_ms([&] { hipLaunchKernelGGL((product_per_read<6, 3>), dim3(cus), dim3(256), 0, 0, out, products / 6, src); }));
  const double dma2 = tflops(best_ms([&] { hipLaunchKernelGGL((product_per_read<6, 2>), dim3(cus), dim3(256), 0, 0, out, products / 6, src); }));
  const double dma1 = tflops(best_ms([&] { hipLaunchKernelGGL((product_per_read<6, 1>), dim3(cus), dim3(256), 0, 0, out, products / 6, src); }));

  printf("{\"cus\": %d, \"clock_ghz_assumed\": %.2f, "
         "\"lds_read_bytes_per_clk_per_cu\": {\"ds_read_b128\": %.0f, \"ds_read_b64\": %.0f, \"ds_read_b64_tr_b16\": %.0f}, "
         "\"one_wave_per_simd_tflops\": {\"ring_3\": %.0f, \"ring_6\": %.0f, \"ring_6_request_every_3rd_product\": %.0f, "
         "\"ring_6_request_every_2nd_product\": %.0f, \"ring_6_request_every_product\": %.0f}}\n",
         cus, ghz, b128, b64, tr64, ring3, ring6, dma3, dma2, dma1);
  CHECK(hipFree(out));
  CHECK(hipFree(src));
  return 0;
}
