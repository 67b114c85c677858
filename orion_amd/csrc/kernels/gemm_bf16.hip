// High-priority co-location kernel: C[M,N] = A[M,K] * B[N,K]^T, bf16 inputs,
// fp32 accumulation on the gfx950 matrix cores, bf16 or fp32 output.
//
// MFMA-bound: 2*M*N*K flops against (M*K + N*K) * 2 + M*N * sizeof(out)
// algorithmic bytes.  Both operands are K-contiguous, so one 16-byte load gives
// a lane the eight consecutive K values v_mfma_f32_32x32x16_bf16 wants.
//
// Tiling (64-wide wavefronts, one workgroup resident per CU):
//   workgroup  256 x 256 x 64   4 wavefronts, 2 x 2
//   wavefront  128 x 128        4 x 4 MFMA tiles of 32 x 32, 256 accumulators
//   LDS        2 stages x (A 32 KiB + B 32 KiB) = 128 KiB of the CU's 160 KiB
// Rows of an LDS tile are 128 bytes (eight 16-byte chunks); chunk c of row r is
// stored at chunk position c ^ (r & 7), so the 16-byte fragment reads of any
// eight consecutive lanes (eight consecutive rows, same logical chunk) cover
// all banks exactly once.
//
// The reference system has no device code of its own; this kernel stands in for
// the compute-bound half of its toy co-location pair
// (benchmarking/benchmark_suite/toy_models/conv_trainer.py:20-27).

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "kernels.h"

namespace {

constexpr int BM = 256;
constexpr int BN = 256;
constexpr int BK = 64;
constexpr int kThreads = 256;
constexpr int kRowBytes = BK * 2;                 // 128
constexpr int kChunksPerRow = kRowBytes / 16;     // 8
constexpr int kTileBytes = BM * kRowBytes;        // 32 KiB (BM == BN)
constexpr int kLoadsPerThread = BM * kChunksPerRow / kThreads;  // 8

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ uint16_t f32_to_bf16_rne(float f) {
  uint32_t u = __builtin_bit_cast(uint32_t, f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40u);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}

__device__ __forceinline__ void store_out(float* p, float v) { *p = v; }
__device__ __forceinline__ void store_out(uint16_t* p, float v) {
  *p = f32_to_bf16_rne(v);
}

// Workgroup id -> output tile.  Hardware hands consecutive workgroup ids to the
// eight XCDs in turn, each with a private L2.  Ids are regrouped so that one
// XCD owns a contiguous run of tiles, and a run is walked in bands of kGroupM
// tile rows, so the CUs of an XCD that run together share A and B panels in
// that XCD's L2.
constexpr int kXcds = 8;
constexpr int kGroupM = 4;

__device__ __forceinline__ void tile_of_block(int bid, int tiles_m, int tiles_n,
                                              int* tm, int* tn) {
  const int total = tiles_m * tiles_n;
  int lid = bid;
  if (total % kXcds == 0) lid = (bid % kXcds) * (total / kXcds) + bid / kXcds;
  const int band = kGroupM * tiles_n;
  const int g = lid / band;
  const int first_m = g * kGroupM;
  const int rows = (tiles_m - first_m < kGroupM) ? (tiles_m - first_m) : kGroupM;
  const int in_band = lid - g * band;
  *tm = first_m + in_band % rows;
  *tn = in_band / rows;
}

template <typename OutT>
__global__ __launch_bounds__(kThreads, 1) void gemm_bf16_nt_kernel(
    const uint16_t* __restrict__ A, const uint16_t* __restrict__ B,
    OutT* __restrict__ C, int M, int N, int K) {
  __shared__ __attribute__((aligned(16))) unsigned char lds[4 * kTileBytes];
  unsigned char* lds_a = lds;                   // two stages of A
  unsigned char* lds_b = lds + 2 * kTileBytes;  // two stages of B

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm = wave >> 1;
  const int wn = wave & 1;
  const int lrow = lane & 31;
  const int lhalf = lane >> 5;

  int tm, tn;
  tile_of_block(blockIdx.x, M / BM, N / BN, &tm, &tn);
  const size_t row0_a = (size_t)tm * BM;
  const size_t row0_b = (size_t)tn * BN;

  // Global -> register staging: thread handles chunk id = i*256 + tid, i.e.
  // row = id / 8, chunk = id % 8: eight neighbouring lanes read one contiguous
  // 128-byte row segment.
  const int g_chunk = tid & 7;
  const int g_row = tid >> 3;  // + 32 * i
  const uint16_t* gA = A + (row0_a + g_row) * (size_t)K + g_chunk * 8;
  const uint16_t* gB = B + (row0_b + g_row) * (size_t)K + g_chunk * 8;
  const size_t g_step = (size_t)32 * K;  // 32 rows per i

  // (row & 7) is the same for every i because rows advance by 32.
  const int st_off = g_row * kRowBytes + ((g_chunk ^ (g_row & 7)) << 4);

  u32x4 ra[kLoadsPerThread], rb[kLoadsPerThread];

  auto load_global = [&](int kt) {
    const uint16_t* pa = gA + (size_t)kt * BK;
    const uint16_t* pb = gB + (size_t)kt * BK;
#pragma unroll
    for (int i = 0; i < kLoadsPerThread; ++i) {
      ra[i] = *reinterpret_cast<const u32x4*>(pa + i * g_step);
      rb[i] = *reinterpret_cast<const u32x4*>(pb + i * g_step);
    }
  };
  auto store_lds = [&](int stage) {
    unsigned char* sa = lds_a + stage * kTileBytes + st_off;
    unsigned char* sb = lds_b + stage * kTileBytes + st_off;
#pragma unroll
    for (int i = 0; i < kLoadsPerThread; ++i) {
      *reinterpret_cast<u32x4*>(sa + i * 32 * kRowBytes) = ra[i];
      *reinterpret_cast<u32x4*>(sb + i * 32 * kRowBytes) = rb[i];
    }
  };

  f32x16 acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

  // Fragment read offsets.  Row of fragment (mi) is wm*128 + mi*32 + lrow, so
  // (row & 7) == (lrow & 7) for every mi.
  const int frag_row_a = wm * 128 + lrow;
  const int frag_row_b = wn * 128 + lrow;
  const int sw = lrow & 7;

  const int KT = K / BK;
  load_global(0);
  store_lds(0);
  __syncthreads();

  for (int kt = 0; kt < KT; ++kt) {
    const int cur = kt & 1;
    if (kt + 1 < KT) load_global(kt + 1);

    const unsigned char* sa = lds_a + cur * kTileBytes + frag_row_a * kRowBytes;
    const unsigned char* sb = lds_b + cur * kTileBytes + frag_row_b * kRowBytes;
#pragma unroll
    for (int kk = 0; kk < BK / 16; ++kk) {
      const int coff = ((kk * 2 + lhalf) ^ sw) << 4;
      bf16x8 fa[4], fb[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        fa[i] = *reinterpret_cast<const bf16x8*>(sa + i * 32 * kRowBytes + coff);
        fb[i] = *reinterpret_cast<const bf16x8*>(sb + i * 32 * kRowBytes + coff);
      }
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[i], fb[j],
                                                              acc[i][j], 0, 0, 0);
    }

    if (kt + 1 < KT) store_lds(cur ^ 1);
    __syncthreads();
  }

  // Epilogue.  Accumulator register r of a 32x32 tile holds
  // row (r/4)*8 + lhalf*4 + r%4, column lrow.
  const size_t c_row0 = row0_a + wm * 128;
  const size_t c_col0 = row0_b + wn * 128 + lrow;
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const size_t row = c_row0 + i * 32 + (r >> 2) * 8 + lhalf * 4 + (r & 3);
        const size_t col = c_col0 + j * 32;
        store_out(C + row * (size_t)N + col, acc[i][j][r]);
      }
}

}  // namespace

extern "C" int orion_gemm_bf16_nt(const void* A, const void* B, void* C, int M,
                                  int N, int K, int out_is_f32, void* stream) {
  if (M == 0 || N == 0) return ORION_OK;
  if (A == nullptr || B == nullptr || C == nullptr) return ORION_ERR_ARG;
  if (M < 0 || N < 0 || K <= 0) return ORION_ERR_ARG;
  if (M % BM != 0 || N % BN != 0 || K % BK != 0) return ORION_ERR_SHAPE;
  if ((((uintptr_t)A | (uintptr_t)B | (uintptr_t)C) & 15u) != 0)
    return ORION_ERR_ALIGN;
  const long long tiles = (long long)(M / BM) * (N / BN);
  if (tiles > 0x7fffffffLL) return ORION_ERR_SHAPE;
  dim3 grid((unsigned)tiles), block(kThreads);
  if (out_is_f32) {
    hipLaunchKernelGGL(gemm_bf16_nt_kernel<float>, grid, block, 0,
                       (hipStream_t)stream, (const uint16_t*)A,
                       (const uint16_t*)B, (float*)C, M, N, K);
  } else {
    hipLaunchKernelGGL(gemm_bf16_nt_kernel<uint16_t>, grid, block, 0,
                       (hipStream_t)stream, (const uint16_t*)A,
                       (const uint16_t*)B, (uint16_t*)C, M, N, K);
  }
  return hipGetLastError() == hipSuccess ? ORION_OK : ORION_ERR_LAUNCH;
}
