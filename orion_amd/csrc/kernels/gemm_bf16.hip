// High-priority co-location kernel: C[M,N] = A[M,K] * B[N,K]^T, bf16 inputs,
// fp32 accumulation on the gfx950 matrix cores, bf16 or fp32 output.
//
// MFMA-bound: 2*M*N*K flops against (M*K + N*K) * 2 + M*N * sizeof(out)
// algorithmic bytes.  Both operands are K-contiguous, so one 16-byte load gives
// a lane the eight consecutive K values v_mfma_f32_32x32x16_bf16 wants.
//
// Tiling (64-wide wavefronts, one workgroup resident per CU):
//   workgroup  256 x 256 x 32   4 wavefronts, 2 x 2
//   wavefront  128 x 128        4 x 4 MFMA tiles of 32 x 32, 256 accumulators
//   LDS        4 stages x (A 16 KiB + B 16 KiB) = 128 KiB of the CU's 160 KiB,
//              filled straight from global memory (global_load_lds_dwordx4),
//              two k-tiles ahead of the one being multiplied
// An LDS row is 64 bytes (four 16-byte chunks).  Two rows form a 128-byte
// super-row; chunk c of row r sits at position ((r & 1) * 4 + c) ^ ((r >> 1) & 7)
// of its super-row, so the 16-byte fragment reads of any eight consecutive lanes
// (eight consecutive rows, same logical chunk) cover all banks exactly once.
//
// Issue order inside a k-tile (one wave per SIMD, so nothing else hides a
// stall): every group of four MFMAs is preceded by the two fragment reads the
// NEXT k-step needs and followed by one global->LDS load of the tile two ahead;
// bursts of LDS reads or of loads in front of the MFMAs cost 8-25 % here.
//
// The reference system has no device code of its own; this kernel stands in for
// the compute-bound half of its toy co-location pair
// (benchmarking/benchmark_suite/toy_models/conv_trainer.py:20-27).

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

#include "kernels.h"

namespace {

constexpr int BM = 256;
constexpr int BN = 256;
constexpr int BK = 32;
constexpr int kThreads = 256;
constexpr int kStages = 4;
constexpr int kMatBytes = BM * BK * 2;      // 16 KiB per operand and stage
constexpr int kStageBytes = 2 * kMatBytes;  // A then B

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

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
// eight XCDs in turn, each with a private L2, and 256 workgroups (one per CU)
// run at a time.  When the tile grid divides into 16 x 16 super-tiles, every
// such round of 256 workgroups covers one super-tile (16 A panels + 16 B panels
// enter the chip per round instead of 32 + 8 per band), and inside it XCD x owns
// the 4 x 8 block at rows (x / 2) * 4, columns (x % 2) * 8, so the 32 CUs of an
// XCD share 4 A panels and 8 B panels in that XCD's L2.  Other grids fall back
// to bands of kGroupM tile rows per XCD.
constexpr int kXcds = 8;
constexpr int kGroupM = 4;
constexpr int kSuper = 16;

__device__ __forceinline__ void tile_of_block(int bid, int tiles_m, int tiles_n,
                                              int* tm, int* tn) {
  const int total = tiles_m * tiles_n;
  if (tiles_m % kSuper == 0 && tiles_n % kSuper == 0) {
    const int xcd = bid % kXcds;
    const int seq = bid / kXcds;       // order of this workgroup within its XCD
    const int super = seq / 32;        // 32 tiles of every super-tile per XCD
    const int local = seq % 32;
    const int supers_n = tiles_n / kSuper;
    *tm = (super / supers_n) * kSuper + (xcd / 2) * 4 + local % 4;
    *tn = (super % supers_n) * kSuper + (xcd % 2) * 8 + local / 4;
    return;
  }
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
  __shared__ __attribute__((aligned(16))) unsigned char lds[kStages * kStageBytes];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform
  const int wm = wave >> 1;
  const int wn = wave & 1;
  const int lrow = lane & 31;
  const int lhalf = lane >> 5;

  int tm, tn;
  tile_of_block(blockIdx.x, M / BM, N / BN, &tm, &tn);
  const size_t row0_a = (size_t)tm * BM;
  const size_t row0_b = (size_t)tn * BN;

  // Global -> LDS without a stop in registers: global_load_lds_dwordx4 writes
  // the 16 bytes a lane loads to LDS at (wave-uniform base) + lane * 16, so one
  // instruction of a wave fills eight super-rows (sixteen rows).  Lane l owns
  // super-row l / 8, PHYSICAL position l % 8 and fetches the (row, chunk) the
  // swizzle stores there: v = (l % 8) ^ (l / 8), row = 2 * (l / 8) + v / 4,
  // chunk = v % 4.  Wave w issues row groups w, w + 4, w + 8, w + 12 of A and B.
  const int v = (lane & 7) ^ (lane >> 3);
  const int l_row = wave * 16 + (lane >> 3) * 2 + (v >> 2);
  const int l_chunk = v & 3;
  const uint16_t* gA = A + (row0_a + l_row) * (size_t)K + l_chunk * 8;
  const uint16_t* gB = B + (row0_b + l_row) * (size_t)K + l_chunk * 8;
  const size_t g_step = (size_t)64 * K;  // 64 rows between a wave's row groups

  // idx 0..3: row groups of A, 4..7: of B
  auto load_one = [&](int kt, int stage, int idx) {
    const int i = idx & 3;
    const uint16_t* p = (idx < 4 ? gA : gB) + (size_t)kt * BK + i * g_step;
    unsigned char* d = lds + stage * kStageBytes + (idx < 4 ? 0 : kMatBytes) +
                       (i * 4 + wave) * 1024;
    __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)p,
                                     (__attribute__((address_space(3))) void*)d, 16, 0, 0);
  };

  f32x16 acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

  // Fragment reads.  Fragment i of a wave covers rows base + i*32 + lrow; base
  // and i*32 are multiples of 16, so the swizzle terms depend on lrow only.
  const int fr_sw = (lrow >> 1) & 7;
  const int fr_sub4 = (lrow & 1) * 4;
  const int fr_a = ((wm * 128 + lrow) >> 1) * 128;
  const int fr_b = ((wn * 128 + lrow) >> 1) * 128;
  // Two fragment register sets: the MFMAs of one k-step run out of one set
  // while the reads of the next k-step fill the other.
  bf16x8 fa[2][4], fb[2][4];
  auto read_one = [&](int set, int stage, int kk, int i) {
    const unsigned char* sa = lds + stage * kStageBytes + fr_a;
    const unsigned char* sb = lds + stage * kStageBytes + kMatBytes + fr_b;
    const int off = ((fr_sub4 + kk * 2 + lhalf) ^ fr_sw) << 4;
    fa[set][i] = *reinterpret_cast<const bf16x8*>(sa + i * 16 * 128 + off);
    fb[set][i] = *reinterpret_cast<const bf16x8*>(sb + i * 16 * 128 + off);
  };

  const int KT = K / BK;
#pragma unroll
  for (int idx = 0; idx < 8; ++idx) load_one(0, 0, idx);
  if (KT > 1) {
#pragma unroll
    for (int idx = 0; idx < 8; ++idx) load_one(1, 1, idx);
  }
  __builtin_amdgcn_s_waitcnt(0x0070);  // vmcnt(0) lgkmcnt(0)
  __builtin_amdgcn_s_barrier();
#pragma unroll
  for (int i = 0; i < 4; ++i) read_one(0, 0, 0, i);

  // One k-tile.  Invariant on entry: LDS stage kt % 4 holds tile kt, fragment
  // set 0 holds its first k-step, every load of tile kt + 1 has been issued.
  // The barrier sits between the two k-steps: the second step's MFMAs cover it
  // and the first fragment reads of tile kt + 1.  Tile kt + 2 is loaded into the
  // stage that held tile kt - 2, whose last read lies before the previous
  // iteration's barrier.
  auto k_tile = [&](int kt, auto with_loads) {
    constexpr bool kLoads = decltype(with_loads)::value;
    const int cur = kt & 3, nxt = (kt + 1) & 3, ld = (kt + 2) & 3;
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      read_one(1, cur, 1, i);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int j = 0; j < 4; ++j)
        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[0][i], fb[0][j], acc[i][j], 0, 0, 0);
      if (kLoads) load_one(kt + 2, ld, i);
      __builtin_amdgcn_sched_barrier(0);
    }
    if (kt + 1 < KT) {
      // lgkmcnt(0): this wave's reads of stage cur have returned (the stage is
      // overwritten two iterations on); vmcnt: all but the loads just issued,
      // i.e. tile kt + 1 has landed.
      if (kLoads) __builtin_amdgcn_s_waitcnt(0x0074);  // vmcnt(4) lgkmcnt(0)
      else __builtin_amdgcn_s_waitcnt(0x0070);         // vmcnt(0) lgkmcnt(0)
      __builtin_amdgcn_s_barrier();
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      if (kt + 1 < KT) read_one(0, nxt, 0, i);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int j = 0; j < 4; ++j)
        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[1][i], fb[1][j], acc[i][j], 0, 0, 0);
      if (kLoads) load_one(kt + 2, ld, 4 + i);
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  int kt = 0;
  for (; kt + 2 < KT; ++kt) k_tile(kt, std::true_type{});
  for (; kt < KT; ++kt) k_tile(kt, std::false_type{});

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
