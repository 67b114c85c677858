// High-priority co-location kernel: C[M,N] = A[M,K] * B[N,K]^T, bf16 inputs,
// fp32 accumulation on the gfx950 matrix cores, bf16 or fp32 output.
//
// MFMA-bound: 2*M*N*K flops against (M*K + N*K) * 2 + M*N * sizeof(out)
// algorithmic bytes.  Both operands are K-contiguous, so one 16-byte load gives
// a lane the eight consecutive K values v_mfma_f32_16x16x32_bf16 wants.
//
// Tiling (64-wide wavefronts, one workgroup resident per CU):
//   workgroup  256 x 256 x 64   4 wavefronts, 2 x 2
//   wavefront  128 x 128        8 x 8 tiles of v_mfma_f32_16x16x32_bf16, 256
//                               accumulators; a k-tile is two MFMA k-steps
//   LDS        2 stages x (A 32 KiB + B 32 KiB) = 128 KiB of the CU's 160 KiB,
//              filled straight from global memory (global_load_lds_dwordx4)
// An LDS row is one 128-byte cache line of an operand row (eight 16-byte
// chunks); chunk c of row r sits at position c ^ (r & 7), so the 16-byte
// fragment reads of any eight consecutive lanes (eight consecutive rows, same
// logical chunk) cover all banks exactly once.
//
// What shaped it, measured on MI355X at 8192^3 (the GPU sits at its 1400 W
// power limit throughout, so speed is energy per flop as much as overlap):
// v_mfma_f32_16x16x32_bf16 sustains 15 % more than 32x32x16 on random data;
// loading whole 128-byte lines per row (k-tile 64) instead of half lines took
// the global->LDS stream alone from 0.64 to 0.44 ms; with one wave per SIMD the
// matrix core idles whenever the wave issues anything else for longer than one
// MFMA runs, so every other instruction sits alone between two MFMAs.
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
constexpr int BK = 64;
constexpr int kThreads = 256;
constexpr int kStages = 2;
constexpr int kMatBytes = BM * BK * 2;      // 32 KiB per operand and stage
constexpr int kStageBytes = 2 * kMatBytes;  // A then B

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

// c += a * b on the matrix core; c lives in accumulator registers and is
// updated in place (as a builtin call the register allocator shuffles the 256
// accumulators between register files in every iteration).
__device__ __forceinline__ void mfma_16x16x32(f32x4& c, const bf16x8& a, const bf16x8& b) {
  asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
}

typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

// Four consecutive elements of a row of C from one accumulator tile.
__device__ __forceinline__ void store_quad(float* p, const f32x4& v) {
  *reinterpret_cast<f32x4*>(p) = v;
}
// bf16: round to nearest even (v_cvt_pk_bf16_f32 on gfx950), two per register.
__device__ __forceinline__ void store_quad(uint16_t* p, const f32x4& v) {
  const f32x2 lo = {v[0], v[1]}, hi = {v[2], v[3]};
  u32x2 packed;
  packed[0] = __builtin_bit_cast(uint32_t, __builtin_convertvector(lo, bf16x2));
  packed[1] = __builtin_bit_cast(uint32_t, __builtin_convertvector(hi, bf16x2));
  *reinterpret_cast<u32x2*>(p) = packed;
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
    // super-tiles in boustrophedon order: consecutive rounds share their A or
    // their B panels, which the memory-side cache still holds
    const int sr = super / supers_n;
    const int sc = (sr & 1) ? supers_n - 1 - super % supers_n : super % supers_n;
    *tm = sr * kSuper + (xcd / 2) * 4 + local % 4;
    *tn = sc * kSuper + (xcd % 2) * 8 + local / 4;
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
  const int l16 = lane & 15;  // row (A, B) or column (C) within a 16x16 tile
  const int lq = lane >> 4;   // 16-byte k chunk of a fragment; row group of C

  int tm, tn;
  tile_of_block(blockIdx.x, M / BM, N / BN, &tm, &tn);
  const size_t row0_a = (size_t)tm * BM;
  const size_t row0_b = (size_t)tn * BN;

  // Global -> LDS without a stop in registers: global_load_lds_dwordx4 writes
  // the 16 bytes a lane loads to LDS at (wave-uniform base) + lane * 16, so one
  // instruction of a wave fills eight 128-byte rows, each a whole cache line of
  // the operand.  Lane l owns row l / 8, PHYSICAL chunk l % 8 and fetches the
  // logical chunk the swizzle stores there, (l % 8) ^ (l / 8).  Wave w issues row
  // blocks w, w + 4, ..., w + 28 of A and of B.
  const int l_chunk = (lane & 7) ^ (lane >> 3);
  const int l_row = wave * 8 + (lane >> 3);
  const uint16_t* gA = A + (row0_a + l_row) * (size_t)K + l_chunk * 8;
  const uint16_t* gB = B + (row0_b + l_row) * (size_t)K + l_chunk * 8;
  const size_t g_step = (size_t)32 * K;  // 32 rows between a wave's row blocks

  // idx 0..7: row blocks of A, 8..15: of B
  auto load_one = [&](int kt, int stage, int idx) {
    const int i = idx & 7;
    const uint16_t* p = (idx < 8 ? gA : gB) + (size_t)kt * BK + i * g_step;
    unsigned char* d = lds + stage * kStageBytes + (idx < 8 ? 0 : kMatBytes) +
                       (i * 4 + wave) * 1024;
    __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)p,
                                     (__attribute__((address_space(3))) void*)d, 16, 0, 0);
  };

  f32x4 acc[8][8];
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int j = 0; j < 8; ++j)
#pragma unroll
      for (int r = 0; r < 4; ++r) acc[i][j][r] = 0.0f;

  // Fragment reads.  Fragment i of a wave covers rows base + i*16 + l16; of each
  // 128-byte row, k-step ks uses logical chunks ks*4 .. ks*4+3 and lane group lq
  // takes chunk ks*4 + lq.  base and i*16 are multiples of 8, so the swizzle term
  // is l16 % 8.
  const int fr_a = (wm * 128 + l16) * 128;
  const int fr_b = kMatBytes + (wn * 128 + l16) * 128;
  const int fr_k0 = (lq ^ (l16 & 7)) << 4;
  const int fr_k1 = ((4 + lq) ^ (l16 & 7)) << 4;
  // Two fragment register sets, one per k-step of a tile.
  bf16x8 fa[2][8], fb[2][8];
  auto read_one = [&](auto ks_c, int stage, int r) {
    constexpr int KS = decltype(ks_c)::value;
    const unsigned char* st = lds + stage * kStageBytes + (KS ? fr_k1 : fr_k0);
    if (r < 8) fb[KS][r] = *reinterpret_cast<const bf16x8*>(st + fr_b + r * 2048);
    else fa[KS][r - 8] = *reinterpret_cast<const bf16x8*>(st + fr_a + (r - 8) * 2048);
  };
  using KS0 = std::integral_constant<int, 0>;
  using KS1 = std::integral_constant<int, 1>;

  const int KT = K / BK;
#pragma unroll
  for (int idx = 0; idx < 16; ++idx) load_one(0, 0, idx);
  if (KT > 1) {
#pragma unroll
    for (int idx = 0; idx < 16; ++idx) load_one(1, 1, idx);
    __builtin_amdgcn_s_waitcnt(0x4070);  // vmcnt(16): tile 0 has landed
  } else {
    __builtin_amdgcn_s_waitcnt(0x0070);  // vmcnt(0)
  }
  __builtin_amdgcn_s_barrier();
#pragma unroll
  for (int r = 0; r < 16; ++r) read_one(KS0{}, 0, r);

  // One k-tile = two MFMA k-steps of 64 MFMAs.  With one wave per SIMD the
  // matrix core idles whenever the wave issues anything else for longer than one
  // MFMA runs (16 cycles), so every other instruction sits alone between two
  // MFMAs: a fragment read after every third MFMA (all sixteen are out by the
  // 47th, the last sixteen MFMAs cover their latency), a global->LDS load after
  // every fourth in the second k-step.
  //
  // On entry set 0 holds the first k-step of tile kt and every load of tile
  // kt + 1 has been issued.  First k-step: fragment reads of the second.  The
  // wait + barrier after it mean that every wave has all of tile kt in
  // registers and that tile kt + 1 has landed.  Second k-step: first fragment
  // reads of tile kt + 1, loads of tile kt + 2 into the stage tile kt has left.
  auto read_slot = [&](auto ks_c, int stage, int m) {
    // B fragments first: every MFMA row of the next k-step needs all of them
    if (m % 3 == 1) read_one(ks_c, stage, m / 3);
  };
  auto k_tile = [&](int kt, auto has_next, auto has_loads) {
    constexpr bool kNext = decltype(has_next)::value;
    constexpr bool kLoads = decltype(has_loads)::value;
    const int cur = kt & 1, nxt = cur ^ 1;
    __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0): set 0 is complete
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int m = 0; m < 64; ++m) {
      mfma_16x16x32(acc[m >> 3][m & 7], fb[0][m & 7], fa[0][m >> 3]);
      read_slot(KS1{}, cur, m);
      __builtin_amdgcn_sched_barrier(0);
    }
    __builtin_amdgcn_s_waitcnt(0x0070);  // vmcnt(0) lgkmcnt(0)
    if (kNext) __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int m = 0; m < 64; ++m) {
      mfma_16x16x32(acc[m >> 3][m & 7], fb[1][m & 7], fa[1][m >> 3]);
      if (kNext) read_slot(KS0{}, nxt, m);
      if (kLoads && (m & 3) == 2) load_one(kt + 2, cur, m >> 2);
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  int kt = 0;
  for (; kt + 2 < KT; ++kt) k_tile(kt, std::true_type{}, std::true_type{});
  if (kt + 1 < KT) { k_tile(kt, std::true_type{}, std::false_type{}); ++kt; }
  k_tile(kt, std::false_type{}, std::false_type{});

  // The MFMAs above are opaque to the compiler's hazard handling: give the last
  // ones time to write their accumulators before anything reads them.
  asm volatile("s_nop 15\n\ts_nop 15\n\ts_nop 15" ::: "memory");

  // Epilogue.  The MFMAs ran with the B fragment as first operand, so a lane's
  // four accumulators of tile (i, j) are four CONSECUTIVE columns of one row of
  // C: row i*16 + l16, columns j*16 + lq*4 .. +3.  They are converted, packed
  // and written as one 8- or 16-byte piece into the wave's own quarter of the
  // LDS (free now); whole rows are then read back and stored 16 bytes per lane,
  // so every store instruction covers full cache lines.  A row is cut into
  // 16-byte slots; slot s of row R sits at s ^ (R & 15), which keeps the sixteen
  // rows one write instruction touches apart.
  __builtin_amdgcn_s_waitcnt(0xc07f);
  __builtin_amdgcn_s_barrier();  // every wave has read its last fragments
  constexpr int kElt = (int)sizeof(OutT);
  constexpr int kRowB = 128 * kElt;          // bytes of one row of the block
  constexpr int kPassRows = 32768 / kRowB;   // rows that fit the wave's quarter
  constexpr int kPasses = 128 / kPassRows;   // 1 (bf16) or 2 (fp32)
  constexpr int kIPerPass = 8 / kPasses;
  constexpr int kSlots = kRowB / 16;         // 16-byte slots per row
  constexpr int kRowsPerStore = 64 / kSlots;
  unsigned char* ep = lds + wave * 32768;
  const int st_row = lane / kSlots;
  const int st_slot = lane % kSlots;
  OutT* c_block = C + (row0_a + wm * 128) * (size_t)N + row0_b + wn * 128;
#pragma unroll
  for (int pass = 0; pass < kPasses; ++pass) {
#pragma unroll
    for (int ii = 0; ii < kIPerPass; ++ii)
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const int byte = (j * 16 + lq * 4) * kElt;
        unsigned char* dst = ep + (ii * 16 + l16) * kRowB +
                             (((byte >> 4) ^ l16) << 4) + (byte & 15);
        store_quad(reinterpret_cast<OutT*>(dst), acc[pass * kIPerPass + ii][j]);
      }
#pragma unroll
    for (int it = 0; it < kPassRows / kRowsPerStore; ++it) {
      const int R = it * kRowsPerStore + st_row;
      const u32x4 v = *reinterpret_cast<const u32x4*>(ep + R * kRowB +
                                                      ((st_slot ^ (R & 15)) << 4));
      __builtin_nontemporal_store(
          v, reinterpret_cast<u32x4*>(c_block + (size_t)(pass * kPassRows + R) * N) + st_slot);
    }
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
