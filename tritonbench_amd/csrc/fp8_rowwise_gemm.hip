// Row-wise scaled FP8 (e4m3fn) GEMM for MI355X (gfx950, CDNA4): kernels and C ABI.
//
//   C[M,N] bf16 = bf16( (sum_k A[m,k] * B[n,k]) * a_scale[m] * b_scale[n] + bias[n] )
//
// A is [M,K] and B is [N,K], both K-contiguous, one byte per element. The contraction runs
// on the gfx950 f8f6f4 MFMA instructions (full FP8 rate) with fp32 accumulation; scales and
// bias are applied in fp32 to the accumulator and the result is rounded to bf16 once.
//
// Kernels:
//   gemm_tiled_kernel        persistent workgroups walk (split, tile) work items; BM x BN x 128
//                            steps staged global->LDS with direct-to-LDS loads into swizzled
//                            rings (2 or 3 stages of A, one more of B), 32x32x64 MFMA, epilogue
//                            turned through LDS into 16-byte row stores. Tiles of 256x256,
//                            128x128 (two ring depths), 256x128, 64x256, 128x256 and 192x256; grouped
//                            and block-scaled forms.
//   splitk_finalize_kernel   adds the fp32 partial sums of a split-K launch, applies scales/bias.
//   gemm_skinny_kernel       M <= 64: every workgroup owns 16 rows of B and all of K, its waves
//                            split K between them and reduce through LDS; B is streamed once.
//   gemm_skinny_persistent_kernel  M <= 16 (M <= 32 at K = 4096): one 16-wave workgroup per CU keeps
//                            its share of A in registers and walks 16-row tiles of B.
//   gemm_skinny_pair_kernel  M <= 16, N <= 8192, K <= 8192: one or two 16-row tiles of B per CU, A parked
//                            in LDS, a tile's rows requested in one burst.
//   gemm_narrow_kernel       M <= 64 (M <= 256 in row blocks), K in 512-byte steps, at most one tile of
//                            up to 64 columns per CU: a workgroup owns all of K (no split, no second
//                            launch); separate waves fetch A and B.
//   gemm_generic_kernel      any K, leading dimension and alignment: byte loads, f32 multiply-adds.
//   quantize_rows_*_kernel   row-wise e4m3fn quantiser (amax, scale, convert), one row per workgroup.
//   quantize_blocks_kernel   128 x 128 block-wise e4m3fn quantiser, one block per workgroup.
//   fused_rowwise_quant_kernel  RMSNorm or SiLU-mul of bf16 rows followed by the same quantiser, one pass.
//
// Operand roles inside the MFMA are swapped on purpose (rows of B feed the instruction's
// "A" port, rows of A its "B" port) so each lane ends up holding 4 consecutive columns n of
// one output row m (8 bytes of 16-bit results for the epilogue's LDS turn and for the skinny
// kernels' direct stores).

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdarg.h>
#include <stdio.h>
#include <string.h>
#include <atomic>
#include <type_traits>

#include "../../include/mi355x_fp8_rowwise.h"

// ------------------------------------------------------------------------------------
// Building in parts. This file compiles on its own (`hipcc -shared` on it gives the library), and
// it compiles faster as several translation units in parallel, which is what the package's build
// script does: with -DMI355X_TILED_PART=<k> a unit holds only the instantiations of tile
// configuration k of the plain tiled kernel (where nearly all of the compile time goes), with
// -DMI355X_SPLIT_MAIN it holds everything else and calls those through the functions below.
// What the units share lives in this namespace (hidden from the library's users): the parameter
// block, the error text, the table of kernels that need a raised LDS limit, the device set-up.
// ------------------------------------------------------------------------------------
#if defined(MI355X_TILED_PART) && defined(MI355X_SPLIT_MAIN)
#error "a translation unit is either a part or the main unit"
#endif
namespace mi355x_shared __attribute__((visibility("hidden"))) {
struct GemmParams {
  const uint8_t* a;
  const uint8_t* b;
  const float* a_scale;
  const float* b_scale;
  const uint16_t* bias;  // bf16 bits or nullptr
  uint16_t* c;           // bf16 bits
  int M, N, K;
  long lda, ldb, ldc;
  int tiles_m, tiles_n;
  int group_m;           // tile rows walked together so an XCD's resident tiles share A and B panels
  // split-K: every tile is cut into `splits` work items of `steps_per_split` 128-byte K steps
  // (the last one takes what is left); with splits > 1 the items write fp32 partial sums to
  // partial[split][M][N] and a second kernel adds them up and applies the epilogue
  int splits, steps_per_split;
  float* partial;
  // grouped form: `groups` consecutive row blocks of A and C, block g of m_sizes[g] rows
  // (device memory) multiplied with rows [g*N, (g+1)*N) of B and scaled by b_scale[g*N + n]
  const int32_t* m_sizes;
  int groups;
  int out_f16;  // C holds IEEE binary16 instead of bf16 (same size, same stores)
  // tiled kernel, plain form: reciprocals of the two run-time divisors of the tile walk (the number
  // of tiles, and the tiles of a full group of tile rows), prepared on the host: see fast_div()
  uint32_t div_tiles_mul, div_tiles_shift, div_group_mul, div_group_shift;
  // tiled kernel: where every workgroup leaves its start and end readings of the shader clock and of
  // the constant 100 MHz clock (4 values per workgroup), or nullptr
  unsigned long long* stamps;
};

extern thread_local char err[512];
struct LdsKernel {
  const void* kernel;
  size_t lds_bytes;
};
constexpr int kMaxLdsKernels = 256;
extern LdsKernel lds_kernels[kMaxLdsKernels];
extern int num_lds_kernels;
extern bool lds_table_overflow;
int ready_device(int* dev_out);
// tile configuration k of the plain tiled kernel: picks the instantiation for the plan in `p` and launches it
constexpr int kNumTiledParts = 7;
int tiled_config_0(const GemmParams& p, hipStream_t stream);
int tiled_config_1(const GemmParams& p, hipStream_t stream);
int tiled_config_2(const GemmParams& p, hipStream_t stream);
int tiled_config_3(const GemmParams& p, hipStream_t stream);
int tiled_config_4(const GemmParams& p, hipStream_t stream);
int tiled_config_5(const GemmParams& p, hipStream_t stream);
int tiled_config_6(const GemmParams& p, hipStream_t stream);
}  // namespace mi355x_shared

namespace {

typedef int   v4i  __attribute__((ext_vector_type(4)));
typedef int   v8i  __attribute__((ext_vector_type(8)));
typedef float v4f  __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef unsigned short us4 __attribute__((ext_vector_type(4)));
typedef unsigned int v2u __attribute__((ext_vector_type(2)));

constexpr int kNumXcd = 8;       // accelerator complex dies; workgroup ids round-robin over them
constexpr int kNumCu = 256;
constexpr int kChunk = 16;       // bytes moved per lane per load

using mi355x_shared::GemmParams;

// Where a tile sits: rows [m0, m_end) of A and C it may touch, first column, group.
struct TileLoc {
  int m0, m_end, n0, group;
};

// Cursor over the groups for the grouped form. Tiles are numbered group by group; inside a
// group column-major (consecutive tiles share a B panel). A walker only moves forward.
struct GroupWalk {
  int group, tile_begin, tile_end, row_begin, tiles_m;
};

__device__ __forceinline__ uint16_t f32_to_bf16_rne(float f) {
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u);  // quiet NaN
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}

__device__ __forceinline__ float bf16_to_f32(uint16_t h) {
  return __uint_as_float(((uint32_t)h) << 16);
}

// Two f32 -> two bf16 (round to nearest even, NaN kept) in one gfx950 instruction;
// `lo` lands in bits 0..15.
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
  uint32_t r;
  asm("v_cvt_pk_bf16_f32 %0, %1, %2" : "=v"(r) : "v"(lo), "v"(hi));
  return r;
}

// Two f32 -> two IEEE binary16 (round to nearest even; beyond 65504 rounds to infinity as the
// conversion instruction does); `lo` lands in bits 0..15.
__device__ __forceinline__ uint32_t pack_f16x2(float lo, float hi) {
  const _Float16 l = (_Float16)lo, h = (_Float16)hi;
  return (uint32_t)__builtin_bit_cast(uint16_t, l) | ((uint32_t)__builtin_bit_cast(uint16_t, h) << 16);
}

// Output element type is a launch parameter (uniform branch, outside the hot loop).
__device__ __forceinline__ uint32_t pack_out_x2(float lo, float hi, bool f16) {
  return f16 ? pack_f16x2(lo, hi) : pack_bf16x2(lo, hi);
}

// Kernel arguments live in memory and reach a wave through scalar loads that the compiler issues
// where it first needs each value: several dependent round trips of a few hundred nanoseconds each at
// the start of a kernel (the argument block is cold in the scalar cache at every launch). The decode
// kernels are a few microseconds long, so they ask for everything they will use in one batch, first
// thing (measured on the pair kernel at M=16, N=K=8192: 13.2 -> 12.6 us; whether the compiler's own
// placement is the fast or the slow one changes with unrelated edits).
__device__ __forceinline__ void fetch_arguments_now(const GemmParams& p) {
  asm volatile("" ::"s"(p.a), "s"(p.b), "s"(p.a_scale), "s"(p.b_scale), "s"(p.bias), "s"(p.c), "s"(p.M), "s"(p.N), "s"(p.K),
               "s"(p.lda), "s"(p.ldb), "s"(p.ldc), "s"(p.tiles_m), "s"(p.tiles_n), "s"(p.out_f16));
}
// the same for what only the tiled kernel and its second pass read
__device__ __forceinline__ void fetch_tiled_arguments_now(const GemmParams& p) {
  asm volatile("" ::"s"(p.splits), "s"(p.steps_per_split), "s"(p.partial), "s"(p.m_sizes), "s"(p.groups), "s"(p.div_tiles_mul),
               "s"(p.div_tiles_shift), "s"(p.div_group_mul), "s"(p.div_group_shift), "s"(p.stamps));
}

// ------------------------------------------------------------------------------------
// Tile scheduler: static, no atomics (safe under graph capture).
//
// Hardware hands consecutive workgroup ids to consecutive XCDs, each with a private L2.
// Workgroup b therefore belongs to XCD b % 8 and is that XCD's slot b / 8. The tile list is
// cut into 8 contiguous chunks, one per XCD, and walked in "grouped" order (group_m tile
// rows at a time, column-major inside a group) so the tiles an XCD has in flight at any
// moment form a compact rectangle sharing A row panels and B column panels in its L2.
// ------------------------------------------------------------------------------------
struct TileWalk {
  int chunk_begin, chunk_len, slot, slots;
};

__device__ __forceinline__ TileWalk make_walk(int total_tiles) {
  const int xcd = blockIdx.x % kNumXcd;
  const int q = total_tiles / kNumXcd, rem = total_tiles % kNumXcd;
  TileWalk w;
  w.chunk_begin = xcd * q + (xcd < rem ? xcd : rem);
  w.chunk_len = q + (xcd < rem ? 1 : 0);
  w.slot = blockIdx.x / kNumXcd;
  w.slots = gridDim.x / kNumXcd;
  return w;
}

// Division of a wave-uniform n < 2^31 by a run-time divisor d whose reciprocal the host prepared:
// mul = ceil(2^shift / d), shift = 31 + ceil(log2 d), and then floor(n / d) = (n * mul) >> shift
// exactly (mul * d lies within 2^(shift-31) of 2^shift). Three scalar instructions where the
// compiler's expansion of a division is a few dozen, on the path that moves a load cursor from one
// tile to the next in the middle of the K pipeline.
__device__ __forceinline__ int fast_div(int n, uint32_t mul, uint32_t shift) {
  return (int)(uint32_t)(((uint64_t)(uint32_t)n * mul) >> shift);
}
inline void make_fast_div(uint32_t d, uint32_t& mul, uint32_t& shift) {
  int l = 0;
  while ((1ull << l) < d) ++l;
  shift = 31u + (uint32_t)l;
  mul = (uint32_t)(((1ull << shift) + d - 1) / d);
}

constexpr int kGroupM = 4;  // tile rows walked together (a group); the last group may hold fewer

// tile number -> tile row and column in grouped order (kGroupM tile rows at a time, column-major inside a group)
__device__ __forceinline__ void tile_coords(int t, int tiles_m, int tiles_n, uint32_t group_mul, uint32_t group_shift,
                                            int& tm, int& tn) {
  const int per_group = kGroupM * tiles_n;
  const int g = fast_div(t, group_mul, group_shift);
  const int first_m = g * kGroupM;
  const int gsz = min(tiles_m - first_m, kGroupM);
  const int in_g = t - g * per_group;
  // in_g / gsz for gsz in 1..4
  tn = gsz == 4 ? in_g >> 2 : gsz == 3 ? fast_div(in_g, 0xAAAAAAABu, 33) : gsz == 2 ? in_g >> 1 : in_g;
  tm = first_m + in_g - tn * gsz;
}

// ------------------------------------------------------------------------------------
// LDS layout of the tiled kernel. A "stage" of an operand holds a 128-byte K slab of the
// tile's rows: 128 bytes per row = 8 chunks of 16 bytes, fetched from global memory as whole
// 128-byte lines. Chunk c of row r sits at chunk position c ^ ((r >> 1) & 7): the MFMA
// operand reads (consecutive lanes = consecutive rows, same logical chunk) then spread over
// all banks. With a load distance of 2 steps A has two stages,
// B three (2*32 KB + 3*32 KB = all 160 KB of a 256x256 tile's LDS); the 256x128 tile runs at a
// distance of 3 (3*32 KB + 4*16 KB). (Distances of 3 and 4 were measured on the 128x128 tile with one
// workgroup per CU and bought under 10 %: that tile is bound by what the L2->L1->LDS path delivers
// per CU, about 48 bytes per clock against the 64 its two workgroups ask for at the full MFMA
// rate, not by the latency of a load.)
// ------------------------------------------------------------------------------------
constexpr int kStepK = 128;
constexpr int kDefaultDist = 2;  // steps a load runs ahead of its use; A ring = DIST stages, B ring = DIST + 1

__device__ __forceinline__ int swz128(int row) { return (row >> 1) & 7; }

// One wave-wide load of 16 bytes per lane from a buffer straight into LDS: lane i's bytes land at
// lds_wave_base + 16*i. The address is the descriptor's base + lane_off + wave_off, range-checked
// against the descriptor's extent (bytes past it arrive as zeros). STREAM marks the lines as used
// once (the instruction's `nt` bit): they leave the L2 early instead of pushing out lines other
// workgroups will ask for again.
template <bool STREAM>
__device__ __forceinline__ void load_chunk_to_lds(__amdgpu_buffer_rsrc_t rsrc, uint8_t* lds_wave_base,
                                                  uint32_t lane_off, uint32_t wave_off) {
#if defined(__HIP_DEVICE_COMPILE__)  // (the host pass does not know the builtin)
  __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (__attribute__((address_space(3))) void*)lds_wave_base, 16,
                                           (int)lane_off, (int)wave_off, 0, STREAM ? 2 : 0);
#endif
}

// Range-checked register loads through a buffer descriptor: 4 floats / 4 bf16 / one bf16 per lane;
// elements past the descriptor's extent read as zero bits.
__device__ __forceinline__ v4f load_f32x4_checked(__amdgpu_buffer_rsrc_t rsrc, uint32_t lane_off) {
#if defined(__HIP_DEVICE_COMPILE__)
  return __builtin_bit_cast(v4f, __builtin_amdgcn_raw_buffer_load_b128(rsrc, (int)lane_off, 0, 0));
#else
  return (v4f){0.f, 0.f, 0.f, 0.f};
#endif
}
__device__ __forceinline__ us4 load_u16x4_checked(__amdgpu_buffer_rsrc_t rsrc, uint32_t lane_off) {
#if defined(__HIP_DEVICE_COMPILE__)
  return __builtin_bit_cast(us4, __builtin_amdgcn_raw_buffer_load_b64(rsrc, (int)lane_off, 0, 0));
#else
  return (us4){0, 0, 0, 0};
#endif
}
__device__ __forceinline__ uint16_t load_u16_checked(__amdgpu_buffer_rsrc_t rsrc, uint32_t lane_off) {
#if defined(__HIP_DEVICE_COMPILE__)
  return __builtin_amdgcn_raw_buffer_load_b16(rsrc, (int)lane_off, 0, 0);
#else
  return 0;
#endif
}

// Range-checked store of 4 floats per lane through a buffer descriptor (dropped past the extent).
__device__ __forceinline__ void store_f32x4_checked(v4f data, __amdgpu_buffer_rsrc_t rsrc, uint32_t lane_off, uint32_t wave_off) {
#if defined(__HIP_DEVICE_COMPILE__)
  __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(v4i, data), rsrc, (int)lane_off, (int)wave_off, 0);
#endif
}

// One wave-wide streaming store of 16 bytes per lane through a buffer descriptor (address = base +
// lane_off + wave_off): the output is written once and read by a later kernel at best.
__device__ __forceinline__ void store_chunk_streaming(v4i data, __amdgpu_buffer_rsrc_t rsrc, uint32_t lane_off,
                                                      uint32_t wave_off) {
#if defined(__HIP_DEVICE_COMPILE__)
  __builtin_amdgcn_raw_buffer_store_b128(data, rsrc, (int)lane_off, (int)wave_off, 2);
#endif
}

// Waits until at most VM of this wave's global loads and none of its LDS operations are
// outstanding, then joins the workgroup barrier. Written with the s_waitcnt builtin (not
// inline asm) so the compiler's own wait-count bookkeeping knows the LDS queue is empty
// afterwards and does not add full waits in front of the MFMAs that follow.
template <int VM>
__device__ __forceinline__ void wait_loads_and_barrier() {
  // gfx9 encoding: vmcnt[3:0] | expcnt[6:4] | lgkmcnt[11:8] | vmcnt[5:4] at [15:14]
  constexpr int imm = (VM & 15) | ((VM >> 4) << 14) | (7 << 4) | (0 << 8);
  __builtin_amdgcn_s_waitcnt(imm);
  __builtin_amdgcn_s_barrier();
}

// Cursor over the (tile, K step) sequence a workgroup walks; one for the A loads, one for
// the B loads (which run a step further ahead).
struct StepCursor {
  int item, kt, kt_begin, kt_end, left, issued;  // kt walks [kt_begin, kt_end) cyclically, `left` steps to go
};

// The kernel is one software pipeline over "steps" (a 128-byte K slab of one tile) that runs
// through all tiles a workgroup owns without draining at tile boundaries. For step g, with
// loads running DIST (= 2) steps ahead:
//
//   [A] MFMAs of (g, first K half), interleaved with the LDS reads of (g, second half) and
//       the loads of B(g+DIST) (its stage was released at the previous barrier)
//       wait for own loads of A(g+1) and B(g+1); workgroup barrier
//   [B] MFMAs of (g, second half), interleaved with the LDS reads of (g+1, first half) and
//       the loads of A(g+DIST) into the A stage step g just released
//   after a tile's last step: epilogue (loads of the next tile are already in flight)
//
// Two register sets of operand fragments alternate between the halves; one barrier per step.
//
// EPI selects what happens to a finished accumulator tile: scaled bf16 store (kEpiPlain),
// the same with the bias added (kEpiBias), or a raw fp32 partial-sum store for split-K
// (kEpiPartial). Tiles small enough for two workgroups per CU are compiled for two waves per
// SIMD (256 registers each).
constexpr int kEpiPlain = 0, kEpiBias = 1, kEpiPartial = 2;

constexpr size_t tiled_lds_bytes(int BM, int BN, int dist = kDefaultDist) {
  return (size_t)(dist * BM + (dist + 1) * BN) * kStepK;
}
constexpr int tiled_wgs_per_cu(int BM, int BN, bool blockscale = false, int dist = kDefaultDist) {
  (void)blockscale;
  return tiled_lds_bytes(BM, BN, dist) <= 80 * 1024 ? 2 : 1;
}

//
// GROUPED walks the tiles of a stack of row blocks whose sizes are read from device memory.
//
// BLOCKSCALE turns the kernel into the 128x128x128 block-scaled GEMM: a_scale is then
// [ceil(M/128)][ceil(K/128)], b_scale [ceil(N/128)][ceil(K/128)], and every K step's product
// is multiplied by a_scale[mb][kb] * b_scale[nb][kb] before it is added up. With wave tiles
// inside one scale block and 128-byte steps that factor is one number per wave and step:
// the accumulators are kept in units of the current step's factor (multiplied by the ratio of
// consecutive factors in front of each step's MFMAs) and by the last factor in the epilogue.
//
// STREAM_B: the rows of B are fetched with the streaming cache policy. For launches with one or
// two tile rows, where a panel of B is read by one or two workgroups and never again
// (measured: M=128, N=K=8192 27.6 -> 24.2 us, M=64 22.5 -> 19.6 us; with more tile rows the
// panels are shared through the L2 and the same policy costs 5-8 %).
template <int BM, int BN, int WAVES_M, int WAVES_N, bool KTAIL, int EPI, bool GROUPED = false, bool BLOCKSCALE = false,
          int DIST = kDefaultDist, bool STREAM_B = false>
__global__ __launch_bounds__(WAVES_M* WAVES_N * 64)
__attribute__((amdgpu_waves_per_eu(tiled_wgs_per_cu(BM, BN, BLOCKSCALE, DIST) * WAVES_M * WAVES_N / 4,
                                   tiled_wgs_per_cu(BM, BN, BLOCKSCALE, DIST) * WAVES_M * WAVES_N / 4)))
void gemm_tiled_kernel(GemmParams p) {
  constexpr int kStagesA = DIST, kStagesB = DIST + 1;
  static_assert(DIST >= 2 && tiled_lds_bytes(BM, BN, DIST) <= 160 * 1024, "the stage rings must fit the LDS");
  static_assert(!GROUPED || EPI == kEpiPlain, "the grouped form has neither bias nor split-K");
  static_assert(!STREAM_B || (!BLOCKSCALE && !GROUPED), "the rotated K order is for the plain form only");
  static_assert(!BLOCKSCALE || (128 % (BM / WAVES_M) == 0 && 128 % (BN / WAVES_N) == 0 && EPI == kEpiPlain && !GROUPED),
                "a wave's tile must lie inside one 128x128 scale block: one factor per wave and step");
  constexpr bool HAS_BIAS = EPI == kEpiBias;
  constexpr int NW = WAVES_M * WAVES_N;
  constexpr int WTM = BM / WAVES_M;    // wave tile rows (m)
  constexpr int WTN = BN / WAVES_N;    // wave tile cols (n)
  constexpr int MT = WTM / 32, NT = WTN / 32;
  constexpr int STAGE_A = BM * kStepK, STAGE_B = BN * kStepK;
  constexpr int LDS_B0 = kStagesA * STAGE_A;  // B stages follow the A stages
  constexpr int A_GROUPS = BM / 8 / NW;       // 8-row groups (1 KB of LDS) each wave fetches per step
  constexpr int B_GROUPS = BN / 8 / NW;
  static_assert(BM % (8 * NW) == 0 && BN % (8 * NW) == 0, "tile rows must split over waves");
  static_assert(WTM % 32 == 0 && WTN % 32 == 0, "wave tile must be a multiple of 32x32");
  static_assert(DIST * (A_GROUPS + B_GROUPS) < 64, "outstanding-load count must fit the vmcnt field");

  fetch_arguments_now(p);
  fetch_tiled_arguments_now(p);
  extern __shared__ __attribute__((aligned(1024))) uint8_t lds[];

  // (diagnostic launches only: the shader clock and the constant 100 MHz clock at this workgroup's start)
  unsigned long long stamp_cycles = 0, stamp_ticks = 0;
  if (p.stamps) {
    stamp_cycles = __builtin_readcyclecounter();
    stamp_ticks = __builtin_amdgcn_s_memrealtime();
  }

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int wm = wave / WAVES_N, wn = wave % WAVES_N;
  const int l32 = lane & 31, half = lane >> 5;

  // ---- per-lane constants of the global->LDS copy: a wave-wide load fills 8 rows
  const int ld_row = lane >> 3;
  const int ld_pc = lane & 7;  // physical chunk this lane's 16 bytes land in
  // 8*group + ld_row: the swizzle key depends on ld_row and the parity of the group only
  auto ld_chunk_off = [&](int group) { return (ld_pc ^ swz128(group * 8 + ld_row)) * kChunk; };

  // ---- per-lane constants of the LDS->register operand reads. For K half s (64 bytes) and
  // j in {0,1}, lane (l32, half) takes logical chunk 4*half + 2*s + j of its row. Any
  // assignment is valid as long as A and B use the same one; this one keeps the two halves
  // of the wave in different 64-byte halves of a row.
  int rd_off[2][2];
#pragma unroll
  for (int s = 0; s < 2; ++s)
#pragma unroll
    for (int j = 0; j < 2; ++j)
      rd_off[s][j] = l32 * kStepK + (((4 * half + 2 * s + j) ^ swz128(l32)) * kChunk);
  const int a_rd_base = (wm * WTM) * kStepK;
  const int b_rd_base = LDS_B0 + (wn * WTN) * kStepK;

  // Work items are (split, tile) pairs, split-major: consecutive items are neighbouring
  // tiles of the same K range, so an XCD's chunk of the list still shares operand panels.
  int total_tiles = p.tiles_m * p.tiles_n;
  // rows of group g, given the rows before it: never negative, never past row M
  auto group_rows = [&](int g, int row_begin) { return min(max(p.m_sizes[g], 0), p.M - row_begin); };
  if (GROUPED) {
    total_tiles = 0;
    for (int g = 0, rows = 0; g < p.groups; ++g) {
      const int mg = group_rows(g, rows);
      total_tiles += ((mg + BM - 1) / BM) * p.tiles_n;
      rows += mg;
    }
  }
  const TileWalk walk = make_walk(total_tiles * p.splits);
  if (walk.slot >= walk.chunk_len) return;  // uniform over the workgroup
  const int k_full = p.K / kStepK;             // whole 128-byte steps
  const int k_tail = p.K - k_full * kStepK;    // 0 or a multiple of 16
  const int k_steps = k_full + (k_tail ? 1 : 0);
  // (the grouped form counts its tiles on the device and divides the ordinary way; an unsplit launch has
  // nothing to divide)
  auto item_split = [&](int li) {
    const int t = walk.chunk_begin + li;
    return GROUPED ? t / total_tiles : p.splits == 1 ? 0 : fast_div(t, p.div_tiles_mul, p.div_tiles_shift);
  };
  auto item_tile = [&](int li) {
    const int t = walk.chunk_begin + li;
    return GROUPED ? t % total_tiles : p.splits == 1 ? t : t - fast_div(t, p.div_tiles_mul, p.div_tiles_shift) * total_tiles;
  };
  auto split_begin = [&](int sp) { return sp * p.steps_per_split; };
  auto split_end = [&](int sp) { return min((sp + 1) * p.steps_per_split, k_steps); };
  int total_steps = 0;
  for (int li = walk.slot; li < walk.chunk_len; li += walk.slots)
    total_steps += split_end(item_split(li)) - split_begin(item_split(li));

  // item -> tile location. Plain form: grouped walk order over the tile grid. Grouped form:
  // the walker steps through m_sizes until it reaches the group that holds the tile.
  auto locate = [&](GroupWalk& w, int li) -> TileLoc {
    const int tile = item_tile(li);
    if (!GROUPED) {
      int tm, tn;
      tile_coords(tile, p.tiles_m, p.tiles_n, p.div_group_mul, p.div_group_shift, tm, tn);
      return TileLoc{tm * BM, p.M, tn * BN, 0};
    }
    while (tile >= w.tile_end && w.group + 1 < p.groups) {
      w.row_begin += group_rows(w.group, w.row_begin);
      ++w.group;
      w.tiles_m = (group_rows(w.group, w.row_begin) + BM - 1) / BM;
      w.tile_begin = w.tile_end;
      w.tile_end += w.tiles_m * p.tiles_n;
    }
    const int t = tile - w.tile_begin;
    const int tm = t % max(w.tiles_m, 1), tn = t / max(w.tiles_m, 1);
    return TileLoc{w.row_begin + tm * BM, w.row_begin + group_rows(w.group, w.row_begin), tn * BN, w.group};
  };
  auto first_group = [&]() -> GroupWalk {
    GroupWalk w = {0, 0, 0, 0, 0};
    if (GROUPED) {
      w.tiles_m = (group_rows(0, 0) + BM - 1) / BM;
      w.tile_end = w.tiles_m * p.tiles_n;
    }
    return w;
  };
  GroupWalk walk_a = first_group(), walk_b = first_group(), walk_c = first_group();

  // ---- load side of the pipeline
  StepCursor ca = {walk.slot, 0, 0, 0, 0, 0}, cb = {walk.slot, 0, 0, 0, 0, 0};
  // STREAM_B launches start every tile column at a different K step and wrap around. Their
  // workgroups stream disjoint rows of B in lockstep; with a power-of-two row pitch all the
  // addresses in flight at one moment would agree in their low bits and crowd a few memory
  // channels (M=32, N=57344, K=8192 with an 8192-byte pitch: 100 us; the same data at a pitch
  // of 8320 bytes: 71 us). The sum over K does not care where it starts. Launches whose tiles
  // share panels of B through the L2 keep the common order: there the sharing needs it. So do
  // plans with more than two splits, whose items are already spread over K (M=128, N=K=8192 with
  // four splits lost 5 % to the rotation; two splits gain 5 %, unsplit plans 11-28 %).
  auto start_cursor = [&](StepCursor& c, int li, const TileLoc& loc) {
    c.kt_begin = split_begin(item_split(li));
    c.kt_end = split_end(item_split(li));
    c.left = c.kt_end - c.kt_begin;
    c.kt = c.kt_begin + (STREAM_B && p.splits <= 2 ? (loc.n0 / BN) % c.left : 0);
  };
  // Source of the loads: one buffer descriptor per operand and tile, base = the tile's first row,
  // extent = its valid rows (the hardware returns zeros for anything past the extent, so rows past
  // the matrix edge need neither clamping nor predication: they read as zeros and are never
  // stored). A lane's 16 bytes in the i-th 8-row group a wave fetches (grp = wave + NW*i) lie at
  //   lane part (vector register, the same for every group, step and tile: ld_row*ld + chunk,
  //              the chunk swizzle depends on the group's parity only, which a wave's groups share)
  // + scalar part (K offset + 8*grp*ld, one scalar add per load).
  // The range check adds the two before it compares, so the sum must stay below 2^32: the host
  // admits leading dimensions up to 2^31 / 256.
  static_assert(NW % 2 == 0, "all groups of a wave must share their parity");
  struct OperandSrc {
    const uint8_t* base;
    uint32_t extent;                  // bytes from base that may be read
    uint32_t wave_off, group_stride;  // 8*wave*ld and 8*NW*ld
  };
  constexpr int kRsrcFlags = 0x00020000;  // raw buffer, 32-bit data format: plain byte addressing with range check
  auto make_src = [&](const uint8_t* base, int rows_valid, int rows_tile, long ld) -> OperandSrc {
    // (a tile always starts on a valid row, so rows_valid >= 1; clamping at zero as well would turn
    // the pair into a three-operand median, which exists as a vector instruction only and would
    // pull the descriptor out of the scalar registers)
    const uint32_t extent = (uint32_t)min(rows_valid, rows_tile) * (uint32_t)ld;
    // Base and extent are the same for every lane; they are pinned to scalar registers because a
    // descriptor that the compiler takes for lane-dependent (the grouped form derives these from
    // sizes it loads, through a clamp that only exists as a vector instruction) makes every load a
    // loop over the distinct descriptors of the wave.
    OperandSrc o;
    const uintptr_t b = reinterpret_cast<uintptr_t>(base);
    o.base = reinterpret_cast<const uint8_t*>(
        ((uintptr_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(b >> 32)) << 32) |
        (uintptr_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)b));
    o.extent = (uint32_t)__builtin_amdgcn_readfirstlane((int)extent);
    o.wave_off = 8u * (uint32_t)wave * (uint32_t)ld;
    o.group_stride = 8u * NW * (uint32_t)ld;
    return o;
  };
  // 24-bit multiplies (row < 8, leading dimension < 2^24 by the host's check)
  const uint32_t lane_chunk = (uint32_t)ld_chunk_off(wave);
  const uint32_t a_lane = __umul24((uint32_t)ld_row, (uint32_t)p.lda) + lane_chunk;
  const uint32_t b_lane = __umul24((uint32_t)ld_row, (uint32_t)p.ldb) + lane_chunk;
  // K tail (KTAIL kernels only): in the partial last step, lanes whose chunk lies at or past K
  // must fetch zeros (whatever follows a row in memory could decode to NaN): their lane part is
  // pushed past every extent for that step. A lane's logical chunk is the same for all its
  // groups.
  const bool tail_chunk_ok = ((ld_pc ^ swz128(wave * 8 + ld_row)) * kChunk) < k_tail;
  constexpr uint32_t kPastExtent = 0x80000000u;  // extents and scalar parts stay below 2^31
  const uint32_t a_lane_tail = tail_chunk_ok ? a_lane : kPastExtent;
  const uint32_t b_lane_tail = tail_chunk_ok ? b_lane : kPastExtent;
  OperandSrc a_src = {nullptr, 0, 0, 0}, b_src = {nullptr, 0, 0, 0};
  auto setup_a = [&](int li) {
    const TileLoc loc = locate(walk_a, li);
    start_cursor(ca, li, loc);
    a_src = make_src(p.a + (size_t)loc.m0 * p.lda, loc.m_end - loc.m0, BM, p.lda);
  };
  auto setup_b = [&](int li) {
    const TileLoc loc = locate(walk_b, li);
    start_cursor(cb, li, loc);
    b_src = make_src(p.b + ((size_t)loc.group * p.N + loc.n0) * p.ldb, p.N - loc.n0, BN, p.ldb);
  };
  // i-th group of one operand's step kt into the stage at sbase
  // (step_off: K offset of the step + the wave's first group, prepared once per step)
  auto load_group = [&](auto stream_tag, const OperandSrc& src, uint32_t lane_off, uint32_t step_off, int i, uint8_t* sbase) {
    // (the descriptor is put together from its scalar parts here: one scalar instruction)
    const __amdgpu_buffer_rsrc_t rsrc =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t*>(src.base), 0, (int)src.extent, kRsrcFlags);
    load_chunk_to_lds<decltype(stream_tag)::value>(rsrc, sbase + (wave + NW * i) * 1024, lane_off,
                                                   step_off + (uint32_t)i * src.group_stride);
  };
  auto lane_part = [&](uint32_t whole, uint32_t tail, int kt) -> uint32_t {
    return KTAIL && kt >= k_full ? tail : whole;
  };
  // Ring positions the next loads of A and of B go to (= issued % stages, kept as counters that wrap).
  int fill_a = 0, fill_b = 0;
  auto next_fill_a = [&]() { fill_a = (fill_a + 1 == kStagesA) ? 0 : fill_a + 1; };
  auto next_fill_b = [&]() { fill_b = (fill_b + 1 == kStagesB) ? 0 : fill_b + 1; };
  // Issues one operand's loads for its cursor's step into the next stage of its ring. Past the
  // last step it re-issues the last one into a stage nobody reads again, which keeps the
  // path free of branches.
  auto issue_a = [&]() {
    const uint32_t lo = lane_part(a_lane, a_lane_tail, ca.kt);
#pragma unroll
    for (int i = 0; i < A_GROUPS; ++i)
      load_group(std::false_type{}, a_src, lo, (uint32_t)ca.kt * kStepK + a_src.wave_off, i, lds + fill_a * STAGE_A);
    next_fill_a();
    ++ca.issued;
  };
  auto issue_b = [&]() {
    const uint32_t lo = lane_part(b_lane, b_lane_tail, cb.kt);
#pragma unroll
    for (int i = 0; i < B_GROUPS; ++i)
      load_group(std::integral_constant<bool, STREAM_B>{}, b_src, lo, (uint32_t)cb.kt * kStepK + b_src.wave_off, i,
                 lds + LDS_B0 + fill_b * STAGE_B);
    next_fill_b();
    ++cb.issued;
  };
  // Moves a load cursor to its next step. PLAIN: the caller knows that the next step belongs to the
  // same work item (true for all but the last DIST + 1 steps of an item): no branch, no tile set-up.
  auto advance_a = [&](auto plain_tag) {
    if (!decltype(plain_tag)::value) {
      if (ca.issued >= total_steps) return;  // stay on the last step
      if (--ca.left == 0) {
        ca.item += walk.slots;
        setup_a(ca.item);
        return;
      }
    } else {
      --ca.left;
    }
    ca.kt = (ca.kt + 1 == ca.kt_end) ? ca.kt_begin : ca.kt + 1;
  };
  auto advance_b = [&](auto plain_tag) {
    if (!decltype(plain_tag)::value) {
      if (cb.issued >= total_steps) return;
      if (--cb.left == 0) {
        cb.item += walk.slots;
        setup_b(cb.item);
        return;
      }
    } else {
      --cb.left;
    }
    cb.kt = (cb.kt + 1 == cb.kt_end) ? cb.kt_begin : cb.kt + 1;
  };

  // ---- operand fragments: two register sets; each fragment is two 16-byte LDS reads
  struct Frag {
    v4i lo, hi;
  };
  Frag xa[MT], xb[NT], ya[MT], yb[NT];
  auto read_lo = [&](const uint8_t* rows, int s, int i) -> v4i {
    return *(const v4i*)(rows + i * 32 * kStepK + rd_off[s][0]);
  };
  auto read_hi = [&](const uint8_t* rows, int s, int i) -> v4i {
    return *(const v4i*)(rows + i * 32 * kStepK + rd_off[s][1]);
  };
  auto as_v8 = [](const Frag& f) -> v8i {
    return (v8i){f.lo[0], f.lo[1], f.lo[2], f.lo[3], f.hi[0], f.hi[1], f.hi[2], f.hi[3]};
  };

  v16f acc[MT][NT];  // defined by the first step of every work item
  // BLOCKSCALE only. The sum over K blocks of s_k * P_k (P_k the unscaled product of block k) is
  // kept in units of the current block's factor: before step k adds P_k the accumulators are
  // multiplied by s_(k-1) / s_k, and the epilogue multiplies by the last factor. One multiply per
  // accumulator and step on the vector ALU, under the MFMAs' cover, and no second accumulator
  // set: the kernel keeps the register budget of the plain 128x128 tile (two workgroups per CU).
  // A factor of exactly zero is replaced by 2^-60 (its block then contributes P_k * 2^-60, nothing
  // at the output's precision); factors are expected to span less than 2^60 within a row of blocks.
  // Blocks 0 .. n-2 are rescaled in phase [B] of the step before (each under the cover of the next
  // block's MFMA), the last one under the first MFMA of the step itself.
  // s_pend / s_cur: the ratios to the next step / to this one; kt_c: the K step the compute side is
  // at; the lane's share of the item's factors and ratios (sc[r], rt[r] belong to step 64*r + lane).
  float s_pend = 1.0f, s_cur = 1.0f, s_last = 1.0f, n_pend = 1.0f, n_last = 1.0f;
  int kt_c = 0;
  constexpr int SC_REGS = 4;  // 256 steps = K up to 32768
  float sc[SC_REGS] = {0.f, 0.f, 0.f, 0.f}, rt[SC_REGS] = {1.f, 1.f, 1.f, 1.f};
  auto load_block_scales = [&](const TileLoc& loc) {
    // the scale block of this wave's tile (clamped for waves that lie past the matrix edge)
    const int mb = min(loc.m0 + wm * WTM, p.M - 1) / 128, nb = min(loc.n0 + wn * WTN, p.N - 1) / 128;
    const float* sa = p.a_scale + (size_t)mb * k_steps;
    const float* sb = p.b_scale + (size_t)nb * k_steps;
    auto factor = [&](int kb) -> float {
      const float f = sa[kb] * sb[kb];
      return f == 0.0f ? 0x1p-60f : f;
    };
#pragma unroll
    for (int r = 0; r < SC_REGS; ++r) {
      const int kb = min(r * 64 + lane, k_steps - 1);
      sc[r] = factor(kb);
      rt[r] = kb > 0 ? factor(kb - 1) / sc[r] : 1.0f;
    }
  };
  auto lane_value = [&](const float (&regs)[SC_REGS], int kt) -> float {
    const int r = kt >> 6;
    const float v = r == 0 ? regs[0] : r == 1 ? regs[1] : r == 2 ? regs[2] : regs[3];
    return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), kt & 63));
  };
  // brings block t of the accumulators from one step's factor to the next one's
  auto fold_block = [&](int t, float ratio) {
    const int i = t / NT, j = t % NT;
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[i][j][v] *= ratio;
  };

  // t-th MFMA of a half step (t = i*NT + j) on fragment set (fa, fb)
  // (fresh: the block's first MFMA of a tile starts from zero instead of the old contents)
  auto mfma_one = [&](const Frag (&fa)[MT], const Frag (&fb)[NT], int t, bool fresh) {
    const int i = t / NT, j = t % NT;
    const v16f zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(as_v8(fb[j]), as_v8(fa[i]), fresh ? zero : acc[i][j], 0, 0, 0, 0, 0, 0);
  };
  // u-th of the 2*(MT+NT) LDS reads that fill fragment set (fa, fb) with K half s
  auto read_one = [&](Frag (&fa)[MT], Frag (&fb)[NT], const uint8_t* rows_a, const uint8_t* rows_b, int s, int u) {
    const int f = u >> 1;
    if (f < MT) {
      if (u & 1) fa[f].hi = read_hi(rows_a, s, f);
      else fa[f].lo = read_lo(rows_a, s, f);
    } else {
      if (u & 1) fb[f - MT].hi = read_hi(rows_b, s, f - MT);
      else fb[f - MT].lo = read_lo(rows_b, s, f - MT);
    }
  };
  // Per half step: NMFMA MFMAs, NREAD LDS reads, A_GROUPS or B_GROUPS global->LDS loads, the
  // memory instructions placed behind the MFMAs: load l in slot l*NMFMA/GROUPS, the reads RPS
  // per slot in the first half of the slots. The reads have then returned while the last
  // MFMAs still execute, so the wait at the end of the half step (for the barrier, or for
  // the fragments of the next half) costs the matrix pipe nothing.
  constexpr int NMFMA = MT * NT, NREAD = 2 * (MT + NT);
  constexpr int RPS = (NREAD + NMFMA / 2 - 1) / (NMFMA / 2);

  // ---- prologue: A(0) B(0) .. A(DIST-1) B(DIST-1) in flight, first fragments in registers
  setup_a(ca.item);
  setup_b(cb.item);
#pragma unroll
  for (int d = 0; d < DIST; ++d) {
    issue_a(); advance_a(std::false_type{});
    issue_b(); advance_b(std::false_type{});
  }
  wait_loads_and_barrier<(DIST - 1) * (A_GROUPS + B_GROUPS)>();
#pragma unroll
  for (int u = 0; u < NREAD; ++u) read_one(xa, xb, lds + a_rd_base, lds + b_rd_base, 0, u);

  // ---- epilogue. The MFMA leaves lane (l32, half) with row l32 of every 32x32 block and the
  // columns 8*q + 4*half + e (register 4*q + e): storing from there would touch 32 rows per
  // instruction. Instead a lane finishes its own elements first - a_scale[m], b_scale[n], bias[n]
  // in fp32, one rounding to the 16-bit output type, two results per register - and each 32-row
  // block of the wave's tile is then turned through LDS, PASS_J 32-column blocks at a time, as
  // 16-bit values: read back, a lane holds 8 consecutive columns of one row and stores its 16
  // bytes, so a wave-wide store covers whole rows of the pass.
  //
  // The turn-table is the wave's own share (the 1 KB groups it fills itself) of the B stage
  // that held this tile's last step: every wave finished reading that stage before the
  // step's barrier, and only this wave will load into these groups again. A pass fills half of
  // it, so the passes alternate between two halves: while one pass is read back and stored, the
  // next is converted and written (LDS runs a wave's operations in order, so neither half needs
  // a wait before it is written again). A pass row is CPR 16-byte chunks; chunk c of row r sits
  // at chunk position c ^ key(r): the 16-byte reads of 8 lanes spread over all banks, the 8-byte
  // writes of 16 consecutive rows meet in pairs (a two-way conflict on 64 of the epilogue's
  // instructions, which are bound by their arithmetic; undoing it costs the readers register moves).
  constexpr int PASS_J = B_GROUPS / 4;          // 32-column blocks per pass (2 KB of 16-bit values each)
  constexpr int NJP = NT / PASS_J;              // passes per 32-row block
  constexpr int CPR = PASS_J * 4;               // 16-byte chunks per pass row
  constexpr int ROW_BYTES = CPR * 16;
  constexpr int ROWS_PER_GROUP = 1024 / ROW_BYTES;
  constexpr int GROUPS_PER_PASS = 32 / ROWS_PER_GROUP;  // = B_GROUPS / 2
  constexpr int LPR = CPR;                      // lanes per row when reading back (one chunk each)
  constexpr int ROWS_PER_READ = 64 / LPR;
  constexpr int ITERS = 32 / ROWS_PER_READ;
  static_assert(B_GROUPS % 4 == 0 && NT % PASS_J == 0 && (CPR == 4 || CPR == 8) && 2 * GROUPS_PER_PASS == B_GROUPS,
                "turn-table geometry");
  auto epilogue = [&](const TileLoc& loc, auto vector_tag, auto f16_tag, uint8_t* free_b_stage) {
    const int m0 = loc.m0, n0 = loc.n0;
    // VECTOR: C takes 16-byte stores (base and row pitch aligned, N a multiple of 8, so no lane's 8
    // columns straddle the edge). Edge tiles take it too: rows past the edge fall outside the output
    // descriptor's extent and lanes past column N are sent there. Anything else stores element by element.
    constexpr bool VECTOR = decltype(vector_tag)::value;
    constexpr bool OUT_F16 = decltype(f16_tag)::value;      // IEEE binary16 instead of bf16
    // row r of the pass kept in half h of the table
    auto row_addr = [&](int h, int r) -> uint8_t* {
      return free_b_stage + (wave + NW * (h * GROUPS_PER_PASS + r / ROWS_PER_GROUP)) * 1024 + (r % ROWS_PER_GROUP) * ROW_BYTES;
    };
    auto key = [](int r) { return (r * ROW_BYTES / 128) % CPR; };
    // The lane-dependent addresses below are the same for every tile; derived from an opaque
    // copy of the lane id they are recomputed here (a few integer operations) instead of
    // being hoisted out of the tile loop, where they would occupy registers through the K loop.
    // (the lane id itself comes from the hardware's lane count, inside the opaque statement: as a
    // loop invariant it would be moved in front of the K loop and, with no register to spare there,
    // spilled; its reload at this point waits for every load in flight)
    int lane_e;
    asm volatile("v_mbcnt_lo_u32_b32 %0, -1, 0\n\tv_mbcnt_hi_u32_b32 %0, -1, %0" : "=v"(lane_e));
    const int l32 = lane_e & 31, half = lane_e >> 5;
    const int wr_key = key(l32);
    const int wr_half = half * 8;  // where this lane's 8 bytes sit inside a chunk
    const int rd_row = lane_e / LPR, rd_chunk = lane_e % LPR;  // 8 columns of the pass row this lane stores
    const int rd_col = rd_chunk * 8;

    // scales and bias of the lane's own elements: row l32 of every 32-row block, columns
    // 32*j + 8*q + 4*half + e, fetched through descriptors that end at column N (whatever lies
    // past it reads as zero and belongs to columns that are never stored), four at a time
    // whatever the alignment; only a bias that starts on an odd element is fetched one by one.
    // (the bias stays as loaded, two bf16 per register, and is widened where it is used)
    float sam[MT], sbv[NT][4][4];
    us4 bv[HAS_BIAS ? NT : 1][4];
#pragma unroll
    for (int i = 0; i < MT; ++i)
      sam[i] = BLOCKSCALE ? s_last : p.a_scale[min(m0 + wm * WTM + i * 32 + l32, loc.m_end - 1)];
    if (!BLOCKSCALE) {
      const int n_wave = n0 + wn * WTN;               // first column of the wave's tile
      const int n_left = __builtin_amdgcn_readfirstlane(max(p.N - n_wave, 0));  // columns from there to the edge
      const __amdgpu_buffer_rsrc_t s_rsrc = __builtin_amdgcn_make_buffer_rsrc(
          const_cast<float*>(p.b_scale) + ((GROUPED ? (size_t)loc.group * p.N : 0) + n_wave), 0, n_left * 4, 0x00020000);
      const __amdgpu_buffer_rsrc_t bias_rsrc = __builtin_amdgcn_make_buffer_rsrc(
          const_cast<uint16_t*>(HAS_BIAS ? p.bias + n_wave : nullptr), 0, HAS_BIAS ? n_left * 2 : 0, 0x00020000);
      // (the check works on whole 4-byte words: with an odd N the last word of the bias is half inside.
      // Fetched four at a time from a 4-byte aligned base that word is read whole: it cannot cross a
      // page, and its upper half belongs to a column that is never stored.)
      const __amdgpu_buffer_rsrc_t bias4_rsrc = __builtin_amdgcn_make_buffer_rsrc(
          const_cast<uint16_t*>(HAS_BIAS ? p.bias + n_wave : nullptr), 0, HAS_BIAS ? ((n_left + 1) & ~1) * 2 : 0, 0x00020000);
      const bool bias_by_four = (reinterpret_cast<uintptr_t>(p.bias) & 3) == 0;  // (n_wave is a multiple of 32)
#pragma unroll
      for (int j = 0; j < NT; ++j) {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const uint32_t col = (uint32_t)(j * 32 + 8 * q + 4 * half);
          const v4f s4 = load_f32x4_checked(s_rsrc, col * 4);
#pragma unroll
          for (int e = 0; e < 4; ++e) sbv[j][q][e] = s4[e];
          if (HAS_BIAS) {
            if (bias_by_four) {
              bv[HAS_BIAS ? j : 0][q] = load_u16x4_checked(bias4_rsrc, col * 2);
            } else {
#pragma unroll
              for (int e = 0; e < 4; ++e) bv[HAS_BIAS ? j : 0][q][e] = load_u16_checked(bias_rsrc, (col + e) * 2);
            }
          }
        }
      }
    } else {  // the factors were applied step by step
#pragma unroll
      for (int j = 0; j < NT; ++j)
#pragma unroll
        for (int q = 0; q < 4; ++q)
#pragma unroll
          for (int e = 0; e < 4; ++e) sbv[j][q][e] = 1.0f;
    }
    // pass pp = (32-row block i, column blocks jp*PASS_J ..): finished 16-bit values into half pp & 1.
    // One 32x32 block at a time in three sweeps over its 16 values (row scale, column scale and
    // bias, rounding): neighbouring instructions then do not wait for each other's results.
    auto convert_and_write = [&](int pp) {
      const int i = pp / NJP, jp = pp % NJP;
      uint8_t* const wr_row = row_addr(pp & 1, l32);
#pragma unroll
      for (int jj = 0; jj < PASS_J; ++jj) {
        const int j = jp * PASS_J + jj;
        float t[16], x[16];
        uint32_t packed[8];
#pragma unroll
        for (int v = 0; v < 16; ++v) t[v] = acc[i][j][v] * sam[i];
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int v = 0; v < 16; ++v)
          x[v] = HAS_BIAS ? __builtin_fmaf(t[v], sbv[j][v / 4][v % 4], bf16_to_f32(bv[HAS_BIAS ? j : 0][v / 4][v % 4]))
                          : t[v] * sbv[j][v / 4][v % 4];
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int v = 0; v < 8; ++v) packed[v] = pack_out_x2(x[2 * v], x[2 * v + 1], OUT_F16);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int q = 0; q < 4; ++q)
          *(v2u*)(wr_row + (((jj * 4 + q) ^ wr_key) * 16) + wr_half) = (v2u){packed[2 * q], packed[2 * q + 1]};
      }
    };
    // The wave's part of the tile as a buffer: origin at its first element, extent = its valid rows
    // (none for a wave that lies past the edge); offsets stay below 2^31 by the host's check of ldc.
    const uint32_t c_row_bytes = (uint32_t)p.ldc * 2u;
    // (pinned to a scalar register: the double clamp exists as a vector instruction only, and a
    // descriptor held in vector registers makes every store a loop)
    const int c_rows = __builtin_amdgcn_readfirstlane(min(max(loc.m_end - (m0 + wm * WTM), 0), WTM));
    const __amdgpu_buffer_rsrc_t c_rsrc = __builtin_amdgcn_make_buffer_rsrc(
        p.c + ((size_t)(m0 + wm * WTM) * p.ldc + n0 + wn * WTN), 0, (int)((uint32_t)c_rows * c_row_bytes), 0x00020000);
    const uint32_t c_lane = (uint32_t)rd_row * c_row_bytes + (uint32_t)rd_col * 2u;
    constexpr int NP = MT * NJP;
    __builtin_amdgcn_sched_barrier(0);
    convert_and_write(0);
#pragma unroll
    for (int pp = 0; pp < NP; ++pp) {
      const int i = pp / NJP, jp = pp % NJP;
      __builtin_amdgcn_sched_barrier(0);
      v4i rows16[ITERS];
#pragma unroll
      for (int it = 0; it < ITERS; ++it) {
        const int r = it * ROWS_PER_READ + rd_row;
        rows16[it] = *(const v4i*)(row_addr(pp & 1, r) + ((rd_chunk ^ key(r)) * 16));
      }
      __builtin_amdgcn_sched_barrier(0);
      if (pp + 1 < NP) convert_and_write(pp + 1);  // under the latency of the reads above
      __builtin_amdgcn_sched_barrier(0);
      const int n = n0 + wn * WTN + jp * PASS_J * 32 + rd_col;
      // (a lane whose columns lie past N is sent past the extent: its stores are dropped)
      const uint32_t c_lane_pass = n < p.N ? c_lane : 0x80000000u;
#pragma unroll
      for (int it = 0; it < ITERS; ++it) {
        const int r = it * ROWS_PER_READ + rd_row;
        const v4i out = rows16[it];
        if (VECTOR) {
          // lane part (rd_row, rd_col) + scalar part (block row, read round, pass column)
          store_chunk_streaming(out, c_rsrc, c_lane_pass,
                                (uint32_t)(i * 32 + it * ROWS_PER_READ) * c_row_bytes + (uint32_t)(jp * PASS_J * 32 * 2));
        } else {
          const int m = m0 + wm * WTM + i * 32 + r;
          uint16_t* dst = p.c + (size_t)m * p.ldc + n;
          if (m < loc.m_end) {
#pragma unroll
            for (int e = 0; e < 8; ++e)
              if (n + e < p.N) dst[e] = (uint16_t)((unsigned)out[e / 2] >> (16 * (e & 1)));
          }
        }
      }
    }
    __builtin_amdgcn_sched_barrier(0);
  };

  // ---- split-K: raw fp32 partial sums of this item to partial[split][m][n]: the lane layout the
  // MFMA leaves (4 consecutive n per lane), one 16-byte buffer store per 4 values when N is a multiple
  // of 4: rows past M fall outside the descriptor's extent, lanes past N are sent there, and the
  // values go from the accumulators to memory without passing through other registers.
  auto store_partial = [&](int m0, int n0, int split) {
    int lane_e;  // (inside the opaque statement for the reason given in the epilogue)
    asm volatile("v_mbcnt_lo_u32_b32 %0, -1, 0\n\tv_mbcnt_hi_u32_b32 %0, -1, %0" : "=v"(lane_e));
    const int l32 = lane_e & 31, half = lane_e >> 5;
    float* base = p.partial + (size_t)split * p.M * p.N;
    if ((p.N & 3) == 0) {
      const uint32_t row_bytes = (uint32_t)p.N * 4u;  // (N*4*128 < 2^31 by the host's check of the workspace plan)
      const int rows = __builtin_amdgcn_readfirstlane(min(max(p.M - (m0 + wm * WTM), 0), WTM));  // (scalar: see the epilogue)
      const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(
          base + ((size_t)(m0 + wm * WTM) * p.N + n0 + wn * WTN), 0, (int)((uint32_t)rows * row_bytes), 0x00020000);
      const uint32_t lane_off = (uint32_t)l32 * row_bytes + (uint32_t)(4 * half) * 4u;
#pragma unroll
      for (int j = 0; j < NT; ++j) {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int n = n0 + wn * WTN + j * 32 + 8 * q + 4 * half;
          const uint32_t lo = n < p.N ? lane_off : 0x80000000u;
#pragma unroll
          for (int i = 0; i < MT; ++i) {
            const v4f v = {acc[i][j][4 * q], acc[i][j][4 * q + 1], acc[i][j][4 * q + 2], acc[i][j][4 * q + 3]};
            store_f32x4_checked(v, rsrc, lo, (uint32_t)(i * 32) * row_bytes + (uint32_t)(j * 32 + 8 * q) * 4u);
          }
        }
      }
    } else {
#pragma unroll
      for (int i = 0; i < MT; ++i) {
        const int m = m0 + wm * WTM + i * 32 + l32;
#pragma unroll
        for (int j = 0; j < NT; ++j) {
          __builtin_amdgcn_sched_barrier(0);
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            const int n = n0 + wn * WTN + j * 32 + 8 * q + 4 * half;
            if (m < p.M) {
              float* dst = base + (size_t)m * p.N + n;
#pragma unroll
              for (int e = 0; e < 4; ++e)
                if (n + e < p.N) dst[e] = acc[i][j][4 * q + e];
            }
          }
        }
      }
    }
    __builtin_amdgcn_sched_barrier(0);
  };

  int sa = 0, sb = 0;  // stages holding the step being computed
  const uint8_t* cur_a = lds + a_rd_base;  // where this wave reads the step being computed ...
  const uint8_t* cur_b = lds + b_rd_base;
  const uint8_t* nxt_a = cur_a;            // ... and the step after it
  const uint8_t* nxt_b = cur_b;
  // What a phase's loads need, put together while the previous phase's last MFMAs run: between
  // the last MFMA of one phase and the first of the next a wave, which issues its instructions in
  // order, should find as little as possible (every scalar instruction there is time the matrix
  // pipe waits once its 64 cycles of cover are used up).
  struct LoadPhase {
    uint32_t lane_off, step_off;
    uint8_t* stage;
  };
  LoadPhase ph_a = {0, 0, lds}, ph_b = {0, 0, lds};  // loads of A (issued in phase [B]) / of B (issued in phase [A])
  auto prepare_b_loads = [&]() {
    ph_b.lane_off = lane_part(b_lane, b_lane_tail, cb.kt);
    ph_b.step_off = (uint32_t)cb.kt * kStepK + b_src.wave_off;
    ph_b.stage = lds + LDS_B0 + fill_b * STAGE_B;
    next_fill_b();
    ++cb.issued;
  };
  auto prepare_a_loads = [&]() {
    ph_a.lane_off = lane_part(a_lane, a_lane_tail, ca.kt);
    ph_a.step_off = (uint32_t)ca.kt * kStepK + a_src.wave_off;
    ph_a.stage = lds + fill_a * STAGE_A;
    next_fill_a();
    ++ca.issued;
  };
  constexpr int B_LAST = (B_GROUPS - 1) * NMFMA / B_GROUPS;  // slots of a phase's last load
  constexpr int A_LAST = (A_GROUPS - 1) * NMFMA / A_GROUPS;
  // One K step. READ_NEXT: fetch the first-half fragments of the following step behind the
  // second-half MFMAs (left out on a tile's last step, so that the epilogue has those
  // registers; the fragments are then read after it).
  // PLAIN: neither load cursor leaves its work item in this step.
  // slots behind which the next phase is prepared (two, so that neither holds more scalar work than
  // an MFMA covers)
  constexpr int PREP_T = NMFMA / 2, PREP_T2 = NMFMA >= 8 ? NMFMA / 2 + 1 : NMFMA / 2;
  auto step = [&](auto first_tag, auto read_next_tag, auto plain_tag) {
    constexpr bool FIRST = decltype(first_tag)::value;
    constexpr bool READ_NEXT = decltype(read_next_tag)::value;
    if (BLOCKSCALE) {  // (fetched from the lanes that hold them during the previous step, or at the item's start)
      s_cur = s_pend;    // ratio that brought the accumulators to this step
      s_pend = n_pend;   // ratio to the next step (applied in phase [B])
      s_last = n_last;   // this step's factor: what the epilogue multiplies by after the last step
    }

    // [A] MFMAs on x* (first K half of this step). Behind them, one per MFMA: the LDS reads
    //     of the second half (-> y*), and behind every other one a global->LDS load of
    //     B(g+DIST) into the B stage released at the previous barrier. The fences pin this
    //     interleaving: every wave-level memory instruction hides behind an MFMA, and the
    //     load queue never holds more than the matrix pipe can cover. Half way through, phase [B]
    //     is prepared; behind the last loads the B cursor moves on. Behind the phase's last MFMA
    //     there is nothing but the wait and the barrier, which its 64 cycles cover.
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int t = 0; t < NMFMA; ++t) {
      mfma_one(xa, xb, t, FIRST);
      __builtin_amdgcn_sched_barrier(0);  // the MFMA goes first: what follows is issued under its cover
      // (the last block of the previous step is brought to this step's units here, under the first MFMA's cover)
      if (BLOCKSCALE && !FIRST && t == 0) fold_block(NMFMA - 1, s_cur);
#pragma unroll
      for (int l = 0; l < B_GROUPS; ++l)
        if (l * NMFMA / B_GROUPS == t)
          load_group(std::integral_constant<bool, STREAM_B>{}, b_src, ph_b.lane_off, ph_b.step_off, l, ph_b.stage);
#pragma unroll
      for (int u = t * RPS; u < (t + 1) * RPS; ++u)
        if (u < NREAD) read_one(ya, yb, cur_a, cur_b, 1, u);
      if (t == B_LAST) advance_b(plain_tag);
      if (t == PREP_T) prepare_a_loads();
      if (BLOCKSCALE && t == PREP_T) {
        n_pend = lane_value(rt, min(kt_c + 2, k_steps - 1));
        n_last = lane_value(sc, min(kt_c + 1, k_steps - 1));
      }
      if (t == PREP_T2) {
        sa = (sa + 1 == kStagesA) ? 0 : sa + 1;
        sb = (sb + 1 == kStagesB) ? 0 : sb + 1;
        nxt_a = lds + a_rd_base + sa * STAGE_A;
        nxt_b = lds + b_rd_base + sb * STAGE_B;
      }
      __builtin_amdgcn_sched_barrier(0);
    }

    // own loads of A(g+1) and B(g+1) have landed (the younger B(g+2) .. B(g+DIST) and
    // A(g+2) .. A(g+DIST-1) may still be in flight); past the barrier everyone's have, and
    // every wave is done reading this step's stages
    wait_loads_and_barrier<(DIST - 1) * B_GROUPS + (DIST - 2) * A_GROUPS>();

    // [B] MFMAs on y* (second K half); behind them the loads of A(g+DIST) into the A stage just
    //     released and the LDS reads of step g+1's first half (-> x*; at the end of a tile
    //     these already belong to the next tile)
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int t = 0; t < NMFMA; ++t) {
      mfma_one(ya, yb, t, false);
      __builtin_amdgcn_sched_barrier(0);
      // block t-1 has had its last MFMA of this step: into the next step's units, under this MFMA's cover
      if (BLOCKSCALE && READ_NEXT && t >= 1) fold_block(t - 1, s_pend);
#pragma unroll
      for (int l = 0; l < A_GROUPS; ++l)
        if (l * NMFMA / A_GROUPS == t) load_group(std::false_type{}, a_src, ph_a.lane_off, ph_a.step_off, l, ph_a.stage);
#pragma unroll
      for (int u = t * RPS; u < (t + 1) * RPS; ++u)
        if (READ_NEXT && u < NREAD) read_one(xa, xb, nxt_a, nxt_b, 0, u);
      if (t == A_LAST) advance_a(plain_tag);
      if (t == PREP_T) {
        prepare_b_loads();
        cur_a = nxt_a;
        cur_b = nxt_b;
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    if (BLOCKSCALE) ++kt_c;
  };
  auto read_first_half = [&]() {
#pragma unroll
    for (int u = 0; u < NREAD; ++u) read_one(xa, xb, cur_a, cur_b, 0, u);
  };

  // Item loop around the K loop. The first step of an item is its own copy of the step code
  // whose first-half MFMAs start from zero: the accumulators then have one live range per
  // item (defined there, dead after the epilogue) and need no clearing or copying between
  // items.
  prepare_b_loads();  // of the first step's phase [A]
  for (int c_item = walk.slot; c_item < walk.chunk_len; c_item += walk.slots) {
    const int c_split = item_split(c_item);
    const int n_steps = split_end(c_split) - split_begin(c_split);
    if (BLOCKSCALE) {
      load_block_scales(locate(walk_c, c_item));
      kt_c = split_begin(c_split);
      n_pend = lane_value(rt, min(kt_c + 1, k_steps - 1));
      n_last = lane_value(sc, kt_c);
    }
    if (n_steps == 1) {
      step(std::true_type{}, std::false_type{}, std::false_type{});
    } else {
      // step k loads for step k + DIST and then moves the cursors to step k + DIST + 1, which is
      // still this item's for k < n_steps - DIST - 1
      step(std::true_type{}, std::true_type{}, std::false_type{});
      int k = 1;
      for (; k < n_steps - DIST - 1; ++k) step(std::false_type{}, std::true_type{}, std::true_type{});
      for (; k < n_steps - 1; ++k) step(std::false_type{}, std::true_type{}, std::false_type{});
      step(std::false_type{}, std::false_type{}, std::false_type{});
    }
    {
      const TileLoc loc = locate(walk_c, c_item);
      if (EPI == kEpiPartial) {
        store_partial(loc.m0, loc.n0, c_split);
      } else {
        // sb already names the next step's stage; the one before it held this tile's last step
        uint8_t* free_b = lds + LDS_B0 + ((sb + kStagesB - 1) % kStagesB) * STAGE_B;
        // 16-byte stores need C's base and row pitch aligned and N a multiple of 8 (no lane's 8 columns
        // straddle the edge); anything else stores element by element
        const uintptr_t bits = reinterpret_cast<uintptr_t>(p.c) | (uintptr_t)(p.ldc * 2) | (uintptr_t)(p.N * 2);
        // (the output type is a compile-time property of the epilogue code: one uniform branch per tile)
        if ((bits & 15) == 0) {
          if (p.out_f16) epilogue(loc, std::true_type{}, std::true_type{}, free_b);
          else epilogue(loc, std::true_type{}, std::false_type{}, free_b);
        } else {
          if (p.out_f16) epilogue(loc, std::false_type{}, std::true_type{}, free_b);
          else epilogue(loc, std::false_type{}, std::false_type{}, free_b);
        }
      }
    }
    read_first_half();  // of the next item's first step (landed before this item's last barrier)
  }
  __builtin_amdgcn_s_waitcnt(0x0070);  // the trailing dummy loads must land before LDS is released
  if (p.stamps && threadIdx.x == 0) {
    unsigned long long* out = p.stamps + 4 * (size_t)blockIdx.x;
    out[0] = stamp_cycles;
    out[1] = __builtin_readcyclecounter();
    out[2] = stamp_ticks;
    out[3] = __builtin_amdgcn_s_memrealtime();
  }
}

// Second pass of a split-K launch: sums the splits' partials in a fixed order (results do not
// depend on scheduling), applies the scales and the bias and rounds to bf16. One thread per
// 4 consecutive columns.
__global__ __launch_bounds__(256) void splitk_finalize_kernel(GemmParams p) {
  fetch_arguments_now(p);
  fetch_tiled_arguments_now(p);
  const long quads_per_row = (p.N + 3) / 4;
  const long idx = (long)blockIdx.x * 256 + threadIdx.x;
  if (idx >= quads_per_row * p.M) return;
  const int m = (int)(idx / quads_per_row);
  const int n = (int)(idx % quads_per_row) * 4;
  const size_t plane = (size_t)p.M * p.N;
  const float* src = p.partial + (size_t)m * p.N + n;
  const bool vec = (p.N & 3) == 0;  // then n + 3 < N and every row start is 16-byte aligned
  const float sa_m = p.a_scale[m];  // fetched beside the partial sums, not after them
  v4f sum = {0.f, 0.f, 0.f, 0.f};
  if (vec) {
    // four splits' loads in flight at a time; added in split order, as the scalar form does
    int s = 0;
    for (; s + 4 <= p.splits; s += 4) {
      v4f part[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) part[u] = __builtin_nontemporal_load((const v4f*)(src + (s + u) * plane));
#pragma unroll
      for (int u = 0; u < 4; ++u) sum += part[u];
    }
    for (; s < p.splits; ++s) sum += __builtin_nontemporal_load((const v4f*)(src + s * plane));
  } else {
    for (int s = 0; s < p.splits; ++s) {
#pragma unroll
      for (int e = 0; e < 4; ++e)
        if (n + e < p.N) sum[e] += src[s * plane + e];
    }
  }
  float r[4];
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    const int ne = min(n + e, p.N - 1);
    const float t = sum[e] * sa_m;
    r[e] = p.bias ? __builtin_fmaf(t, p.b_scale[ne], bf16_to_f32(p.bias[ne])) : t * p.b_scale[ne];
  }
  const uint32_t lo = pack_out_x2(r[0], r[1], p.out_f16), hi = pack_out_x2(r[2], r[3], p.out_f16);
  uint16_t* dst = p.c + (size_t)m * p.ldc + n;
  if (n + 3 < p.N && ((p.ldc & 3) == 0) && ((reinterpret_cast<uintptr_t>(p.c) & 7) == 0)) {
    *(v2u*)dst = (v2u){lo, hi};
  } else {
    dst[0] = (uint16_t)lo;
    if (n + 1 < p.N) dst[1] = (uint16_t)(lo >> 16);
    if (n + 2 < p.N) dst[2] = (uint16_t)hi;
    if (n + 3 < p.N) dst[3] = (uint16_t)(hi >> 16);
  }
}

// ------------------------------------------------------------------------------------
// Generic kernel: operands the other families cannot take (K, lda or ldb not a multiple of 16,
// A or B not 16-byte aligned, leading dimensions beyond a buffer descriptor's range). Byte loads,
// codes widened to f32 in LDS, f32 multiply-adds (the product of two e4m3fn values is exact in
// f32), 64x64 tile per workgroup, 4x4 outputs per lane. A few TFLOP/s: a correct answer for
// odd shapes, not a fast one. Same epilogue arithmetic as the other kernels.
// ------------------------------------------------------------------------------------
__device__ __forceinline__ float e4m3fn_to_f32(uint8_t code) {
  const uint32_t mag = code & 0x7fu;
  // the 7 magnitude bits placed at an f32's exponent/mantissa boundary are the value times 2^-120
  // (subnormal codes become subnormal floats, which the multiply takes as they are)
  float v = __uint_as_float(mag << 20) * 0x1p120f;
  if (mag == 0x7fu) v = __uint_as_float(0x7fc00000u);
  return (code & 0x80u) ? -v : v;
}

constexpr int kGenericTile = 64, kGenericStepK = 32;

__global__ __launch_bounds__(256) void gemm_generic_kernel(GemmParams p) {
  __shared__ float as[kGenericStepK][kGenericTile + 1];
  __shared__ float bs[kGenericStepK][kGenericTile + 1];
  const int tid = threadIdx.x;
  const long m0 = (long)blockIdx.y * kGenericTile, n0 = (long)blockIdx.x * kGenericTile;
  const int ld_row = tid / 4, ld_k = (tid % 4) * 8;  // the 8 bytes of one tile row a lane widens per step
  const int ty = tid / 16, tx = tid % 16;
  float acc[4][4] = {};
  for (long k0 = 0; k0 < p.K; k0 += kGenericStepK) {
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const long k = k0 + ld_k + e;
      const bool in_k = k < p.K;
      as[ld_k + e][ld_row] = in_k && m0 + ld_row < p.M ? e4m3fn_to_f32(p.a[(size_t)(m0 + ld_row) * p.lda + k]) : 0.0f;
      bs[ld_k + e][ld_row] = in_k && n0 + ld_row < p.N ? e4m3fn_to_f32(p.b[(size_t)(n0 + ld_row) * p.ldb + k]) : 0.0f;
    }
    __syncthreads();
#pragma unroll 8
    for (int kk = 0; kk < kGenericStepK; ++kk) {
      float av[4], bv[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) av[i] = as[kk][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) bv[j] = bs[kk][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = __builtin_fmaf(av[i], bv[j], acc[i][j]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const long m = m0 + ty * 4 + i;
    if (m >= p.M) continue;
    const float sa_m = p.a_scale[m];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const long n = n0 + tx * 4 + j;
      if (n >= p.N) continue;
      const float t = acc[i][j] * sa_m;
      const float r = p.bias ? __builtin_fmaf(t, p.b_scale[n], bf16_to_f32(p.bias[n])) : t * p.b_scale[n];
      p.c[(size_t)m * p.ldc + n] = (uint16_t)pack_out_x2(r, 0.0f, p.out_f16);
    }
  }
}

// ------------------------------------------------------------------------------------
// Skinny kernel (M <= 16*MT, HBM-bound): B is streamed exactly once and nothing is reused, so
// what matters is whole-line coalesced loads and as many bytes in flight as a plain copy has.
//
// A workgroup owns 16*NTW rows of B and all of K; its KW waves split K between them in
// interleaved 128-byte steps (wave w takes steps w, w+KW, ...: the workgroup reads KW*128-byte runs
// of every row). Registers are the landing zone: a wave keeps DEPTH steps of loads in flight
// (16 bytes per lane, 8 lanes per row, so every wave-wide load moves 8 whole 128-byte lines;
// letting each MFMA lane fetch its own row instead costs the memory pipeline four times the
// tag look-ups). A landed step is transposed into the MFMA lane layout through a small
// wave-private LDS buffer (swizzled like the tiled kernel's stages); LDS executes a wave's
// operations in order, so the loop needs no barrier. A [16*MT rows] takes the same route.
// Partial 16x16 results are summed across the waves through LDS at the end.
// ------------------------------------------------------------------------------------
template <int MT, int NTW, int DEPTH, int KW>
__global__ __launch_bounds__(KW * 64) void gemm_skinny_kernel(GemmParams p) {
  constexpr int TILE = 16 * kStepK;                 // one 16-row operand tile of one step: 2 KB
  constexpr int NTILE = NTW + MT;                   // tiles per step: B tiles then A tiles
  constexpr int BUF = NTILE * TILE;                 // wave-private transpose buffer
  static_assert(NTW * MT * 1024 <= BUF, "the reduction reuses a wave's buffer for its partials");
  fetch_arguments_now(p);

  extern __shared__ __attribute__((aligned(1024))) uint8_t lds[];

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  uint8_t* buf = lds + wave * BUF;
  const int n0 = blockIdx.x * (16 * NTW);

  // global load: lane (ld_row, ld_c) of a wave-wide load fetches chunk ld_c (16 bytes) of row
  // ld_row of an 8-row half tile and parks it in LDS at the swizzled chunk position
  const int ld_row = lane >> 3, ld_c = lane & 7;
  const uint8_t* src[NTILE][2];
  int wr_off[2];
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    const int r = h * 8 + ld_row;
    wr_off[h] = r * kStepK + ((ld_c ^ swz128(r)) * kChunk);
#pragma unroll
    for (int t = 0; t < NTW; ++t)
      src[t][h] = p.b + (size_t)min(n0 + t * 16 + r, p.N - 1) * p.ldb + ld_c * kChunk;
#pragma unroll
    for (int t = 0; t < MT; ++t)
      src[NTW + t][h] = p.a + (size_t)min(t * 16 + r, p.M - 1) * p.lda + ld_c * kChunk;
  }
  // LDS->register: lane (r, g) of the 16x16x128 MFMA takes logical chunks 2g, 2g+1 of row r
  const int r16 = lane & 15, g4 = lane >> 4;
  const int rd0 = r16 * kStepK + (((2 * g4) ^ swz128(r16)) * kChunk);
  const int rd1 = r16 * kStepK + (((2 * g4 + 1) ^ swz128(r16)) * kChunk);

  const int k_full = p.K / kStepK;
  const int k_tail = p.K - k_full * kStepK;
  const int my_steps = (k_full > wave) ? (k_full - wave + KW - 1) / KW : 0;  // whole steps this wave owns

  v4f acc[NTW][MT];
#pragma unroll
  for (int t = 0; t < NTW; ++t)
#pragma unroll
    for (int u = 0; u < MT; ++u) acc[t][u] = (v4f){0.f, 0.f, 0.f, 0.f};

  // The lanes that will finish an output quad (one per lane of each 16x16 result) fetch its
  // scales and bias now, so that their latency is not left over at the end of the kernel.
  // Lane layout of a 16x16 result: m = u*16 + lane%16, n = n0 + t*16 + 4*(lane/16) + e.
  static_assert(NTW * MT * 64 <= KW * 64, "one finishing lane per output quad");
  const bool finisher = threadIdx.x < NTW * MT * 64;
  const int fin_tu = threadIdx.x >> 6;
  const int fin_m = (fin_tu % MT) * 16 + (lane & 15);
  const int fin_n = n0 + (fin_tu / MT) * 16 + 4 * (lane >> 4);
  float fin_sa = 0.f, fin_sb[4] = {0.f, 0.f, 0.f, 0.f}, fin_bias[4] = {0.f, 0.f, 0.f, 0.f};
  if (finisher) {
    fin_sa = p.a_scale[min(fin_m, p.M - 1)];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int ne = min(fin_n + e, p.N - 1);
      fin_sb[e] = p.b_scale[ne];
      if (p.bias) fin_bias[e] = bf16_to_f32(p.bias[ne]);
    }
  }

  // DEPTH register sets, one per step in flight
  v4i land[DEPTH][NTILE][2];
  auto fetch = [&](int i, v4i (&dst)[NTILE][2]) {
    const size_t kb = (size_t)(wave + KW * i) * kStepK;
#pragma unroll
    for (int t = 0; t < NTILE; ++t)
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        // B is read once and never again: stream it past the caches; A is shared by everyone
        if (t < NTW) dst[t][h] = __builtin_nontemporal_load((const v4i*)(src[t][h] + kb));
        else dst[t][h] = *(const v4i*)(src[t][h] + kb);
      }
  };
  auto consume = [&](const v4i (&got)[NTILE][2]) {
#pragma unroll
    for (int t = 0; t < NTILE; ++t)
#pragma unroll
      for (int h = 0; h < 2; ++h) *(v4i*)(buf + t * TILE + wr_off[h]) = got[t][h];
    v8i f[NTILE];
#pragma unroll
    for (int t = 0; t < NTILE; ++t) {
      const v4i lo = *(const v4i*)(buf + t * TILE + rd0);
      const v4i hi = *(const v4i*)(buf + t * TILE + rd1);
      f[t] = (v8i){lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
    }
#pragma unroll
    for (int t = 0; t < NTW; ++t)
#pragma unroll
      for (int u = 0; u < MT; ++u)
        acc[t][u] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(f[t], f[NTW + u], acc[t][u], 0, 0, 0, 0, 0, 0);
  };

  // The loop is unrolled DEPTH times so every register set has a fixed name; the compiler's
  // own wait counts then make each consume() wait for exactly its set's loads (they return
  // in issue order, so the younger sets stay in flight). That only works on paths without
  // conditional fetches: where paths with different numbers of younger loads meet, the
  // compiler has to assume the fewest and ends up draining the whole queue once per round.
  // So the rounds in which every consume is followed by a fetch form their own loop, the
  // last full round (consumes only) is straight-line code, and only ragged step counts take
  // the conditional form. (Measured: worth 2 % with four steps in flight; with two steps in
  // flight the drained form is 8-11 % faster, so those configurations keep it.)
  constexpr bool kSteadyLoop = DEPTH >= 4;
  int i = 0;
  if (kSteadyLoop && my_steps >= DEPTH) {
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) fetch(d, land[d]);
    for (; i + 2 * DEPTH <= my_steps; i += DEPTH) {
#pragma unroll
      for (int d = 0; d < DEPTH; ++d) {
        consume(land[d]);
        fetch(i + d + DEPTH, land[d]);
      }
    }
    if (i + DEPTH == my_steps) {
#pragma unroll
      for (int d = 0; d < DEPTH; ++d) consume(land[d]);
      i += DEPTH;
    }
  } else {
#pragma unroll
    for (int d = 0; d < DEPTH; ++d)
      if (d < my_steps) fetch(d, land[d]);
  }
  for (; i < my_steps; i += DEPTH) {
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) {
      if (i + d < my_steps) {
        consume(land[d]);
        if (i + d + DEPTH < my_steps) fetch(i + d + DEPTH, land[d]);
      }
    }
  }
  // K tail (K % 128 != 0): one partial step, taken by the wave whose turn it would be; the
  // lanes fetch their own 16-byte chunks and chunks at or past K count as zero
  if (k_tail && (k_full % KW) == wave) {
    const size_t kb = (size_t)k_full * kStepK;
    const bool in0 = (2 * g4) * kChunk < k_tail, in1 = (2 * g4 + 1) * kChunk < k_tail;
    const v4i z = {0, 0, 0, 0};
    v8i bf[NTW], af[MT];
#pragma unroll
    for (int t = 0; t < NTW; ++t) {
      const uint8_t* row = p.b + (size_t)min(n0 + t * 16 + r16, p.N - 1) * p.ldb + kb;
      const v4i lo = in0 ? *(const v4i*)(row + 2 * g4 * kChunk) : z;
      const v4i hi = in1 ? *(const v4i*)(row + (2 * g4 + 1) * kChunk) : z;
      bf[t] = (v8i){lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
    }
#pragma unroll
    for (int u = 0; u < MT; ++u) {
      const uint8_t* row = p.a + (size_t)min(u * 16 + r16, p.M - 1) * p.lda + kb;
      const v4i lo = in0 ? *(const v4i*)(row + 2 * g4 * kChunk) : z;
      const v4i hi = in1 ? *(const v4i*)(row + (2 * g4 + 1) * kChunk) : z;
      af[u] = (v8i){lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
    }
#pragma unroll
    for (int t = 0; t < NTW; ++t)
#pragma unroll
      for (int u = 0; u < MT; ++u)
        acc[t][u] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(bf[t], af[u], acc[t][u], 0, 0, 0, 0, 0, 0);
  }

  // ---- cross-wave reduction through each wave's own (now idle) buffer
  v4f* mine = (v4f*)buf;
#pragma unroll
  for (int t = 0; t < NTW; ++t)
#pragma unroll
    for (int u = 0; u < MT; ++u) mine[(t * MT + u) * 64 + lane] = acc[t][u];
  __syncthreads();

  if (finisher && fin_m < p.M && fin_n < p.N) {
    v4f sum = ((const v4f*)lds)[fin_tu * 64 + lane];
#pragma unroll
    for (int w = 1; w < KW; ++w) sum += ((const v4f*)(lds + w * BUF))[fin_tu * 64 + lane];
    float r[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      r[e] = sum[e] * fin_sa * fin_sb[e];
      if (p.bias) r[e] += fin_bias[e];
    }
    const uint32_t lo = pack_out_x2(r[0], r[1], p.out_f16), hi = pack_out_x2(r[2], r[3], p.out_f16);
    uint16_t* dst = p.c + (size_t)fin_m * p.ldc + fin_n;
    if (fin_n + 3 < p.N && ((p.ldc & 3) == 0) && ((reinterpret_cast<uintptr_t>(p.c) & 7) == 0)) {
      *(v2u*)dst = (v2u){lo, hi};
    } else {
      dst[0] = (uint16_t)lo;
      if (fin_n + 1 < p.N) dst[1] = (uint16_t)(lo >> 16);
      if (fin_n + 2 < p.N) dst[2] = (uint16_t)hi;
      if (fin_n + 3 < p.N) dst[3] = (uint16_t)(hi >> 16);
    }
  }
}

// ------------------------------------------------------------------------------------
// Persistent skinny kernel for M <= 16*MT (MT = 1, 2) and K = 16*SPW 128-byte steps (K = 2048 ..
// 8192): one workgroup of 16 waves per CU walks a contiguous run of 16-row tiles of B. Wave w
// owns the K steps w, w+16, ... of every tile and keeps its share of A (MT*SPW fragments, 8
// registers each) in registers for the whole launch: A crosses the L2->L1 path once per CU
// instead of once per tile, which is where the one-tile-per-workgroup kernel above loses a
// tenth of its time at M = 16 and a quarter at M = 32. The loads of B run LAG steps ahead of
// their use (a whole tile with one block of A; two steps with two, whose fragments take the
// registers); per tile the waves' partial 16x16 results meet in LDS (two alternating areas, one
// barrier per tile) and one wave per 16x16 result, a different one every time, adds them in
// wave order and stores.
// Workgroup g starts its K walk at step 2*(g/8) (workgroups g, g+8, ... share an XCD): the
// workgroups of an XCD then ask its L2 for different lines of A at any one time, and the
// addresses of B in flight do not all agree in their low bits (measured at N=K=8192, M=16:
// 13.2 -> 12.7 us).
// ------------------------------------------------------------------------------------
constexpr int kPersistWaves = 16;

constexpr size_t persistent_lds_bytes(int MT) { return (size_t)kPersistWaves * 2048 + (size_t)2 * kPersistWaves * MT * 1024; }

// VEC: b_scale, bias and C are aligned for 16-, 8- and 8-byte accesses (else element by element).
template <int SPW, int MT, int LAG, bool VEC>
__global__ __launch_bounds__(kPersistWaves * 64) void gemm_skinny_persistent_kernel(GemmParams p) {
  constexpr int WAVES = kPersistWaves;
  constexpr int STEPS = WAVES * SPW;
  static_assert(LAG >= 1 && LAG <= SPW && SPW % LAG == 0, "the landing registers are a ring of LAG steps");
  fetch_arguments_now(p);
  extern __shared__ __attribute__((aligned(1024))) uint8_t lds[];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  uint8_t* buf = lds + wave * 2048;             // this wave's transpose buffer (one 16 x 128 B step)
  v4f* red = (v4f*)(lds + WAVES * 2048);        // [2][MT][WAVES][64] partial results

  // this workgroup's run of tiles: the first `rem` workgroups take one tile more (quotient and
  // remainder of tiles by workgroups come from the host: the division would sit in front of the
  // first load)
  const int g = blockIdx.x;
  const int q = p.tiles_m, rem = p.tiles_n;
  const int tile0 = g * q + min(g, rem);
  const int count = q + (g < rem ? 1 : 0);
  if (count <= 0) return;

  // byte offset of this wave's i-th K step inside a row; wave-uniform, pinned to scalar registers
  const int base_step = (wave + 2 * (g >> 3)) % STEPS;
  uint32_t kofs[SPW];
#pragma unroll
  for (int i = 0; i < SPW; ++i) {
    int s = base_step + WAVES * i;
    if (s >= STEPS) s -= STEPS;
    kofs[i] = (uint32_t)__builtin_amdgcn_readfirstlane(s * kStepK);
  }
  // a wave-uniform 64-bit offset pinned to scalar registers: loads then take the scalar-base +
  // 32-bit lane-offset form instead of a 64-bit address pair per lane and load
  auto uniform = [](size_t v) -> size_t {
    const uint32_t lo = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)v);
    const uint32_t hi = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(v >> 32));
    return ((size_t)hi << 32) | lo;
  };
  const int r16 = lane & 15, g4 = lane >> 4;
  const int ld_row = lane >> 3, ld_c = lane & 7;
  uint32_t b_lane[2];
  int wr_off[2];
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    const int r = h * 8 + ld_row;
    wr_off[h] = r * kStepK + ((ld_c ^ swz128(r)) * kChunk);
    b_lane[h] = (uint32_t)r * (uint32_t)p.ldb + ld_c * kChunk;
  }
  const int rd0 = r16 * kStepK + (((2 * g4) ^ swz128(r16)) * kChunk);
  const int rd1 = r16 * kStepK + (((2 * g4 + 1) ^ swz128(r16)) * kChunk);

  v4i land[LAG][2];
  const size_t tile_pitch = (size_t)16 * p.ldb;
  size_t cur_tile = uniform((size_t)tile0 * tile_pitch);  // byte offset of the tile being multiplied
  auto fetch = [&](int slot, size_t tile_off, int i) {
    const uint8_t* sbase = p.b + (tile_off + kofs[i]);
#pragma unroll
    for (int h = 0; h < 2; ++h) land[slot][h] = __builtin_nontemporal_load((const v4i*)(sbase + b_lane[h]));
  };
  // The first rows of B are asked for before anything else: they come from HBM.
#pragma unroll
  for (int i = 0; i < LAG; ++i) fetch(i, cur_tile, i);
  __builtin_amdgcn_sched_barrier(0);
  // A: whole-line loads (8 lanes per row, rows past M repeat the last one), turned into the
  // MFMA lane layout through the transpose buffer, once, one 16-row block at a time
  v8i fa[MT][SPW];
#pragma unroll
  for (int u = 0; u < MT; ++u) {
    v4i la[SPW][2];
#pragma unroll
    for (int i = 0; i < SPW; ++i) {
      const uint8_t* sbase = p.a + kofs[i];
#pragma unroll
      for (int h = 0; h < 2; ++h)
        la[i][h] = *(const v4i*)(sbase + ((uint32_t)min(u * 16 + h * 8 + ld_row, p.M - 1) * (uint32_t)p.lda + ld_c * kChunk));
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int i = 0; i < SPW; ++i) {
      *(v4i*)(buf + wr_off[0]) = la[i][0];
      *(v4i*)(buf + wr_off[1]) = la[i][1];
      const v4i lo = *(const v4i*)(buf + rd0);
      const v4i hi = *(const v4i*)(buf + rd1);
      fa[u][i] = (v8i){lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
    }
    __builtin_amdgcn_sched_barrier(0);
  }
  // The 16x16 results are numbered q = MT*j + u (tile j of the run, block u of A); wave w finishes
  // the results q = w, w + 16, ...: lane (m = 16u + lane % 16, quad lane / 16) owns
  // C[m, 16*tile + 4*(lane/16) .. +3]. The column scales and bias of a wave's next result are
  // fetched long before they are used (here, and after each finished result) and kept as loaded;
  // a run without a result for this wave reads the run's last tile instead.
  // Without a bias the same loads read the head of b_scale instead and the bits are masked off:
  // the loads stay unconditional and in the global address space either way.
  const uint16_t* const bias_src = p.bias ? p.bias : reinterpret_cast<const uint16_t*>(p.b_scale);
  const int bias_stride = p.bias ? 1 : 0;
  const uint16_t bias_mask = p.bias ? 0xffffu : 0u;
  float sb_raw[4], fin_sa;
  uint16_t bias_raw[4];
  auto load_epi = [&](int qi) {
    const int qc = min(qi, count * MT - 1);
    const int n = (tile0 + qc / MT) * 16 + 4 * g4;
    fin_sa = p.a_scale[min((qc % MT) * 16 + r16, p.M - 1)];
    if (VEC) {
      const v4f s4 = *(const v4f*)(p.b_scale + n);
      const us4 b4 = *(const us4*)(bias_src + n * bias_stride);
#pragma unroll
      for (int x = 0; x < 4; ++x) sb_raw[x] = s4[x], bias_raw[x] = b4[x];
    } else {
#pragma unroll
      for (int x = 0; x < 4; ++x) sb_raw[x] = p.b_scale[n + x], bias_raw[x] = bias_src[(n + x) * bias_stride];
    }
  };
  load_epi(wave);

  auto consume = [&](int slot, int i, v4f (&acc)[MT]) {
    *(v4i*)(buf + wr_off[0]) = land[slot][0];
    *(v4i*)(buf + wr_off[1]) = land[slot][1];
    const v4i lo = *(const v4i*)(buf + rd0);
    const v4i hi = *(const v4i*)(buf + rd1);
    const v8i fb = (v8i){lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
#pragma unroll
    for (int u = 0; u < MT; ++u)
      acc[u] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(fb, fa[u][i], acc[u], 0, 0, 0, 0, 0, 0);
  };
  auto finish = [&](int j, const v4f (&acc)[MT]) {
    v4f* area = red + (j & 1) * (MT * WAVES * 64);
#pragma unroll
    for (int u = 0; u < MT; ++u) area[(u * WAVES + wave) * 64 + lane] = acc[u];
    __syncthreads();
    // (the area is written again two tiles later, behind the next barrier, which the finishing
    // waves reach only after these reads)
#pragma unroll
    for (int u = 0; u < MT; ++u) {
      if (wave == ((j * MT + u) & (WAVES - 1))) {
        const v4f* part = area + u * WAVES * 64 + lane;
        v4f sum = {0.f, 0.f, 0.f, 0.f};
#pragma unroll 1
        for (int w0 = 0; w0 < WAVES; w0 += 8) {  // eight partials in flight at a time: all sixteen cost 64 registers
#pragma unroll
          for (int w = 0; w < 8; ++w) sum += part[(w0 + w) * 64];
        }
        const int m = u * 16 + r16;
        if (m < p.M) {
          float r[4];
#pragma unroll
          for (int x = 0; x < 4; ++x) r[x] = __builtin_fmaf(sum[x] * fin_sa, sb_raw[x], bf16_to_f32(bias_raw[x] & bias_mask));
          const uint32_t lo = pack_out_x2(r[0], r[1], p.out_f16), hi = pack_out_x2(r[2], r[3], p.out_f16);
          uint16_t* dst = p.c + (size_t)m * p.ldc + (tile0 + j) * 16 + 4 * g4;
          if (VEC) {
            *(v2u*)dst = (v2u){lo, hi};
          } else {
            dst[0] = (uint16_t)lo; dst[1] = (uint16_t)(lo >> 16);
            dst[2] = (uint16_t)hi; dst[3] = (uint16_t)(hi >> 16);
          }
        }
        load_epi(j * MT + u + WAVES);
      }
    }
  };

  int j = 0;
  for (; j + 1 < count; ++j) {
    const size_t next_tile = uniform(cur_tile + tile_pitch);
    v4f acc[MT];
#pragma unroll
    for (int u = 0; u < MT; ++u) acc[u] = (v4f){0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int i = 0; i < SPW; ++i) {
      consume(i % LAG, i, acc);
      if (i + LAG < SPW) fetch(i % LAG, cur_tile, i + LAG);
      else fetch(i % LAG, next_tile, i + LAG - SPW);
    }
    finish(j, acc);
    cur_tile = next_tile;
  }
  {
    v4f acc[MT];
#pragma unroll
    for (int u = 0; u < MT; ++u) acc[u] = (v4f){0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int i = 0; i < SPW; ++i) {
      consume(i % LAG, i, acc);
      if (i + LAG < SPW) fetch(i % LAG, cur_tile, i + LAG);
    }
    finish(j, acc);
  }
}

// ------------------------------------------------------------------------------------
// Narrow-tile kernel: one workgroup per tile of 32*MB rows and 32*NB columns of C (MB, NB = 1, 2)
// owns all of K, so there are no partial sums and no second launch. It is the form for shapes
// that give every CU at most one such tile when A has more rows than the persistent kernel
// above keeps in registers: up to 64 rows on any panel, up to 256 in row blocks.
//
// Eight waves. A K step is 512 bytes: wave w of the first four fetches and multiplies the
// step's w-th 128-byte slab of A (rows of A are L2 hits: a short queue, DA steps ahead), wave
// 4+w fetches the same slab of the tile's rows of B (from HBM, DB steps ahead).
// Loads return to a wave in order: with A and B in one queue every A line would wait behind
// the B lines in front of it and see HBM's latency. Both go straight into LDS stages laid out
// as [slab][row][128 bytes] with the tiled kernel's chunk swizzle; one barrier per step. The
// four partial 32x32 (x MB x NB) results meet in LDS at the end; wave w finishes columns 8w..8w+7
// of every 32-row block.
// What bounds it (measured with the loads taken out of the K loop: M=128, N=K=8192 13.5 instead of
// 21.7 us; M=64, N=4096 8.2 instead of 13.0): the bytes the CUs pull from L2 together, about 17 TB/s
// chip-wide in every form (32 KB per step and CU with 32x32 tiles, 64 KB with 64x64), not the depth of
// either ring and not the order of LDS reads and MFMAs.
// Workgroup g starts its walk over K at step 5g mod steps and wraps around: with a power-of-two
// row pitch the rows in flight at one moment would otherwise agree in their low address bits
// and crowd a few memory channels (measured, M=32, N=K=8192, K loop only: 19.8 -> 13.4 us).
// ------------------------------------------------------------------------------------
constexpr int kNarrowKS = 512;
// NB: 32-column blocks per tile (2: 64-column tiles, for panels of one to two 32-column tiles per CU).
// Steps the loads run ahead of their use: what the 160 KB of LDS allow.
constexpr int narrow_b_dist(int MB, int NB) { return NB == 1 ? 5 : MB == 1 ? 3 : 2; }
// A's stages: a compute wave is the only reader of the slab it fetches, so it refills a stage as soon as
// its own fragment reads of it have returned, in the same step: as many steps ahead as there are stages.
constexpr int narrow_a_dist(int MB, int NB) { return MB == 1 && NB == 1 ? 3 : 2; }
constexpr size_t narrow_lds_bytes(int MB, int NB) {
  return (size_t)narrow_a_dist(MB, NB) * MB * 32 * kNarrowKS + (size_t)(narrow_b_dist(MB, NB) + 1) * NB * 32 * kNarrowKS;
}
static_assert(narrow_lds_bytes(2, 1) <= 160 * 1024 && narrow_lds_bytes(1, 2) <= 160 * 1024 && narrow_lds_bytes(2, 2) <= 160 * 1024,
              "stage rings must fit the LDS");

// waits until at most VM of this wave's global loads are outstanding (LDS operations are not waited for)
template <int VM>
__device__ __forceinline__ void wait_loads() {
  constexpr int imm = (VM & 15) | ((VM >> 4) << 14) | (7 << 4) | (15 << 8);
  __builtin_amdgcn_s_waitcnt(imm);
}

template <int MB, int NB>
__global__ __launch_bounds__(512) void gemm_narrow_kernel(GemmParams p) {
  constexpr int BM = 32 * MB, BN = 32 * NB, KS = kNarrowKS;
  constexpr int DA = narrow_a_dist(MB, NB), DB = narrow_b_dist(MB, NB);
  constexpr int RA = DA, RB = DB + 1;
  constexpr int STA = BM * KS, STB = BN * KS;  // bytes per stage
  constexpr int LA = BM / 8, LB = BN / 8;      // wave-wide loads per wave and step (8 rows x 128 bytes each)
  static_assert((DA - 1) * LA < 64 && (DB - 1) * LB < 64, "outstanding-load counts must fit the wait instruction");
  fetch_arguments_now(p);
  extern __shared__ __attribute__((aligned(1024))) uint8_t lds[];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  // More than BM rows of A: a workgroup per tile and row block. The workgroups of one tile sit next to
  // each other on one XCD (workgroup ids go round the XCDs), so the tile's rows of B come from HBM once
  // and from that XCD's L2 for the others.
  const int row_blocks = (p.M + BM - 1) / BM;
  // Columns of C a tile owns: BN, or fewer where that deals the columns out evenly over the CUs (the host's
  // choice, a multiple of 4). Rows of B past them lie outside the tile's descriptor and read as zeros without
  // a memory access; their products are computed and not stored.
  const int tile_cols = p.tiles_n;
  int tile = blockIdx.x, row_block = 0;
  if (row_blocks > 1) {
    const int slot = blockIdx.x / kNumXcd;
    row_block = slot % row_blocks;
    tile = (slot / row_blocks) * kNumXcd + (blockIdx.x % kNumXcd);
    if (tile * tile_cols >= p.N) return;  // (the grid is rounded up to whole rounds of the XCDs)
  }
  const int n0 = tile * tile_cols, m0 = row_block * BM;
  const int n_end = min(n0 + tile_cols, p.N);
  const int ksteps = (p.K + KS - 1) / KS;  // the last step may be partial (K is a multiple of 16)
  const int rot = (int)(((unsigned)tile * 5u) % (unsigned)ksteps);
  // a lane's 16 bytes of an 8-row group: row lane/8; LDS position lane%8 holds logical chunk
  // position ^ key(row), key = (row >> 1) & 7: for the even groups of a slab that is ld_row >> 1, for
  // the odd ones 4 more, which flips bit 6 of the byte offset
  const int ld_row = lane >> 3, ld_pc = lane & 7;
  const uint32_t chunk_even = (uint32_t)((ld_pc ^ (ld_row >> 1)) * kChunk);
  auto step_of = [&](int s) { const int t = s + rot; return t >= ksteps ? t - ksteps : t; };
  // A lane whose 16 bytes lie at or past K (only in the last step of a K that is not a multiple of 512)
  // asks for an offset outside every descriptor instead: zeros arrive, and the load still counts.
  constexpr uint32_t kOutside = 0x80000000u;
  auto lane_part = [&](uint32_t inside, uint32_t chunk, uint32_t k_slab) { return k_slab + chunk < (uint32_t)p.K ? inside : kOutside; };

  if (wave < 4) {
    // ---- compute wave: slab `wave` of every step
    const __amdgpu_buffer_rsrc_t ra = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint8_t*>(p.a) + (size_t)m0 * p.lda, 0, (int)((uint32_t)min(p.M - m0, BM) * (uint32_t)p.lda), 0x00020000);
    const uint32_t a_even = (uint32_t)ld_row * (uint32_t)p.lda + chunk_even;
    const uint32_t a_odd = (uint32_t)ld_row * (uint32_t)p.lda + (chunk_even ^ 64u);
    auto issue_a = [&](int s) {
      if (s >= ksteps) return;
      uint8_t* dst = lds + (s % RA) * STA + wave * (BM * kStepK);
      const uint32_t koff = (uint32_t)step_of(s) * KS + (uint32_t)wave * kStepK;
      const uint32_t even = lane_part(a_even, chunk_even, koff), odd = lane_part(a_odd, chunk_even ^ 64u, koff);
#pragma unroll
      for (int g = 0; g < LA; ++g)
        load_chunk_to_lds<false>(ra, dst + g * 1024, (g & 1) ? odd : even, (uint32_t)(g * 8) * (uint32_t)p.lda + koff);
    };
    // this lane's scales and bias, asked for before the loop: row l32 of every 32-row block, columns
    // n0 + 32*jb + 8*wave + 4*half .. +3 of every 32-column block (indices clamped; what lies past an
    // edge is never stored)
    const int l32 = lane & 31, half = lane >> 5;
    const int nq = n0 + 8 * wave + 4 * half;
    float sa[MB], sb[NB][4], bias_f[NB][4];
#pragma unroll
    for (int i = 0; i < MB; ++i) sa[i] = p.a_scale[min(m0 + i * 32 + l32, p.M - 1)];
#pragma unroll
    for (int jb = 0; jb < NB; ++jb)
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int ne = min(nq + 32 * jb + e, p.N - 1);
        sb[jb][e] = p.b_scale[ne];
        bias_f[jb][e] = p.bias ? bf16_to_f32(p.bias[ne]) : 0.0f;
      }
#pragma unroll
    for (int s = 0; s < DA; ++s) issue_a(s);
    if (ksteps > DA) wait_loads<(DA - 1) * LA>(); else wait_loads<0>();
    __builtin_amdgcn_s_barrier();

    v16f acc[MB][NB];
    const v16f zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int i = 0; i < MB; ++i)
#pragma unroll
      for (int jb = 0; jb < NB; ++jb) acc[i][jb] = zero;
    // fragment of K half sh (64 bytes) of this wave's slab: logical chunks 4*half + 2*sh + {0, 1} of row l32
    int rd[2][2];
#pragma unroll
    for (int sh = 0; sh < 2; ++sh)
#pragma unroll
      for (int j = 0; j < 2; ++j) rd[sh][j] = l32 * kStepK + (((4 * half + 2 * sh + j) ^ swz128(l32)) * kChunk);

    // The two K halves of a step are read and multiplied out of phase: while the MFMAs of one half
    // run, the fragment reads of the next are under way (the second half of the same step, or, past
    // the step's barrier, the first half of the next step), so neither the LDS reads nor the MFMAs
    // of the one wave a SIMD has here wait for the other.
    auto read_half = [&](int s, int sh, v4i (&fbh)[NB][2], v4i (&fah)[MB][2]) {
      const uint8_t* sa_rows = lds + (s % RA) * STA + wave * (BM * kStepK);
      const uint8_t* sb_rows = lds + RA * STA + (s % RB) * STB + wave * (BN * kStepK);
#pragma unroll
      for (int jb = 0; jb < NB; ++jb)
#pragma unroll
        for (int j = 0; j < 2; ++j) fbh[jb][j] = *(const v4i*)(sb_rows + jb * 32 * kStepK + rd[sh][j]);
#pragma unroll
      for (int i = 0; i < MB; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) fah[i][j] = *(const v4i*)(sa_rows + i * 32 * kStepK + rd[sh][j]);
    };
    auto mfma_half = [&](const v4i (&fbh)[NB][2], const v4i (&fah)[MB][2]) {
#pragma unroll
      for (int jb = 0; jb < NB; ++jb) {
        const v8i vb = (v8i){fbh[jb][0][0], fbh[jb][0][1], fbh[jb][0][2], fbh[jb][0][3],
                             fbh[jb][1][0], fbh[jb][1][1], fbh[jb][1][2], fbh[jb][1][3]};
#pragma unroll
        for (int i = 0; i < MB; ++i) {
          const v8i va = (v8i){fah[i][0][0], fah[i][0][1], fah[i][0][2], fah[i][0][3],
                               fah[i][1][0], fah[i][1][1], fah[i][1][2], fah[i][1][3]};
          acc[i][jb] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(vb, va, acc[i][jb], 0, 0, 0, 0, 0, 0);
        }
      }
    };
    v4i fb0[NB][2], fa0[MB][2], fb1[NB][2], fa1[MB][2];
    read_half(0, 0, fb0, fa0);
    for (int s = 0; s < ksteps; ++s) {
      read_half(s, 1, fb1, fa1);
      __builtin_amdgcn_sched_barrier(0);
      mfma_half(fb0, fa0);
      // every fragment of the step is in registers: this wave's slab of the A stage is free again, and
      // the loads of step s + DA go into it (nobody else reads or writes that slab)
      __builtin_amdgcn_sched_barrier(0);
      __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0): the LDS reads above have returned
      issue_a(s + DA);
      // own loads of A(s+1) have landed (the younger A(s+2) .. A(s+DA) may be in flight); past the barrier
      // everyone's have, B's included, and every wave is done reading this step's stages
      if (s + DA < ksteps) wait_loads<(DA - 1) * LA>(); else wait_loads<0>();
      __builtin_amdgcn_s_barrier();
      if (s + 1 < ksteps) read_half(s + 1, 0, fb0, fa0);
      __builtin_amdgcn_sched_barrier(0);
      mfma_half(fb1, fa1);
      __builtin_amdgcn_sched_barrier(0);
    }

    // ---- the four waves' partial results meet in LDS (the stages are free: last barrier passed)
    v4f* area = (v4f*)lds;  // [wave][32x32 block][q][lane]
#pragma unroll
    for (int i = 0; i < MB; ++i)
#pragma unroll
      for (int jb = 0; jb < NB; ++jb)
#pragma unroll
        for (int q = 0; q < 4; ++q)
          area[(((wave * MB + i) * NB + jb) * 4 + q) * 64 + lane] =
              (v4f){acc[i][jb][4 * q], acc[i][jb][4 * q + 1], acc[i][jb][4 * q + 2], acc[i][jb][4 * q + 3]};
    __syncthreads();
    const bool vec = ((p.ldc & 3) == 0) && ((reinterpret_cast<uintptr_t>(p.c) & 7) == 0);
#pragma unroll
    for (int i = 0; i < MB; ++i) {
#pragma unroll
      for (int jb = 0; jb < NB; ++jb) {
        v4f sum = area[(((0 * MB + i) * NB + jb) * 4 + wave) * 64 + lane];
#pragma unroll
        for (int w = 1; w < 4; ++w) sum += area[(((w * MB + i) * NB + jb) * 4 + wave) * 64 + lane];
        const int m = m0 + i * 32 + l32, n = nq + 32 * jb;
        if (m < p.M && n < n_end) {
          float r[4];
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const float t = sum[e] * sa[i];
            r[e] = p.bias ? __builtin_fmaf(t, sb[jb][e], bias_f[jb][e]) : t * sb[jb][e];
          }
          const uint32_t lo = pack_out_x2(r[0], r[1], p.out_f16), hi = pack_out_x2(r[2], r[3], p.out_f16);
          uint16_t* dst = p.c + (size_t)m * p.ldc + n;
          if (vec && n + 3 < n_end) {
            *(v2u*)dst = (v2u){lo, hi};
          } else {
            dst[0] = (uint16_t)lo;
            if (n + 1 < n_end) dst[1] = (uint16_t)(lo >> 16);
            if (n + 2 < n_end) dst[2] = (uint16_t)hi;
            if (n + 3 < n_end) dst[3] = (uint16_t)(hi >> 16);
          }
        }
      }
    }
  } else {
    // ---- loader wave for B: slab `wave - 4` of every step, 8 rows per load
    const int w = wave - 4;
    const __amdgpu_buffer_rsrc_t rb = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint8_t*>(p.b) + (size_t)n0 * p.ldb, 0, (int)((uint32_t)(n_end - n0) * (uint32_t)p.ldb), 0x00020000);
    const uint32_t b_even = (uint32_t)ld_row * (uint32_t)p.ldb + chunk_even;
    const uint32_t b_odd = (uint32_t)ld_row * (uint32_t)p.ldb + (chunk_even ^ 64u);
    auto issue_b = [&](int s) {
      if (s >= ksteps) return;
      uint8_t* dst = lds + RA * STA + (s % RB) * STB + w * (BN * kStepK);
      const uint32_t koff = (uint32_t)step_of(s) * KS + (uint32_t)w * kStepK;
      const uint32_t even = lane_part(b_even, chunk_even, koff), odd = lane_part(b_odd, chunk_even ^ 64u, koff);
#pragma unroll
      for (int g = 0; g < LB; ++g)
        load_chunk_to_lds<true>(rb, dst + g * 1024, (g & 1) ? odd : even, (uint32_t)(g * 8) * (uint32_t)p.ldb + koff);
    };
#pragma unroll
    for (int s = 0; s < DB; ++s) issue_b(s);
    if (ksteps > DB) wait_loads<(DB - 1) * LB>(); else wait_loads<0>();
    __builtin_amdgcn_s_barrier();
    for (int s = 0; s < ksteps; ++s) {
      issue_b(s + DB);
      if (s + DB < ksteps) wait_loads<(DB - 1) * LB>(); else wait_loads<0>();
      __builtin_amdgcn_s_barrier();
    }
    __syncthreads();  // the compute waves' hand-over of their partial results
  }
}

// ------------------------------------------------------------------------------------
// Pair kernel: M <= 16, N a multiple of 16 up to 8192 (at most two 16-row tiles of B per CU),
// K up to 8192 (any multiple of 16). The decode shapes proper: the whole launch is one or two
// tiles per workgroup, so there is no steady state to reach and what counts is the order in
// which the requests leave the CU.
//
// One workgroup of 16 waves per CU; wave w owns the K steps w, w+16, ... (SPW of them, those past
// K read as zeros) as in the persistent kernel above. Differences:
//  * A is not kept in registers: each wave copies its SPW-1 first steps of A straight from memory
//    into LDS, already in the order the MFMA lanes read them, and reads a step's fragment from there
//    when it multiplies; only its last step goes through the transpose buffer into registers (LDS:
//    3 x 32 KB of A at SPW = 4, 32 KB of transpose buffers, 32 KB of partial results).
//  * A tile's loads of B leave in one burst: step 0 of the first tile first, then A, then the rest
//    of the first tile together with step 0 of the second; the rest of the second tile follows the
//    first tile's reduction. A tile is 16 rows x K contiguous bytes, so a burst asks for one
//    contiguous region, and at no time is more than one tile per CU in flight: measured cold at
//    M=16, N=K=8192, this order 12.9 us against 13.4 us for the persistent kernel's rolling
//    prefetch (four steps per wave in flight all the time) and 13.9 us for the same rolling
//    prefetch with A in LDS; K = 4096 8.0 against 8.6 us, K = 2048 5.3 against 5.9, N = 4096 9.0
//    against 9.5, M = 1 12.2 against 12.6. Everything requested at once (both tiles) takes 14.9 us.
// All loads of B are range-checked buffer loads: a lane whose 16 bytes lie past K, and every lane of
// a tile that does not exist, asks for an offset outside the descriptor and gets zeros without a
// memory access, so the instruction stream is the same for every wave and the wait counts are exact.
// ------------------------------------------------------------------------------------
constexpr size_t pair_lds_bytes(int SPW) {
  return (size_t)kPersistWaves * 2048 * SPW + (size_t)2 * kPersistWaves * 1024;
}

// KTAIL: K is no multiple of 2048, so some waves own steps that lie (partly) past K and their lanes need a
// predicate per load; HAS_BIAS: a bias vector is added. Both are compile-time properties: this kernel's
// time hangs on how fast a wave gets its burst of loads out, and the few vector instructions either adds
// in front of the loads measured 0.3 and 0.1 us at M=16, N=K=8192.
template <int SPW, bool VEC, bool KTAIL, bool HAS_BIAS>
__global__ __launch_bounds__(kPersistWaves * 64) void gemm_skinny_pair_kernel(GemmParams p) {
  constexpr int WAVES = kPersistWaves;
  constexpr int STEPS = WAVES * SPW;
  constexpr int A_LDS = SPW - 1;  // steps of A per wave that live in LDS
  fetch_arguments_now(p);
  extern __shared__ __attribute__((aligned(1024))) uint8_t lds[];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  uint8_t* a_mine = lds + wave * (A_LDS * 2048);             // this wave's steps of A
  uint8_t* buf = lds + WAVES * A_LDS * 2048 + wave * 2048;   // this wave's transpose buffer (one 16 x 128 B step)
  v4f* red = (v4f*)(lds + WAVES * SPW * 2048);               // [2][WAVES][64] partial results

  // this workgroup's one or two tiles (quotient and remainder of tiles by workgroups come from the host)
  const int g = blockIdx.x;
  const int tile0 = g * p.tiles_m + min(g, p.tiles_n);
  const int count = p.tiles_m + (g < p.tiles_n ? 1 : 0);
  if (count <= 0) return;

  // byte offset of this wave's i-th K step inside a row; workgroups of one XCD start at different steps
  const int base_step = (wave + 2 * (g >> 3)) % STEPS;
  uint32_t kofs[SPW];
#pragma unroll
  for (int i = 0; i < SPW; ++i) {
    int s = base_step + WAVES * i;
    if (s >= STEPS) s -= STEPS;
    kofs[i] = (uint32_t)__builtin_amdgcn_readfirstlane(s * kStepK);
  }
  const int r16 = lane & 15, g4 = lane >> 4;
  const int ld_row = lane >> 3, ld_c = lane & 7;
  constexpr uint32_t kOutside = 0x80000000u;  // past every extent (the host keeps extents below 2^31)
  uint32_t b_lane[2], a_lane[2];
  int wr_off[2];
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    const int r = h * 8 + ld_row;
    wr_off[h] = r * kStepK + ((ld_c ^ swz128(r)) * kChunk);
    b_lane[h] = (uint32_t)r * (uint32_t)p.ldb + ld_c * kChunk;
    // the direct-to-LDS copy puts lane l at position l of a 1 KB half step (8 rows x 128 bytes): the lane
    // asks for the chunk whose swizzled place that is; rows past M repeat the last one
    a_lane[h] = (uint32_t)min(r, p.M - 1) * (uint32_t)p.lda + (uint32_t)((ld_c ^ swz128(r)) * kChunk);
  }
  // the lane's chunk of a step lies inside K? (only the last step of a K that is no multiple of 128 cuts lanes off)
  auto in_k = [&](uint32_t step_off, int chunk) { return !KTAIL || step_off + (uint32_t)(chunk * kChunk) < (uint32_t)p.K; };
  const int rd0 = r16 * kStepK + (((2 * g4) ^ swz128(r16)) * kChunk);
  const int rd1 = r16 * kStepK + (((2 * g4 + 1) ^ swz128(r16)) * kChunk);

  const uint32_t tile_pitch = 16u * (uint32_t)p.ldb;
  const uintptr_t bb = reinterpret_cast<uintptr_t>(p.b) + (size_t)tile0 * tile_pitch;
  const uint8_t* b_base = reinterpret_cast<const uint8_t*>(
      ((uintptr_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(bb >> 32)) << 32) |
      (uintptr_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)bb));
  const __amdgpu_buffer_rsrc_t rb = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<uint8_t*>(b_base), 0, (int)((uint32_t)count * tile_pitch), 0x00020000);
  const __amdgpu_buffer_rsrc_t ra = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<uint8_t*>(p.a), 0, (int)((uint32_t)p.M * (uint32_t)p.lda), 0x00020000);

  v4i land[2][SPW][2];
  auto fetch = [&](int t, int i) {
    const uint32_t so = (uint32_t)t * tile_pitch + kofs[i];
    const bool ok = t < count && in_k(kofs[i], ld_c);
#pragma unroll
    for (int h = 0; h < 2; ++h) {
#if defined(__HIP_DEVICE_COMPILE__)
      land[t][i][h] = __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(rb, (int)(ok ? b_lane[h] : kOutside), (int)so, 2));
#else
      land[t][i][h] = (v4i){0, 0, 0, 0};
#endif
    }
  };
  fetch(0, 0);  // the first rows of B are asked for before anything else: they come from HBM
  __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int i = 0; i < SPW; ++i) {
    uint8_t* dst = i < A_LDS ? a_mine + i * 2048 : buf;
    // (the chunk a lane fetches for LDS position ld_c of row r is ld_c ^ swz128(r))
#pragma unroll
    for (int h = 0; h < 2; ++h)
      load_chunk_to_lds<false>(ra, dst + h * 1024, in_k(kofs[i], ld_c ^ swz128(h * 8 + ld_row)) ? a_lane[h] : kOutside, kofs[i]);
  }
  __builtin_amdgcn_sched_barrier(0);
  // Wave j finishes tile j: lane (m = lane % 16, quad lane / 16) owns C[m, 16*tile + 4*(lane/16) .. +3] (waves
  // without a result read the run's last tile and drop it). Its scales and bias come from memory nobody has
  // touched yet, so they are asked for here, while the wave waits for A anyway - but the wait below must not
  // include them (it holds the burst back: 0.3 us at M=16, N=K=8192), so it has to know how many load
  // instructions they are. With aligned vectors that is exact: one buffer load each through descriptors of
  // their own (nothing the compiler could merge or split). The unaligned form asks behind the burst instead.
  const int fin_n = (tile0 + min(wave, count - 1)) * 16 + 4 * g4;
  float fin_sa = 0.f, sb_raw[4] = {0.f, 0.f, 0.f, 0.f};
  uint16_t bias_raw[4] = {0, 0, 0, 0};
  if constexpr (VEC) {
#if defined(__HIP_DEVICE_COMPILE__)
    const __amdgpu_buffer_rsrc_t rsa = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(p.a_scale), 0, p.M * 4, 0x00020000);
    const __amdgpu_buffer_rsrc_t rsb = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(p.b_scale), 0, p.N * 4, 0x00020000);
    fin_sa = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rsa, min(r16, p.M - 1) * 4, 0, 0));
    const v4f s4 = load_f32x4_checked(rsb, (uint32_t)fin_n * 4u);
#pragma unroll
    for (int x = 0; x < 4; ++x) sb_raw[x] = s4[x];
    if (HAS_BIAS) {
      const __amdgpu_buffer_rsrc_t rbias = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint16_t*>(p.bias), 0, p.N * 2, 0x00020000);
      const us4 b4 = load_u16x4_checked(rbias, (uint32_t)fin_n * 2u);
#pragma unroll
      for (int x = 0; x < 4; ++x) bias_raw[x] = b4[x];
    }
#endif
    __builtin_amdgcn_sched_barrier(0);
    // A has landed once everything in front of those two or three loads has (loads return in order)
    wait_loads<2 + (HAS_BIAS ? 1 : 0)>();
  } else {
    wait_loads<0>();
  }
  v8i fa_last;
  {
    const v4i lo = *(const v4i*)(buf + rd0);
    const v4i hi = *(const v4i*)(buf + rd1);
    fa_last = (v8i){lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
    __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0): in registers before the buffer is written again
  }
  __builtin_amdgcn_sched_barrier(0);

  auto consume = [&](int t, int i, v4f& acc) {
    *(v4i*)(buf + wr_off[0]) = land[t][i][0];
    *(v4i*)(buf + wr_off[1]) = land[t][i][1];
    const v4i lo = *(const v4i*)(buf + rd0);
    const v4i hi = *(const v4i*)(buf + rd1);
    const v8i fb = (v8i){lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
    v8i fa = fa_last;
    if (i < A_LDS) {
      const v4i alo = *(const v4i*)(a_mine + i * 2048 + rd0);
      const v4i ahi = *(const v4i*)(a_mine + i * 2048 + rd1);
      fa = (v8i){alo[0], alo[1], alo[2], alo[3], ahi[0], ahi[1], ahi[2], ahi[3]};
    }
    acc = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(fb, fa, acc, 0, 0, 0, 0, 0, 0);
  };
  // tile 0: the rest of its loads in one burst, the first step of tile 1 behind them
#pragma unroll
  for (int i = 1; i < SPW; ++i) fetch(0, i);
  fetch(1, 0);
  __builtin_amdgcn_sched_barrier(0);
  if constexpr (!VEC) {  // (element by element: a count the compiler may change, so behind the burst)
    fin_sa = p.a_scale[min(r16, p.M - 1)];
#pragma unroll
    for (int x = 0; x < 4; ++x) {
      sb_raw[x] = p.b_scale[fin_n + x];
      if (HAS_BIAS) bias_raw[x] = p.bias[fin_n + x];
    }
  }
  __builtin_amdgcn_sched_barrier(0);
  // the 16 partial results of tile j meet in LDS (one area per tile); wave j adds them in wave order and stores
  auto finish = [&](int j, const v4f& acc) {
    v4f* area = red + j * (WAVES * 64);
    area[wave * 64 + lane] = acc;
    __syncthreads();
    if (wave == j) {
      const v4f* part = area + lane;
      v4f sum = {0.f, 0.f, 0.f, 0.f};
#pragma unroll 1
      for (int w0 = 0; w0 < WAVES; w0 += 8) {  // eight partials in flight at a time
#pragma unroll
        for (int w = 0; w < 8; ++w) sum += part[(w0 + w) * 64];
      }
      if (r16 < p.M) {
        float r[4];
#pragma unroll
        for (int x = 0; x < 4; ++x)
          r[x] = HAS_BIAS ? __builtin_fmaf(sum[x] * fin_sa, sb_raw[x], bf16_to_f32(bias_raw[x])) : sum[x] * fin_sa * sb_raw[x];
        const uint32_t lo = pack_out_x2(r[0], r[1], p.out_f16), hi = pack_out_x2(r[2], r[3], p.out_f16);
        uint16_t* dst = p.c + (size_t)r16 * p.ldc + (tile0 + j) * 16 + 4 * g4;
        if (VEC) {
          *(v2u*)dst = (v2u){lo, hi};
        } else {
          dst[0] = (uint16_t)lo; dst[1] = (uint16_t)(lo >> 16);
          dst[2] = (uint16_t)hi; dst[3] = (uint16_t)(hi >> 16);
        }
      }
    }
  };

  v4f acc0 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int i = 0; i < SPW; ++i) consume(0, i, acc0);
  __builtin_amdgcn_sched_barrier(0);
  finish(0, acc0);
  __builtin_amdgcn_sched_barrier(0);
  // tile 1 (loads that ask for nothing when there is none: the instruction stream stays the same)
#pragma unroll
  for (int i = 1; i < SPW; ++i) fetch(1, i);
  __builtin_amdgcn_sched_barrier(0);
  if (count > 1) {
    v4f acc1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int i = 0; i < SPW; ++i) consume(1, i, acc1);
    finish(1, acc1);
  }
}

// ------------------------------------------------------------------------------------
// Row-wise quantiser: one workgroup per row, two passes over the row (amax, then scale
// and convert). e4m3fn encoding is done with integer arithmetic so the rounding
// (nearest, ties to even, subnormals below 2^-6) does not depend on conversion hardware.
// ------------------------------------------------------------------------------------
__device__ __forceinline__ uint8_t f32_to_e4m3fn_rne(float f) {
  const uint32_t u = __float_as_uint(f);
  const uint32_t sign = (u >> 24) & 0x80u;
  const uint32_t mag = u & 0x7fffffffu;
  if (mag > 0x7f800000u) return (uint8_t)(sign | 0x7fu);  // NaN
  if (mag >= 0x43e80000u) {                                // |f| >= 464: beyond the last finite code
    return (uint8_t)(sign | (mag == 0x43e80000u ? 0x7eu : 0x7fu));
  }
  if (mag < 0x3c800000u) {  // |f| < 2^-6: subnormal target, spacing 2^-9
    const float scaled = __uint_as_float(mag) * 512.0f;  // exact
    const float rounded = __builtin_rintf(scaled);       // ties to even
    return (uint8_t)(sign | (uint32_t)rounded);          // 8 -> 0x08 = 2^-6, the first normal
  }
  // normal: keep 3 mantissa bits, round to nearest even on the 20 dropped bits
  uint32_t v = mag + 0x7ffffu + ((mag >> 20) & 1u);
  v >>= 20;                                // exponent(8) | mantissa(3)
  v -= (uint32_t)(127 - 7) << 3;           // rebias
  return (uint8_t)(sign | v);
}

template <typename SrcT>
struct SrcTraits;
// fp32 source: every step rounds to fp32 once, as the eager PyTorch program does.
template <>
struct SrcTraits<float> {
  static __device__ __forceinline__ float load(const float* p) { return *p; }
  static __device__ __forceinline__ float round(float v) { return v; }
};
// bf16 source: PyTorch evaluates each elementwise op in fp32 and rounds its result back to
// bf16, so amax, the scale, the scaled value and the inverse scale each pass through bf16.
template <>
struct SrcTraits<uint16_t> {
  static __device__ __forceinline__ float load(const uint16_t* p) { return bf16_to_f32(*p); }
  static __device__ __forceinline__ float round(float v) { return bf16_to_f32(f32_to_bf16_rne(v)); }
};

// max(a, b) that returns NaN when either operand is NaN (torch.max does; fmaxf drops the NaN).
// One gfx950 instruction (v_maximum3_f32).
__device__ __forceinline__ float max_keep_nan(float a, float b) { return __builtin_elementwise_maximum(a, b); }

// The row's quantisation scale from its absolute maximum, as eager PyTorch computes it:
// `448.0 / clamp(amax, 1e-12)` evaluates as reciprocal * 448, and clamp keeps a NaN (so a row
// holding a NaN gets a NaN scale, a row holding an infinity the scale 0).
template <typename SrcT>
__device__ __forceinline__ float row_scale(float amax) {
  using T = SrcTraits<SrcT>;
  const float floor_ = T::round(1e-12f);
  const float clamped = amax < floor_ ? floor_ : amax;  // false for NaN: it stays
  const float recip = T::round(1.0f / clamped);
  return T::round(recip * 448.0f);
}

// One element the way the PyTorch program treats it, NaN included: scale, clamp to +-448 (a NaN
// passes the clamp), round to e4m3fn with the integer encoder (NaN -> 0x7f with the sign kept).
template <typename SrcT>
__device__ __forceinline__ uint8_t quantize_one(float x, float scale) {
  using T = SrcTraits<SrcT>;
  float v = T::round(x * scale);
  v = v < -448.0f ? -448.0f : v;
  v = v > 448.0f ? 448.0f : v;
  return f32_to_e4m3fn_rne(v);
}

template <typename SrcT>
__global__ __launch_bounds__(256) void quantize_rows_kernel(const SrcT* x, uint8_t* xq,
                                                            float* inv_scale, int K, long ldx,
                                                            long ldq) {
  using T = SrcTraits<SrcT>;
  __shared__ float wave_max[4];
  const long row = blockIdx.x;
  const SrcT* xr = x + row * ldx;
  uint8_t* qr = xq + row * ldq;

  float amax = 0.0f;
  for (int k = threadIdx.x; k < K; k += 256) amax = max_keep_nan(amax, fabsf(T::load(xr + k)));
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) amax = max_keep_nan(amax, __shfl_xor(amax, o));
  if ((threadIdx.x & 63) == 0) wave_max[threadIdx.x >> 6] = amax;
  __syncthreads();
  amax = max_keep_nan(max_keep_nan(wave_max[0], wave_max[1]), max_keep_nan(wave_max[2], wave_max[3]));

  const float scale = row_scale<SrcT>(amax);
  if (threadIdx.x == 0) inv_scale[row] = T::round(1.0f / scale);
  for (int k = threadIdx.x; k < K; k += 256) qr[k] = quantize_one<SrcT>(T::load(xr + k), scale);
}

// Vector form of the quantiser for 16-byte aligned rows: one workgroup per row, every lane
// moves 16 source bytes per load (a wave-wide load covers whole lines). The first CACHE
// chunks a lane reads stay in registers between the amax pass and the convert pass, so rows
// of up to THREADS*CACHE chunks are read from memory once; the rest of a longer row is read
// again (from cache). The e4m3fn rounding is done by the gfx950 pack-convert instruction
// (OCP format, round to nearest even) on values already clamped to +-448.
template <typename SrcT>
struct VecTraits;
template <>
struct VecTraits<float> {
  static constexpr int EPV = 4;  // elements per 16-byte chunk
  static __device__ __forceinline__ void unpack(const v4i& c, float (&f)[4]) {
#pragma unroll
    for (int e = 0; e < 4; ++e) f[e] = __int_as_float(c[e]);
  }
};
template <>
struct VecTraits<uint16_t> {
  static constexpr int EPV = 8;
  static __device__ __forceinline__ void unpack(const v4i& c, float (&f)[8]) {
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      f[2 * e] = __uint_as_float((uint32_t)c[e] << 16);
      f[2 * e + 1] = __uint_as_float((uint32_t)c[e] & 0xffff0000u);
    }
  }
};

// THREADS lanes per row, ROWS rows per workgroup. Rows short enough for one wave's registers take
// THREADS = 64 with several rows per workgroup: no LDS, no barrier, and a fraction of the workgroups
// (short rows are bound by the rate at which workgroups start, about one per 1.2-2 ns).
template <typename SrcT, int CACHE, int THREADS, int ROWS = 1>
__global__ __launch_bounds__(THREADS* ROWS) void quantize_rows_vec_kernel(const SrcT* x, uint8_t* xq,
                                                                        float* inv_scale, int K, long ldx,
                                                                        long ldq, long rows) {
  static_assert(ROWS == 1 || THREADS == 64, "several rows per workgroup: one wave each");
  using T = SrcTraits<SrcT>;
  using V = VecTraits<SrcT>;
  constexpr int EPV = V::EPV;
  __shared__ float wave_max[THREADS / 64];
  const long row = (long)blockIdx.x * ROWS + (ROWS > 1 ? (long)(threadIdx.x >> 6) : 0);
  if (ROWS > 1 && row >= rows) return;  // (whole waves; this form has no barrier)
  const v4i* xr = (const v4i*)(x + row * ldx);
  uint8_t* qr = xq + row * ldq;
  const int nchunks = K / EPV;
  const int tid = ROWS > 1 ? (int)(threadIdx.x & 63) : (int)threadIdx.x;

  v4i cache[CACHE];
  float amax = 0.0f;
  auto fold = [&](const v4i& c) {
    float f[EPV];
    V::unpack(c, f);
#pragma unroll
    for (int e = 0; e < EPV; ++e) amax = max_keep_nan(amax, fabsf(f[e]));
  };
#pragma unroll
  for (int i = 0; i < CACHE; ++i) {
    // past the row's end a lane re-reads the last chunk: harmless for the maximum, never
    // stored, and it keeps the loads free of branches
    cache[i] = __builtin_nontemporal_load(xr + min(tid + THREADS * i, nchunks - 1));
  }
#pragma unroll
  for (int i = 0; i < CACHE; ++i) fold(cache[i]);
  for (int c = tid + THREADS * CACHE; c < nchunks; c += THREADS) fold(xr[c]);
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) amax = max_keep_nan(amax, __shfl_xor(amax, o));
  if (THREADS > 64) {
    if ((tid & 63) == 0) wave_max[tid >> 6] = amax;
    __syncthreads();
#pragma unroll
    for (int w = 0; w < THREADS / 64; ++w) amax = max_keep_nan(amax, wave_max[w]);
  }

  const float scale = row_scale<SrcT>(amax);
  if (tid == 0) inv_scale[row] = T::round(1.0f / scale);
  // A row that holds a NaN or an infinity (the whole workgroup sees the same amax) takes the
  // element-by-element route, whose clamp and encoder carry NaN through as PyTorch does; the
  // pack-convert route below is for finite rows.
  if (!(amax < __builtin_inff())) {
    const SrcT* xs = x + row * ldx;
    for (int k = tid; k < K; k += THREADS) qr[k] = quantize_one<SrcT>(T::load(xs + k), scale);
    return;
  }

  auto convert = [&](const v4i& src, uint32_t (&out)[EPV / 4]) {
    float f[EPV];
    V::unpack(src, f);
#pragma unroll
    for (int e = 0; e < EPV; ++e) f[e] = fminf(fmaxf(T::round(f[e] * scale), -448.0f), 448.0f);
#pragma unroll
    for (int w = 0; w < EPV / 4; ++w) {
      int packed = __builtin_amdgcn_cvt_pk_fp8_f32(f[4 * w], f[4 * w + 1], 0, false);
      packed = __builtin_amdgcn_cvt_pk_fp8_f32(f[4 * w + 2], f[4 * w + 3], packed, true);
      out[w] = (uint32_t)packed;
    }
  };
  auto convert_store = [&](const v4i& src, int c) {
    uint32_t out[EPV / 4];
    convert(src, out);
    if (EPV == 4) *(uint32_t*)(qr + (size_t)c * 4) = out[0];
    else *(v2u*)(qr + (size_t)c * 8) = (v2u){out[0], out[EPV / 4 - 1]};
  };
  // A chunk turns into EPV output bytes per lane (4 or 8): too little per store instruction.
  // BATCH = 16 / EPV consecutive rounds of the cached chunks are therefore gathered through
  // a wave-private LDS strip (LDS executes a wave's operations in order: no barrier) and
  // leave as one 16-byte store per lane, BATCH runs of 1024 / BATCH contiguous bytes each.
  constexpr int BATCH = 16 / EPV;
  static_assert(CACHE % BATCH == 0, "cached rounds must split into whole batches");
  __shared__ __attribute__((aligned(16))) uint8_t strip[THREADS * ROWS / 64][1024];
  uint8_t* mine = strip[threadIdx.x >> 6];
  const int lane = tid & 63;
  constexpr int LPR = 64 / BATCH;  // lanes that store one round's bytes of this wave
#pragma unroll
  for (int i0 = 0; i0 < CACHE; i0 += BATCH) {
    if (THREADS * (i0 + BATCH) <= nchunks) {  // uniform: every lane of every wave has all BATCH rounds
#pragma unroll
      for (int b = 0; b < BATCH; ++b) {
        uint32_t out[EPV / 4];
        convert(cache[i0 + b], out);
        if (EPV == 4) *(uint32_t*)(mine + b * 256 + lane * 4) = out[0];
        else *(v2u*)(mine + b * 512 + lane * 8) = (v2u){out[0], out[EPV / 4 - 1]};
      }
      const int b = lane / LPR, piece = lane % LPR;
      const v4i bytes = *(const v4i*)(mine + lane * 16);
      // round i0+b, this wave's 64 chunks start at chunk THREADS*(i0+b) + 64*wave
      *(v4i*)(qr + ((size_t)THREADS * (i0 + b) + (tid & ~63)) * EPV + piece * 16) = bytes;
    } else {
#pragma unroll
      for (int b = 0; b < BATCH; ++b) {
        const int c = tid + THREADS * (i0 + b);
        if (c < nchunks) convert_store(cache[i0 + b], c);
      }
    }
  }
  for (int c = tid + THREADS * CACHE; c < nchunks; c += THREADS) convert_store(xr[c], c);
}


// ------------------------------------------------------------------------------------
// Block-wise quantiser: one scale per 128 x 128 block of the source, the input step of the
// block-scaled GEMM. One workgroup per block keeps the block in registers between the
// maximum and the conversion, so the source is read once. Follows the eager PyTorch program of
// tritonbench/operators/fp8_gemm_blockwise/operator.py:86-118:
//   amax  = max |x| over the block (elements past M or K count as zero), clamped from below
//           with 1e-12 in the source type, then widened to f32
//   scale = fl(fl(1 / amax) * 448) in f32 (how PyTorch evaluates 448 / tensor); +inf -> 1
//   xq    = e4m3fn(fl(x * scale)), the product in f32 whatever the source type, no clamp
//           (|x * scale| cannot reach 464, the first value the cast turns into NaN)
//   inv   = fl(1 / scale)
// A block that holds a NaN comes out as NaN codes with a NaN inverse scale; a block that holds an
// infinity gets scale 0 and inverse scale +inf, its finite elements become zero, the infinities NaN.
// ------------------------------------------------------------------------------------
constexpr int kQuantBlock = 128;

template <typename SrcT>
__device__ __forceinline__ float block_scale(float amax) {
  const float floor_ = SrcTraits<SrcT>::round(1e-12f);
  const float clamped = amax < floor_ ? floor_ : amax;  // false for NaN: it stays
  const float scale = (1.0f / clamped) * 448.0f;
  return scale == __builtin_inff() ? 1.0f : scale;
}

// VEC: 16-byte source chunks (rows 16-byte aligned, K a whole number of chunks), 4- or 8-byte stores.
// Otherwise element by element, the block read twice (the second time from cache).
template <typename SrcT, bool VEC>
__global__ __launch_bounds__(256) void quantize_blocks_kernel(const SrcT* x, uint8_t* xq, float* inv_scale, int M,
                                                              int K, long ldx, long ldq, int grid_k) {
  using T = SrcTraits<SrcT>;
  using V = VecTraits<SrcT>;
  constexpr int EPV = V::EPV;
  constexpr int CPR = kQuantBlock / EPV;   // chunks per block row
  constexpr int RPP = 256 / CPR;           // block rows per pass of the workgroup
  constexpr int PASSES = kQuantBlock / RPP;
  __shared__ float wave_max[4];
  const int bk = blockIdx.x, bm = blockIdx.y;
  const int m0 = bm * kQuantBlock, k0 = bk * kQuantBlock;
  const int tid = threadIdx.x;
  const int chunk = tid % CPR, row0 = tid / CPR;

  v4i cache[VEC ? PASSES : 1];
  float amax = 0.0f;
  if constexpr (VEC) {
#pragma unroll
    for (int i = 0; i < PASSES; ++i) {
      const int r = m0 + row0 + i * RPP, c = k0 + chunk * EPV;
      const bool inside = r < M && c < K;
      // (outside the matrix a lane reads the block's first chunk, which exists, and drops it)
      const v4i got = __builtin_nontemporal_load((const v4i*)(x + (inside ? (long)r * ldx + c : (long)m0 * ldx + k0)));
      cache[i] = inside ? got : (v4i){0, 0, 0, 0};
      float f[EPV];
      V::unpack(cache[i], f);
#pragma unroll
      for (int e = 0; e < EPV; ++e) amax = max_keep_nan(amax, fabsf(f[e]));
    }
  } else {
    for (int idx = tid; idx < kQuantBlock * kQuantBlock; idx += 256) {
      const int r = m0 + idx / kQuantBlock, c = k0 + idx % kQuantBlock;
      if (r < M && c < K) amax = max_keep_nan(amax, fabsf(T::load(x + (long)r * ldx + c)));
    }
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) amax = max_keep_nan(amax, __shfl_xor(amax, o));
  if ((tid & 63) == 0) wave_max[tid >> 6] = amax;
  __syncthreads();
  amax = max_keep_nan(max_keep_nan(wave_max[0], wave_max[1]), max_keep_nan(wave_max[2], wave_max[3]));

  const float scale = block_scale<SrcT>(amax);
  if (tid == 0) inv_scale[(long)bm * grid_k + bk] = 1.0f / scale;
  const bool finite = amax < __builtin_inff();  // false for NaN and infinity: the integer encoder carries them

  if constexpr (VEC) {
#pragma unroll
    for (int i = 0; i < PASSES; ++i) {
      const int r = m0 + row0 + i * RPP, c = k0 + chunk * EPV;
      if (r >= M || c >= K) continue;
      float f[EPV];
      V::unpack(cache[i], f);
      uint32_t out[EPV / 4];
      if (finite) {
#pragma unroll
        for (int w = 0; w < EPV / 4; ++w) {
          // (the clamp changes nothing for a finite block; it keeps the pack-convert inside its range)
          float g[4];
#pragma unroll
          for (int e = 0; e < 4; ++e) g[e] = fminf(fmaxf(f[4 * w + e] * scale, -448.0f), 448.0f);
          int packed = __builtin_amdgcn_cvt_pk_fp8_f32(g[0], g[1], 0, false);
          packed = __builtin_amdgcn_cvt_pk_fp8_f32(g[2], g[3], packed, true);
          out[w] = (uint32_t)packed;
        }
      } else {
#pragma unroll
        for (int w = 0; w < EPV / 4; ++w) {
          out[w] = 0;
#pragma unroll
          for (int e = 0; e < 4; ++e) out[w] |= (uint32_t)f32_to_e4m3fn_rne(f[4 * w + e] * scale) << (8 * e);
        }
      }
      uint8_t* dst = xq + (long)r * ldq + c;
      if (EPV == 4) *(uint32_t*)dst = out[0];
      else *(v2u*)dst = (v2u){out[0], out[EPV / 4 - 1]};
    }
  } else {
    for (int idx = tid; idx < kQuantBlock * kQuantBlock; idx += 256) {
      const int r = m0 + idx / kQuantBlock, c = k0 + idx % kQuantBlock;
      if (r < M && c < K) xq[(long)r * ldq + c] = f32_to_e4m3fn_rne(T::load(x + (long)r * ldx + c) * scale);
    }
  }
}

// ------------------------------------------------------------------------------------
// Fused front ends of the row-wise GEMM: the activation is normalised (RMSNorm with a weight
// vector) or gated (SiLU(x1) * x2) and quantised row-wise in one pass, so the bf16 row is read
// from memory once and nothing but the e4m3fn codes and one scale per row is written.
// One workgroup per row; a lane keeps the fp32 values of up to CACHE 16-byte chunks (8 bf16
// each) in registers across the passes: [sum of squares ->] value and row maximum -> convert.
// Rows longer than THREADS*CACHE chunks re-read and recompute the rest. All arithmetic is fp32:
//   RMSNorm   y = (x * rstd) * w,  rstd = 1 / sqrt(mean(x^2) + eps)
//   SiLU-mul  y = (x1 / (1 + exp(-x1))) * x2
// then the quantiser's arithmetic on y as on an fp32 tensor (row_scale<float>, clamp, RNE).
// ------------------------------------------------------------------------------------
constexpr int kFusedRmsNorm = 0, kFusedSiluMul = 1;

template <int OP, int CACHE, int THREADS, int ROWS = 1>
__global__ __launch_bounds__(THREADS* ROWS) void fused_rowwise_quant_kernel(const uint16_t* x1, const uint16_t* x2,
                                                                             float eps, uint8_t* xq, float* inv_scale,
                                                                             int K, long ld1, long ld2, long ldq, long rows) {
  static_assert(ROWS == 1 || THREADS == 64, "several rows per workgroup: one wave each (as in the quantiser)");
  using V = VecTraits<uint16_t>;
  constexpr int EPV = 8;
  __shared__ float wave_part[2][THREADS / 64];  // one set per reduction: neither waits for the other's readers
  const long row = (long)blockIdx.x * ROWS + (ROWS > 1 ? (long)(threadIdx.x >> 6) : 0);
  if (ROWS > 1 && row >= rows) return;  // (whole waves; this form has no barrier)
  const v4i* r1 = (const v4i*)(x1 + row * ld1);
  // RMSNorm: the weight vector, shared by all rows; SiLU-mul: the row of the second operand
  const v4i* r2 = (const v4i*)(OP == kFusedRmsNorm ? x2 : x2 + row * ld2);
  uint8_t* qr = xq + row * ldq;
  const int nchunks = K / EPV;
  const int tid = ROWS > 1 ? (int)(threadIdx.x & 63) : (int)threadIdx.x;

  // sums (or maxima) of one value per lane over the row's lanes; every lane gets the result
  auto block_reduce = [&](int set, float v, auto op) -> float {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = op(v, __shfl_xor(v, o));
    if (THREADS == 64) return v;
    if ((tid & 63) == 0) wave_part[set][tid >> 6] = v;
    __syncthreads();
    float r = wave_part[set][0];
#pragma unroll
    for (int w = 1; w < THREADS / 64; ++w) r = op(r, wave_part[set][w]);
    return r;
  };
  // (hardware exponential and reciprocal, about one ulp each: the result is rounded to 4 significant
  // bits next; the library exponential costs six times the instructions and a correctly rounded
  // quotient ten, which together made the kernel compute-bound)
  auto silu_mul = [](float a, float b) -> float { return (a * __builtin_amdgcn_rcpf(1.0f + __expf(-a))) * b; };

  float vals[CACHE][EPV];
  // (the 1024-lane form has 128 registers per lane and none to spare for them; with 512 lanes and 8 chunks each the
  // weights' registers cost more than the second trip: 8192 x 28672 245 us with them, 167 without)
  constexpr bool EARLY_WEIGHTS = OP == kFusedRmsNorm && (THREADS <= 256 || (THREADS == 512 && CACHE <= 4));
  v4i wts[EARLY_WEIGHTS ? CACHE : 1];
  float rstd = 0.0f;
  if (OP == kFusedRmsNorm) {
    // pass 1: x to registers, sum of squares (lanes past the row's end re-read the last chunk and
    // leave it out of the sum). The weights of the cached chunks are asked for here as well: fetched
    // after the reduction they would put a second trip to the L2 on every row's critical path.
    float ss = 0.0f;
    if (EARLY_WEIGHTS) {
#pragma unroll
      for (int i = 0; i < CACHE; ++i) wts[EARLY_WEIGHTS ? i : 0] = r2[min(tid + THREADS * i, nchunks - 1)];
    }
#pragma unroll
    for (int i = 0; i < CACHE; ++i) {
      const int c = tid + THREADS * i;
      V::unpack(__builtin_nontemporal_load(r1 + min(c, nchunks - 1)), vals[i]);
      if (c < nchunks) {
#pragma unroll
        for (int e = 0; e < EPV; ++e) ss = __builtin_fmaf(vals[i][e], vals[i][e], ss);
      }
    }
    for (int c = tid + THREADS * CACHE; c < nchunks; c += THREADS) {
      float f[EPV];
      V::unpack(r1[c], f);
#pragma unroll
      for (int e = 0; e < EPV; ++e) ss = __builtin_fmaf(f[e], f[e], ss);
    }
    ss = block_reduce(0, ss, [](float a, float b) { return a + b; });
    rstd = 1.0f / sqrtf(ss / (float)K + eps);
  }
  // value of chunk c from its raw operands
  auto value = [&](const float (&a)[EPV], const float (&b)[EPV], float (&y)[EPV]) {
#pragma unroll
    for (int e = 0; e < EPV; ++e) y[e] = OP == kFusedRmsNorm ? (a[e] * rstd) * b[e] : silu_mul(a[e], b[e]);
  };
  // pass 2: values (kept for the cached chunks) and the row's absolute maximum
  float amax = 0.0f;
#pragma unroll
  for (int i = 0; i < CACHE; ++i) {
    const int c = min(tid + THREADS * i, nchunks - 1);
    float a[EPV], b[EPV];
    if (OP == kFusedRmsNorm) {
#pragma unroll
      for (int e = 0; e < EPV; ++e) a[e] = vals[i][e];
    } else {
      V::unpack(__builtin_nontemporal_load(r1 + c), a);
    }
    V::unpack(EARLY_WEIGHTS ? wts[EARLY_WEIGHTS ? i : 0] : OP == kFusedRmsNorm ? r2[c] : __builtin_nontemporal_load(r2 + c), b);
    value(a, b, vals[i]);
#pragma unroll
    for (int e = 0; e < EPV; ++e) amax = max_keep_nan(amax, fabsf(vals[i][e]));
  }
  for (int c = tid + THREADS * CACHE; c < nchunks; c += THREADS) {
    float a[EPV], b[EPV], y[EPV];
    V::unpack(r1[c], a);
    V::unpack(r2[c], b);
    value(a, b, y);
#pragma unroll
    for (int e = 0; e < EPV; ++e) amax = max_keep_nan(amax, fabsf(y[e]));
  }
  amax = block_reduce(1, amax, [](float a, float b) { return max_keep_nan(a, b); });

  const float scale = row_scale<float>(amax);
  if (tid == 0) inv_scale[row] = 1.0f / scale;
  const bool finite_row = amax < __builtin_inff();  // a NaN or an infinity takes the integer encoder, which carries NaN through
  auto convert_store = [&](const float (&y)[EPV], int c) {
    if (finite_row) {
      float f[EPV];
#pragma unroll
      for (int e = 0; e < EPV; ++e) f[e] = fminf(fmaxf(y[e] * scale, -448.0f), 448.0f);
      int lo = __builtin_amdgcn_cvt_pk_fp8_f32(f[0], f[1], 0, false);
      lo = __builtin_amdgcn_cvt_pk_fp8_f32(f[2], f[3], lo, true);
      int hi = __builtin_amdgcn_cvt_pk_fp8_f32(f[4], f[5], 0, false);
      hi = __builtin_amdgcn_cvt_pk_fp8_f32(f[6], f[7], hi, true);
      *(v2u*)(qr + (size_t)c * 8) = (v2u){(uint32_t)lo, (uint32_t)hi};
    } else {
#pragma unroll
      for (int e = 0; e < EPV; ++e) qr[(size_t)c * 8 + e] = quantize_one<float>(y[e], scale);
    }
  };
  // pass 3: convert. Two consecutive rounds of cached chunks meet in a wave-private LDS strip and
  // leave as one 16-byte store per lane (LDS executes a wave's operations in order: no barrier).
  __shared__ __attribute__((aligned(16))) uint8_t strip[THREADS * ROWS / 64][1024];
  uint8_t* mine = strip[threadIdx.x >> 6];
  const int lane = tid & 63;
  static_assert(CACHE % 2 == 0, "cached rounds are stored in pairs");
#pragma unroll
  for (int i0 = 0; i0 < CACHE; i0 += 2) {
    if (finite_row && THREADS * (i0 + 2) <= nchunks) {  // uniform: every lane of every wave has both rounds
#pragma unroll
      for (int b = 0; b < 2; ++b) {
        float f[EPV];
#pragma unroll
        for (int e = 0; e < EPV; ++e) f[e] = fminf(fmaxf(vals[i0 + b][e] * scale, -448.0f), 448.0f);
        int lo = __builtin_amdgcn_cvt_pk_fp8_f32(f[0], f[1], 0, false);
        lo = __builtin_amdgcn_cvt_pk_fp8_f32(f[2], f[3], lo, true);
        int hi = __builtin_amdgcn_cvt_pk_fp8_f32(f[4], f[5], 0, false);
        hi = __builtin_amdgcn_cvt_pk_fp8_f32(f[6], f[7], hi, true);
        *(v2u*)(mine + b * 512 + lane * 8) = (v2u){(uint32_t)lo, (uint32_t)hi};
      }
      const int b = lane / 32, piece = lane % 32;
      const v4i bytes = *(const v4i*)(mine + lane * 16);
      *(v4i*)(qr + ((size_t)THREADS * (i0 + b) + (tid & ~63)) * EPV + piece * 16) = bytes;
    } else {
#pragma unroll
      for (int b = 0; b < 2; ++b) {
        const int c = tid + THREADS * (i0 + b);
        if (c < nchunks) convert_store(vals[i0 + b], c);
      }
    }
  }
  for (int c = tid + THREADS * CACHE; c < nchunks; c += THREADS) {
    float a[EPV], b[EPV], y[EPV];
    V::unpack(r1[c], a);
    V::unpack(r2[c], b);
    value(a, b, y);
    convert_store(y, c);
  }
}

// ------------------------------------------------------------------------------------
// Host side
// ------------------------------------------------------------------------------------
int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(mi355x_shared::err, sizeof(mi355x_shared::err), fmt, ap);
  va_end(ap);
  return code;
}

constexpr int kSkinnyMaxM = 64;

int check_shape(int64_t M, int64_t N, int64_t K) {
  if (M < 1 || N < 1 || K < 1) return fail(MI355X_FP8_EINVAL, "M, N, K must be >= 1 (got %lld, %lld, %lld)",
                                           (long long)M, (long long)N, (long long)K);
  if (M > INT32_MAX || N > INT32_MAX || K > INT32_MAX)
    return fail(MI355X_FP8_ENOTSUP, "dimension exceeds 2^31-1");
  return MI355X_FP8_OK;
}
// What the MFMA families ask of the operands beyond check_shape (the generic family asks nothing).
int check_fast_shape(int64_t K) {
  if (K % 16 != 0) return fail(MI355X_FP8_ENOTSUP, "K must be a multiple of 16 (got %lld)", (long long)K);
  return MI355X_FP8_OK;
}

// ---- tiled-kernel plans: tile configuration x split-K factor
struct TileConfig {
  int bm, bn, wgs_per_cu;
  float us_per_step;        // one 128-byte K step of a work item, every workgroup slot busy
  float us_per_step_alone;  // the same with at most one workgroup per CU
  float us_per_item;        // pipeline refill + epilogue of one work item
  float stream_bytes_per_us;  // operand bytes per microsecond the configuration can stream from HBM
  float wg_stream_share;      // what one workgroup can stream, in units of 1/256 of that rate
};
constexpr int kNumTileConfigs = 7;
static_assert(kNumTileConfigs == mi355x_shared::kNumTiledParts, "one part function per tile configuration");
constexpr int kDeepSmallConfig = 6;  // 128x128 tiles with three steps in flight, one workgroup per CU
constexpr int kNumGroupedTileConfigs = 3;  // the grouped form uses the first three
// Measured on MI355X with normally distributed operands (clock under sustained MFMA load).
constexpr TileConfig kTileConfigs[kNumTileConfigs] = {
    {256, 256, tiled_wgs_per_cu(256, 256), 1.30f, 1.30f, 6.0f, 3.6e6f, 1.8f},
    {128, 128, tiled_wgs_per_cu(128, 128), 1.00f, 0.60f, 5.0f, 4.4e6f, 1.18f},
    {256, 128, tiled_wgs_per_cu(256, 128), 0.87f, 0.87f, 5.0f, 4.0e6f, 1.1f},
    {64, 256, tiled_wgs_per_cu(64, 256), 0.75f, 0.75f, 9.0f, 5.7e6f, 1.42f},
    // (one tile row against a wide panel: 128 x 57344 x 8192 75.2 us with 224 tiles, bound by the stream rate;
    // several tile rows: 512 x 16384 x 16384 125 us with 256 tiles, 4096 x 5120 x 13824 269 us with 640)
    // (a step and a tile's refill and epilogue, from launches that are not bound by the stream rate: 4096 x 2048 x 2048
    // 18.1 us with 256 tiles of 16 steps, 636 x 12288 x 6144 50.3 with 240 of 48, 512 x 16384 x 16384 125 with 256 of 128)
    {128, 256, tiled_wgs_per_cu(128, 256), 0.97f, 0.97f, 2.6f, 5.8e6f, 1.42f},
    // (panels whose 256-column tiles come to more than half a round with 256 rows each but fit one with 192:
    // 1024 x 10240 x 8192 73.3 us with 240 tiles, 2048 x 10240 x 8192 135.4 us with 440)
    // (one tile row against a wide panel: 192 x 57344 x 8192 89.2 us)
    // (one round of tiles costs 7 us beside its steps, not 9: plan_cost_us has it)
    {192, 256, tiled_wgs_per_cu(192, 256), 1.00f, 1.00f, 9.0f, 4.9e6f, 1.42f},
    // 128x128 tiles with loads three steps ahead (112 KB of LDS: one workgroup per CU), for launches of at most
    // one workgroup per CU, where a CU has one wave per SIMD and nothing but the depth of the ring to cover
    // the memory latency with. Operands from HBM, against the two-step form: 1024 x 2048 x 4096 25.4 -> 20.4 us
    // with 128 tiles, 512 x 4096 x 4096 25.6 -> 21.1, 1536 x 1536 x 4096 25.4 -> 20.6, 2048 x 2048 x 4096 27.2 ->
    // 23.0 with 256, 2048^3 15.9 -> 14.4; split (work items still at most one per CU): 1024 x 2048 x 8192 36.1 ->
    // 31.3 in two, 1024 x 2048 x 16384 67.3 -> 48.9 in two, 1024 x 1024 x 8192 36.3 -> 26.5 in two -> 23.0 in four.
    // Operands from the memory-side cache: 0.31 us per step instead of 0.49 (1024 x 2048 x 8192 29.1 -> 24.6).
    // A ring one step deeper measured the same. The step time is the one with operands from HBM and half the
    // CUs at work; plan_cost_us adds what a fuller chip costs.
    {128, 128, 1, 0.49f, 0.49f, 4.8f, 4.4e6f, 1.18f},
};

// The skinny kernel's run time for comparison with the tiled plans at M <= 64: a fixed part
// plus B streamed at a rate that falls with the number of 16-row blocks of A every workgroup
// has to pull through L1 beside its rows of B (measured, MB per microsecond). With three or
// four blocks the register budget leaves one workgroup per CU, and a last round of workgroups
// that fills only part of the CUs streams at that fraction of the rate.
inline bool persistent_skinny_fits(int64_t M, int64_t N, int64_t K);
// The pair kernel: up to 16 rows of A, at most two 16-row tiles of B per CU, K that fits the LDS.
inline bool pair_skinny_fits(int64_t M, int64_t N, int64_t K) {
  return M <= 16 && N % 16 == 0 && N <= 2 * 16 * kNumCu && K <= 4 * kPersistWaves * kStepK;
}
// The narrow-tile kernel. With all rows in one workgroup (M <= 64) its cost is one round of workgroups per
// 256 tiles (measured at N = 8192, cold: 9.8 / 14.3 / 43.0 us for K = 4096 / 8192 / 28672 with up to
// 32 rows of A, 17.1-17.9 / 49.9 us for K = 8192 / 28672 with up to 64).
// Up to 256 rows of A it runs in row blocks where that is one round of workgroups, one per CU
// (measured, K = 8192 unless given: 64x64 tiles 13.7 / 21.5 / 67.6 us for K = 4096 / 8192 / 28672 at
// M = 128, N = 8192; 64x32 tiles 10.7 / 16.0 / 24.2 us for K = 4096 / 8192 / 14336 at M = 128, N = 4096,
// 14.0 us at 192 x 1536; 32x32 tiles 12.6 us at 64 x 4096, 11.3 us at 128 x 2048, 11.0 us at 64 x 1024,
// 8.3 us at 64 x 4096 x 4096, 37.1 us at 64 x 4096 x 28672).
constexpr int kNarrowMaxM = 256;
inline bool narrow_fits(int64_t M, int64_t N, int64_t K) {
  (void)K;
  if (M <= kSkinnyMaxM) return true;
  const long tiles = ((N + 63) / 64 + kNumXcd - 1) / kNumXcd * kNumXcd, row_blocks = (M + 63) / 64;
  return M <= kNarrowMaxM && tiles * row_blocks <= kNumCu;
}
// The form for a shape: 32-row blocks of A per workgroup (the rows beyond them go to further row
// blocks) and 32-column blocks per tile. Up to 32 rows, and up to 64 on panels too wide for row
// blocks: all rows in one workgroup, tiles of narrow_tile_cols() columns (two blocks from 33 columns up).
// Otherwise the smallest tile whose row blocks are one round of workgroups: more CUs at work, and
// less to deliver into each one's LDS.
struct NarrowForm {
  int mb, nb;
};
inline long narrow_workgroups(int64_t M, int64_t N, NarrowForm f) {
  const long tiles = (N + 32 * f.nb - 1) / (32 * f.nb), row_blocks = (M + 32 * f.mb - 1) / (32 * f.mb);
  return row_blocks == 1 ? tiles : (tiles + kNumXcd - 1) / kNumXcd * kNumXcd * row_blocks;
}
// Columns per tile where all rows sit in one workgroup: the columns dealt out evenly over the CUs, in multiples
// of 4 (8-byte stores), up to the 64 a workgroup can take; beyond 64 x 256 columns the launch needs several
// rounds of workgroups anyway and the tiles stay 32 wide.
inline int narrow_tile_cols(int64_t N) {
  if (N > 64 * (int64_t)kNumCu) return 32;
  const int64_t per_cu = (N + kNumCu - 1) / kNumCu;
  const int w = (int)((per_cu + 3) / 4 * 4);
  return w < 4 ? 4 : w;
}
inline NarrowForm narrow_form(int64_t M, int64_t N) {
  if (M <= 32) return {1, narrow_tile_cols(N) > 32 ? 2 : 1};
  static const NarrowForm by_size[3] = {{1, 1}, {2, 1}, {2, 2}};
  for (const NarrowForm f : by_size)
    if (narrow_workgroups(M, N, f) <= kNumCu) return f;
  return {2, narrow_tile_cols(N) > 32 ? 2 : 1};  // (M <= 64: all rows in one workgroup)
}
inline float narrow_cost_us(int64_t M, int64_t N, int64_t K) {
  const NarrowForm f = narrow_form(M, N);
  if (M > 32 * f.mb) {  // row blocks, one round
    const float k1024 = (float)K / 1024.0f;
    const float share = (float)narrow_workgroups(M, N, f) / (float)kNumCu;  // of the CUs at work
    // (64x64 tiles: 1.9 us per 1024 bytes of K with every CU at work, 1.7 with 160 of them, 256 x 2304 x 6656 17.0 us)
    if (f.nb == 2) return 6.0f + k1024 * (K > 16384 ? 2.15f : 1.34f + 0.56f * share);
    if (f.mb == 2) return 5.4f + k1024 * (0.75f + 0.575f * share);
    return 3.5f + k1024 * (0.9f + 0.25f * share);
  }
  // All rows in one workgroup, one round of workgroups: the columns are dealt out evenly (narrow_tile_cols), and
  // what a workgroup waits for is its operands against the fetches a CU can have outstanding (about 64 KB): its
  // rows of B at HBM's latency (2 us), its rows of A at the L2's (0.6 us), plus start and launch. Measured cold at
  // M = 32, K = 8192: N = 1024 8.5 us, 2048 8.9, 4096 11.9, 5120 11.7, 8192 14.5, 10240 17.2, 16384 23.5 (N = 12288:
  // 21.1, three more than this says: with 48-column tiles the chip as a whole delivers less); K = 4096: N = 4096 7.3,
  // 14336 12.9; M = 64: 8192 x 8192 17.9, 10240 x 8192 20.6; M = 16: 13312 x 13312 29.3.
  // (Fewer than 16 rows of A cost what 16 do: 1 x 5120 x 8192 10.1 us, 16 x 5120 x 8192 10.2.)
  if (N <= 64 * (int64_t)kNumCu) {
    const float w = (float)narrow_tile_cols(N);
    // (Narrow panels: with 4 to 16 columns a workgroup there is little to fetch, and what a step of K costs is its
    // trip to memory against the depth of the ring, 0.07 to 0.1 us per 128 bytes. Up to 16 rows, N = 2048: 5.8 / 8.3 /
    // 11.8 / 21.8 us at K = 4096 / 8192 / 13312 / 28672; N = 1024 5.7 / 8.2 / - / 20.6, 3072 6.1 / 8.9 / 12.6 / 23.7;
    // 32 rows, K = 28672: N = 1024 21.7, 2048 23.4, 3072 26.0, 3584 28.8.)
    const float rows = (float)(M < 16 ? 16 : M);
    return fmaxf(4.4f + w * (float)K / 32768.0f + rows * (float)K * (0.6f / 65536.0f),
                 3.2f + (float)K * (5.0e-4f + 0.135e-4f * w + 0.035e-4f * rows));
  }
  const long tiles = (N + 31) / 32;
  const long rounds = (tiles + kNumCu - 1) / kNumCu;
  // per 1024 bytes of K: what the CUs at work can pull from L2, or, with most of them at work and up to 32
  // rows, what HBM delivers of B (measured at M <= 32: 8.6 us at 5120 x 5120, 8.3 at 4096 x 4096, 14.3 at 8192 x 8192)
  const float share = fminf(1.0f, (float)tiles / (float)kNumCu);
  const float k1024 = (float)K / 1024.0f;
  // (with fewer than half the CUs at work the fixed part is larger than this form has it: the old rate stays)
  if (M <= 32) return (float)rounds * (3.5f + k1024 * (tiles >= kNumCu / 2 ? fmaxf(1.08f, 1.38f * share) : 1.38f));
  return (float)rounds * (4.5f + k1024 * (1.1f + 0.52f * share));
}
// The pair kernel. Its time follows the CU with the most tiles, and the K steps are dealt to its 16 waves in whole
// rounds (K = 2304 is 18 steps in 32 slots): half the columns count as dealt evenly, half as the busiest CU's, and K
// as rounded up to 2048. Measured cold: 16 x 8192 x 8192 12.75 us, K = 4096 7.9, K = 2048 5.4; M = 1: 8192 x 8192
// 12.4, 4096 x 8192 8.0, 4096 x 4096 5.6, 8192 x 2048 5.1, 4096 x 2304 5.0; M = 16: 5120 x 8192 11.2, 6144 x 8192 11.5.
// With one tile a CU there is little of B to hide the fetch of A behind (N = 2048, K = 8192: 6.8 us with one row of A,
// 7.8 with 16; K = 4096: 5.1 / 5.5; N = 8192, K = 8192: 12.4 / 12.75).
inline float pair_cost_us(int64_t M, int64_t N, int64_t K) {
  const float cols_busiest = (float)(16 * ((N / 16 + kNumCu - 1) / kNumCu) * kNumCu);
  const float k_slots = (float)((K + 16 * kStepK - 1) / (16 * kStepK) * (16 * kStepK));
  const float a_rows = N <= 16 * kNumCu ? (float)M * (float)K * (1.1e-4f / 16.0f) : 0.0f;
  // (a quarter of the CUs at work: 1 x 1024 x 4096 4.95 us, 1 x 1024 x 8192 6.5)
  const float fixed = N <= 1536 ? 3.35f : N <= 16 * kNumCu ? 3.1f : 2.75f;
  return fixed + 0.5f * ((float)N + cols_busiest) * k_slots / 6.7e6f + a_rows;
}
// The general kernel, one 16- or 32-row tile of B per workgroup.
inline float one_tile_cost_us(int64_t M, int64_t N, int64_t K) {
  static const float rate[4] = {6.0e6f, 4.5e6f, 3.44e6f, 3.6e6f};
  const int blocks = (int)((M + 15) / 16);
  const int b = blocks < 1 ? 0 : blocks > 4 ? 3 : blocks - 1;
  float r = M <= 8 ? 7.2e6f : rate[b];  // (a few rows of A: its loads hit in L1 almost always)
  // two blocks, one round of workgroups (two per CU) and a short K: everything is in flight at once
  if (b == 1 && N <= 16 * 2 * kNumCu && K <= 8192) r = 4.9e6f;
  // The kernel takes as long as its busiest CU: workgroups are dealt out in rounds of one per CU, and a last
  // round that reaches only some CUs costs a whole one (16 x 5120 x 13824: 20.8 us with 320 workgroups, where
  // 4096 x 14336 with 256 takes 12.9).
  // (With one or two blocks of A a single round that leaves CUs idle is left as it was: those shapes are a few
  // microseconds long and bound by the launch, 32 x 2048 x 2048 4.5 us.)
  const long wgs = (N + (b == 3 ? 31 : 15)) / (b == 3 ? 32 : 16);
  const long rounds = (wgs + kNumCu - 1) / kNumCu;
  if (b >= 2 || rounds > 1) r *= (float)wgs / (float)(rounds * kNumCu);
  // (up to 16 rows, measured cold: 1 x 8192 x 8192 12.1 us, 1 x 4096 x 8192 7.5, 1 x 2304 x 2048 3.7,
  // 16 x 8192 x 8192 13.8, 16 x 4096 x 4096 5.6)
  // (two blocks: 32 x 2048 x 2048 4.5 us)
  float t = (b == 0 ? 3.0f : b == 1 ? 3.7f : 5.0f) + (float)N * (float)K / r;
  // (Wide panels with short rows: every workgroup has a start and an end that no other hides, 1.7 ns apiece beyond the
  // first 512, which shows where a workgroup's share of K is short: 3 x 45376 x 1024 14.7 us for 46 MB, 1 x 103104 x
  // 1664 38.1 for 172 MB, 3 x 97728 x 2304 44.6; at K = 8192 half of it is left, 1 x 57344 x 8192 71.5.)
  if (b == 0 && wgs > 2 * kNumCu) t += (float)(wgs - 2 * kNumCu) * 1.66e-3f * fminf(1.0f, 4096.0f / (float)K);
  // Part of the chip at work, up to 32 rows: a workgroup has its CU to itself, and a byte of K costs it what its 16
  // rows of B (from HBM) and its rows of A (from L2) take against the fetches a CU can have outstanding, whatever
  // the number of workgroups. Measured with 128 workgroups (N = 2048) at K = 4096 / 8192 / 16384 / 28672: one row of
  // A 4.5 / 6.2 / 9.7 / 14.9 us, 8 rows 4.7 / 6.6 / 10.6 / 17.0, 16 rows 5.1 / 7.6 / 12.2 / 20.5, 32 rows 6.2 / 9.8 /
  // - / -; with 64 (N = 1024): one row 4.2 / 6.0 / 8.8 / 13.8, 16 rows 4.9 / 7.1 / 11.6 / 19.3; 144 workgroups,
  // K = 16384: 10.8 / 12.5 / 16.4 us with 8 / 16 / 32 rows.
  // (Rows that do not start on a 128-byte boundary: every 128-byte piece of a row lies across two cache lines, and a
  // workgroup alone on its CU, which asks for its rows 128 bytes at a time, takes 1.4-1.5 times as long per byte of K:
  // 17 x 2816 x 18832 23.6 us where aligned rows would take 15.5, 14 x 1536 x 9760 11.4 against 8.4; the narrow-tile
  // kernel, 512 bytes of a row at a time, loses 0-12 % on the same shapes. With several rounds of workgroups every
  // kernel loses about the same, 1.25-1.4, and the order of the estimates holds. K stands in for the row pitch.)
  const float pitch = K % kStepK != 0 ? 1.45f : 1.0f;
  if (b <= 1 && wgs < kNumCu) t = fmaxf(t, 2.6f + pitch * (float)K * (4.1e-4f + 0.13e-4f * (float)M));
  // (three blocks of A, the same way: 48 x 2048 x 4096 7.5-8.0 us, 48 x 2048 x 8192 12.1-12.6, 34 x 2048 x 1024 3.4,
  // 48 x 3584 x 28672 36.8; the rate above, scaled by the share of the CUs at work, has these shapes a quarter slower)
  if (b == 2 && wgs < kNumCu) t = fminf(t, 3.0f + 1.08f * pitch * (float)K * (4.1e-4f + 0.13e-4f * (float)M));
  return t;
}
// The streaming members of the family and which of them runs a shape: the pair kernel where it fits, unless the
// one-tile kernel is expected ahead (at M <= 8 by a few per cent on most shapes, by 15-20 % where K fills the pair
// kernel's step slots badly: 1 x 4096 x 2304 4.3 us against 5.0); the persistent kernel beyond the pair kernel's N.
enum SkinnyStreaming { kStreamPair, kStreamPersistent, kStreamOneTile };
inline SkinnyStreaming skinny_streaming_choice(int64_t M, int64_t N, int64_t K) {
  if (pair_skinny_fits(M, N, K)) return one_tile_cost_us(M, N, K) < pair_cost_us(M, N, K) ? kStreamOneTile : kStreamPair;
  return persistent_skinny_fits(M, N, K) ? kStreamPersistent : kStreamOneTile;
}
inline float skinny_streaming_cost_us(int64_t M, int64_t N, int64_t K) {
  switch (skinny_streaming_choice(M, N, K)) {
    case kStreamPair: return pair_cost_us(M, N, K);
    // the persistent form (measured: 71 us at 16 x 57344 x 8192; two blocks of A, K = 4096: 9.9 us at N = 8192, 8.9 at
    // 24 x 6144 x 4096; one step per wave, K = 2048: a tile is over before the next one's rows have arrived, 4 x 13312 x 2048 8.2 us)
    // (K = 2048, one step per wave: 1 x 128256 x 2048 50.6 us, 4 x 13312 x 2048 8.2)
    case kStreamPersistent:
      if (K <= 2048 && M <= 16) return 3.4f + (float)N * (float)K / 5.7e6f;
      return (K <= 2048 ? 4.2f : 3.0f) + (float)N * (float)K / (M <= 16 ? 6.9e6f : 4.4e6f);
    default: return one_tile_cost_us(M, N, K);
  }
}
// the cheapest member of the M <= 64 family: streaming (persistent or one tile per workgroup) or narrow tiles
inline bool narrow_preferred(int64_t M, int64_t N, int64_t K) {
  if (M > kSkinnyMaxM) return narrow_fits(M, N, K);  // (the streaming kernels stop at 64 rows)
  return narrow_fits(M, N, K) && narrow_cost_us(M, N, K) < skinny_streaming_cost_us(M, N, K);
}
inline float skinny_cost_us(int64_t M, int64_t N, int64_t K) {
  if (M > kSkinnyMaxM && !narrow_fits(M, N, K)) return 1e30f;
  return narrow_preferred(M, N, K) ? narrow_cost_us(M, N, K) : skinny_streaming_cost_us(M, N, K);
}
constexpr int kMaxSplits = 16;
// Tile rows up to which a launch fetches B with the streaming policy (see gemm_tiled_kernel).
constexpr int kStreamTileRows = 2;
// (256x256 tiles: one tile row only. M=256, N=57344, K=8192 120.3 -> 109.7 us; with two tile rows, M=512, the
// policy costs 2-3 %.)
constexpr int stream_tile_rows(int bm, int bn) { return bm == 256 && bn == 256 ? 1 : kStreamTileRows; }

struct TiledPlan {
  int config, splits, steps_per_split;
  float cost_us;
};

inline int k_steps_of(int64_t K) { return (int)((K + kStepK - 1) / kStepK); }

// Splits actually used when `want` are asked for: every split gets the same whole number of
// steps and none is empty.
inline void normalise_splits(int k_steps, int want, int& splits, int& sps) {
  want = want < 1 ? 1 : (want > k_steps ? k_steps : want);
  sps = (k_steps + want - 1) / want;
  splits = (k_steps + sps - 1) / sps;
}

// Estimated run time of a plan. Work items are dealt to 256 * wgs_per_cu workgroup slots in
// rounds; a last round that fills at most one slot per CU runs at the faster stand-alone
// rate. The operands cannot arrive faster than the configuration streams from HBM. Split
// plans add a launch and the partial sums' trip through memory (written once, read once).
inline float plan_cost_us(int64_t M, int64_t N, int64_t K, int config, int splits, int sps) {
  const TileConfig& c = kTileConfigs[config];
  const long tiles = ((M + c.bm - 1) / c.bm) * ((N + c.bn - 1) / c.bn);
  const long items = tiles * splits;
  const long slots = (long)kNumCu * c.wgs_per_cu;
  const long full_rounds = items / slots, rest = items % slots;
  // (256x128 tiles are bound by the delivery of their operands, and rows of a tile past M are not fetched: with a last
  // tile row that is half empty a step takes less, 384 x 16384 x 16384 106.5 us = 0.79 us per step instead of 0.87,
  // 384 x 13312 x 13312 85.7, 640 x 8192 x 8192 53.5, 448 x 10240 x 8192 51.4 where three splits of 256x256 tiles take
  // 62.8. Unsplit plans only: with the same allowance split plans were taken where they measure behind, 448 x 2304 x
  // 13312 in seven 33.0 us against 28.5 for the deep 128x128 form in three.)
  const float rows_fetched = (float)M / (float)((M + c.bm - 1) / c.bm);
  const float step_scale = config == 2 && splits == 1 ? 0.5f + 0.5f * (rows_fetched + (float)c.bn) / (float)(c.bm + c.bn) : 1.0f;
  // (192x256 tiles in a single round: 4712 x 2048 x 1024 14.0-14.8 us with 200 tiles of 8 steps, 416 x 21312 x 1024 15.0
  // with 252, 2560 x 8192 x 1024 26.6 with 448 where 128x256 tiles take 30.3; over several rounds the table's 9 us per
  // tile stands: it leaves the estimate as far above the measurement as that of the 256x256 tiles, 3-4 %, and the order
  // of the two right: 896 x 57344 x 8192 343 us with 256x256 tiles, 354 with these)
  // (64x256 tiles, unsplit, over very short rows, K up to 1664: the table's constants are those of long weight panels;
  // here a step takes 0.54 us and a tile 5 beside its steps: 400 x 8704 x 1536 10.8 us with 238 tiles, 3 x 45376 x 1024
  // 11.6 with 178, 192 x 21312 x 1024 8.9 with 252. Only where 128x128 tiles are more than one round: up to that the
  // deep 128x128 form measures ahead, 400 x 8192 x 1024 7.7 us against 8.5, and its own estimate is a cautious one.)
  const bool short_c3 = config == 3 && splits == 1 && K <= 13 * kStepK && ((M + 127) / 128) * ((N + 127) / 128) > kNumCu;
  // (128x256 tiles over fewer than 8 steps: what a launch costs before its first step is not in the table's 2.6 us a
  // tile, 2129 x 32 x 512 7.2 us with 17 tiles where 128x128 tiles take 5.2: such launches are left to those)
  const float us_per_item = config == 5 && items <= 2 * slots ? 7.0f : short_c3 ? 5.0f : config == 4 && sps < 8 ? 10.0f : c.us_per_item;
  const float us_step = short_c3 ? 0.54f : c.us_per_step, us_step_alone = short_c3 ? 0.54f : c.us_per_step_alone;
  float t = full_rounds * (sps * us_step * step_scale + us_per_item);
  if (rest) t += sps * (rest <= kNumCu ? us_step_alone : us_step) * step_scale + us_per_item;
  // (the deep 128x128 form is for one round only; beyond 128 workgroups its steps slow down with the chip's
  // clock and the shared L2: 0.49 us with 128, 0.58 with 256)
  if (config == kDeepSmallConfig) {
    if (items > kNumCu) return 1e30f;
    if (items > kNumCu / 2) t += sps * 0.09f * (float)(items - kNumCu / 2) / (float)(kNumCu / 2);
  }
  // (one or two tile rows, one for 256x256 tiles: B is fetched with the streaming policy, which is worth 8 % or more)
  const bool streams_b = (M + c.bm - 1) / c.bm <= stream_tile_rows(c.bm, c.bn);
  // (fewer work items than CUs: the busy CUs cannot make up for the idle ones beyond their share)
  const float busy = items >= kNumCu ? 1.0f : fminf(1.0f, c.wg_stream_share * (float)items / (float)kNumCu);
  // (64x256 tiles, unsplit: the rotated K order lifts the rate further; with two splits the plan measured at the
  // plain rate, 48 x 28672 x 8192 47.5 us)
  // (256x256 tiles gain the most: their rate without the policy is the lowest)
  const float policy = !streams_b || config == kDeepSmallConfig ? 1.0f
                       : (config == 3 && splits == 1) ? 1.08f * 1.1f : config == 0 ? 1.2f : 1.08f;
  // (128x128 tiles: the rate was measured with full tiles; rows of a tile past M are not fetched, and what a CU
  // has to take in beside its rows of B shrinks with them: 64 x 28672 x 8192 unsplit 42.4 us = 6.3 MB/us)
  const float rows_a = (float)M / (float)((M + c.bm - 1) / c.bm);
  // (not below 33 rows: there the estimate would undercut the streaming kernels, which measure 25 % ahead)
  // (with short rows, K up to 4096, the allowance holds for any M: there the streaming kernels pay for every workgroup's
  // start and do not measure ahead, 1 x 128256 x 2048 44.7 us with 128x128 tiles against 50.6)
  const float fill = (config == 1 || config == kDeepSmallConfig) && (M > 32 || K <= 4096) ? fmaxf(0.75f, (rows_a + (float)c.bn) / (float)(c.bm + c.bn)) : 1.0f;
  // (the 256-column tiles of one tile row stream less with short rows, where a tile is over after a few steps: of
  // their rate at K >= 4096 they reach 0.8 up to K = 2048 and 0.87 at 2560; 1 x 128256 x 2048 46.8 us with 64x256
  // tiles and 49.6 with 128x256, 2 x 115072 x 2560 50.6 and 53.2, 1 x 128256 x 4096 79.5 and 81.7)
  const float short_rows = (config == 3 || config == 4) && K < 4096 ? fmaxf(0.8f, 0.8f + 0.2f * (float)(K - 2048) / 2048.0f) : 1.0f;
  const float stream = ((float)M * (float)K + (float)N * (float)K) * fill / (c.stream_bytes_per_us * policy * busy * short_rows);
  if (t < stream) t = stream;
  if (splits > 1) t += 3.0f + 2.0f * (float)splits * (float)M * (float)N * 4.0f / 5.0e6f;
  return t;
}

// Cheapest plan by the model above; `max_splits` = 1 restricts it to plans without workspace.
inline TiledPlan plan_tiled(int64_t M, int64_t N, int64_t K, int force_config, int force_splits,
                            int max_splits) {
  const int k_steps = k_steps_of(K);
  TiledPlan best = {0, 1, k_steps, 0.0f};
  float best_cost = -1.0f;
  for (int c = 0; c < kNumTileConfigs; ++c) {
    if (force_config >= 0 && c != force_config) continue;
    for (int want = 1; want <= max_splits; ++want) {
      if (force_splits > 0 && want != force_splits) continue;
      int splits, sps;
      normalise_splits(k_steps, want, splits, sps);
      if (force_splits <= 0 && splits != want) continue;  // duplicate of a smaller request
      // (128x256 tiles are the plan for whole rows of K against wide panels; split, they measured behind what
      // their estimate says: 128 x 8192 x 28672 66.3 us against 56.5 with 128x128 tiles)
      // (192x256 tiles were not measured split either)
      if ((c == 4 || c == 5) && force_splits <= 0 && splits > 1) continue;
      // (the deep ring takes three steps to fill: short rows of K stay with the two-step form, 2048 x 2048 x 512
      // 6.5 us against 6.9)
      if (c == kDeepSmallConfig && force_config < 0 && sps < 8) continue;
      // (With one or two tile rows the other configurations fetch B with the streaming policy; the deep form with
      // that policy measured 37.7 us on 256 x 4096 x 8192 against 20.1 for the 64x256 tiles, so it does not have it.
      // Without it B's lines stay in the caches: on weights small enough to be found there again it is the fastest
      // plan of all at 96 to 256 rows (operands from the memory-side cache: 256 x 6144 x 4096 14.6 us against 23.8,
      // 128 x 13312 x 2048 10.0 against 13.9; from HBM level with the 128x128 form), on large ones the policy wins
      // (64 x 28672 x 8192 from HBM: 51.7 us against 42.7).)
      if (c == kDeepSmallConfig && force_config < 0 && M <= 2 * 128 && N * K > (int64_t)48 << 20) continue;
      const float cost = plan_cost_us(M, N, K, c, splits, sps);
      if (best_cost < 0.0f || cost < best_cost) {
        best_cost = cost;
        best = {c, splits, sps, cost};
      }
    }
  }
  return best;
}

// variant word: bits 0..7 kernel family, bits 8..15 tile configuration + 1 (0 = automatic),
// bits 16..23 split-K factor (0 = automatic)
inline TiledPlan plan_from_variant(int64_t M, int64_t N, int64_t K, int variant, int max_splits) {
  const int cfg = ((variant >> 8) & 0xff) - 1;
  const int spl = (variant >> 16) & 0xff;
  return plan_tiled(M, N, K, cfg, spl, spl > 0 ? spl : max_splits);
}

constexpr int kMaxDevices = 64;
// The tile walk, the grid sizes and the cost tables are written for the whole part: 256 CUs in 8
// XCDs. A device that reports another CU count (a partitioned mode, another product) would be
// scheduled wrongly without any error, so it is turned away, once per device, when the device is
// set up.
int check_device_shape(int dev) {
  int cus = 0;
  const hipError_t e = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
  if (e != hipSuccess) return fail(MI355X_FP8_ELAUNCH, "hipDeviceGetAttribute: %s", hipGetErrorString(e));
  if (cus != kNumCu)
    return fail(MI355X_FP8_ENOTSUP, "device %d does not report the %d compute units these kernels are scheduled for "
                "(a partitioned mode or another part)", dev, kNumCu);
  return MI355X_FP8_OK;
}

// Every kernel instantiation that needs more dynamic LDS than the default limit enters itself in
// this table while the library is loaded (static initialisation, before any call can arrive).
// Setting a device up walks the table once and raises each kernel's limit there, so that no
// launch path has anything but the launch itself to do: a caller whose first use of some
// instantiation happens under graph capture meets no attribute call.
// (The table is shared by the translation units of a build in parts; it is zero-initialised storage,
// so registrations from any unit's static initialisers find it ready.)
bool register_lds_kernel(const void* kernel, size_t lds_bytes) {
  using namespace mi355x_shared;
  if (num_lds_kernels < mi355x_shared::kMaxLdsKernels) lds_kernels[num_lds_kernels++] = {kernel, lds_bytes};
  else lds_table_overflow = true;
  return true;
}
template <auto Kernel, size_t LdsBytes>
struct LdsLimit {
  static inline const bool registered = register_lds_kernel(reinterpret_cast<const void*>(Kernel), LdsBytes);
};

// 0 = not set up, 1 = ready, -1 = refused (wrong device shape). Setting a device up twice from two
// threads is harmless: every step is idempotent.
#if !defined(MI355X_TILED_PART)
std::atomic<int> g_device_state[kMaxDevices];
std::atomic<void*> g_scratch_ptr[kMaxDevices];
int setup_device(int dev);
#endif
inline int ready_device(int* dev_out = nullptr) { return mi355x_shared::ready_device(dev_out); }
}  // namespace

#if !defined(MI355X_TILED_PART)
thread_local char mi355x_shared::err[512] = "";
mi355x_shared::LdsKernel mi355x_shared::lds_kernels[mi355x_shared::kMaxLdsKernels];
int mi355x_shared::num_lds_kernels = 0;
bool mi355x_shared::lds_table_overflow = false;

// The current device, set up. The only HIP call on the ready path is hipGetDevice.
int mi355x_shared::ready_device(int* dev_out) {
  int dev = 0;
  const hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return fail(MI355X_FP8_ELAUNCH, "hipGetDevice: %s", hipGetErrorString(e));
  if (dev < 0 || dev >= kMaxDevices) return fail(MI355X_FP8_ENOTSUP, "device index %d beyond %d", dev, kMaxDevices - 1);
  if (dev_out) *dev_out = dev;
  if (g_device_state[dev].load(std::memory_order_acquire) == 1) return MI355X_FP8_OK;
  return setup_device(dev);
}
#endif

namespace {
template <int BM, int BN, int WAVES_M, int WAVES_N, bool KTAIL, int EPI, bool GROUPED = false, bool BLOCKSCALE = false,
          int DIST = kDefaultDist, bool STREAM_B = false>
int launch_tiled(GemmParams p, hipStream_t stream) {
  constexpr int threads = WAVES_M * WAVES_N * 64;
  constexpr size_t lds_bytes = tiled_lds_bytes(BM, BN, DIST);
  // grouped: the group sizes live on the device; every group adds at most one partial tile row
  p.tiles_m = GROUPED ? p.M / BM + p.groups : (p.M + BM - 1) / BM;
  p.tiles_n = (p.N + BN - 1) / BN;
  p.group_m = kGroupM;
  make_fast_div((uint32_t)p.tiles_m * (uint32_t)p.tiles_n, p.div_tiles_mul, p.div_tiles_shift);
  make_fast_div((uint32_t)kGroupM * (uint32_t)p.tiles_n, p.div_group_mul, p.div_group_shift);
  const long total = (long)p.tiles_m * p.tiles_n * p.splits;
  if (total > (long)INT32_MAX) return fail(MI355X_FP8_ENOTSUP, "more than 2^31-1 work items");
  const long slots = (long)kNumCu * tiled_wgs_per_cu(BM, BN, BLOCKSCALE, DIST);
  long grid = total < slots ? ((total + kNumXcd - 1) / kNumXcd) * kNumXcd : slots;
  constexpr auto kern = gemm_tiled_kernel<BM, BN, WAVES_M, WAVES_N, KTAIL, EPI, GROUPED, BLOCKSCALE, DIST, STREAM_B>;
  (void)LdsLimit<kern, lds_bytes>::registered;
  if (const int st = ready_device()) return st;
  hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(threads), lds_bytes, stream, p);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(MI355X_FP8_ELAUNCH, "tiled kernel launch: %s", hipGetErrorString(e));
  if (EPI == kEpiPartial) {
    const long quads = (long)p.M * ((p.N + 3) / 4);
    hipLaunchKernelGGL(splitk_finalize_kernel, dim3((unsigned)((quads + 255) / 256)), dim3(256), 0, stream, p);
    e = hipGetLastError();
    if (e != hipSuccess) return fail(MI355X_FP8_ELAUNCH, "split-K finalize launch: %s", hipGetErrorString(e));
  }
  return MI355X_FP8_OK;
}

template <int BM, int BN, int WAVES_M, int WAVES_N, bool STREAM_B, bool DEEP = false>
int launch_tiled_epilogue(const GemmParams& p, hipStream_t s) {
  // 256x128 tiles have the LDS for loads three steps ahead (3 A + 4 B stages = 160 KB): worth 6-10 % where
  // the operands come from HBM rather than the memory-side cache (M=1024, N=K=8192 cold: 65.9 -> 60.5 us;
  // K=28672: 220 -> 199 us). The 64x256 tile measured 1-3 % slower that way and stays at two.
  constexpr int D = DEEP || (BM == 256 && BN == 128) ? 3 : kDefaultDist;
  const bool ktail = p.K % kStepK;
  if (p.splits > 1)
    return ktail ? launch_tiled<BM, BN, WAVES_M, WAVES_N, true, kEpiPartial, false, false, D, STREAM_B>(p, s)
                 : launch_tiled<BM, BN, WAVES_M, WAVES_N, false, kEpiPartial, false, false, D, STREAM_B>(p, s);
  if (p.bias)
    return ktail ? launch_tiled<BM, BN, WAVES_M, WAVES_N, true, kEpiBias, false, false, D, STREAM_B>(p, s)
                 : launch_tiled<BM, BN, WAVES_M, WAVES_N, false, kEpiBias, false, false, D, STREAM_B>(p, s);
  return ktail ? launch_tiled<BM, BN, WAVES_M, WAVES_N, true, kEpiPlain, false, false, D, STREAM_B>(p, s)
               : launch_tiled<BM, BN, WAVES_M, WAVES_N, false, kEpiPlain, false, false, D, STREAM_B>(p, s);
}

template <int BM, int BN, int WAVES_M, int WAVES_N, bool MAY_STREAM, bool DEEP = false>
int launch_tiled_config(const GemmParams& p, hipStream_t s) {
  if constexpr (MAY_STREAM) {
    if ((p.M + BM - 1) / BM <= stream_tile_rows(BM, BN))
      return launch_tiled_epilogue<BM, BN, WAVES_M, WAVES_N, true, DEEP>(p, s);
  }
  return launch_tiled_epilogue<BM, BN, WAVES_M, WAVES_N, false, DEEP>(p, s);
}
}  // namespace

// The seven tile configurations of the plain tiled kernel, each behind a function of its own: a unit
// of a build in parts defines one of them, the main unit of such a build none, a single-unit build all.
#if !defined(MI355X_SPLIT_MAIN)
#define MI355X_DEFINE_TILED_PART(k, ...)                                                             \
  int mi355x_shared::tiled_config_##k(const GemmParams& p, hipStream_t stream) { return launch_tiled_config<__VA_ARGS__>(p, stream); }
#if !defined(MI355X_TILED_PART) || MI355X_TILED_PART == 0
MI355X_DEFINE_TILED_PART(0, 256, 256, 2, 2, true)
#endif
#if !defined(MI355X_TILED_PART) || MI355X_TILED_PART == 1
MI355X_DEFINE_TILED_PART(1, 128, 128, 2, 2, true)
#endif
#if !defined(MI355X_TILED_PART) || MI355X_TILED_PART == 2
MI355X_DEFINE_TILED_PART(2, 256, 128, 2, 2, true)
#endif
#if !defined(MI355X_TILED_PART) || MI355X_TILED_PART == 3
MI355X_DEFINE_TILED_PART(3, 64, 256, 1, 4, true)
#endif
#if !defined(MI355X_TILED_PART) || MI355X_TILED_PART == 4
MI355X_DEFINE_TILED_PART(4, 128, 256, 2, 2, true)
#endif
#if !defined(MI355X_TILED_PART) || MI355X_TILED_PART == 5
MI355X_DEFINE_TILED_PART(5, 192, 256, 2, 2, true)
#endif
#if !defined(MI355X_TILED_PART) || MI355X_TILED_PART == 6
MI355X_DEFINE_TILED_PART(6, 128, 128, 2, 2, false, true)  // (never with the streaming policy)
#endif
#undef MI355X_DEFINE_TILED_PART
#endif

#if !defined(MI355X_TILED_PART)  // (everything from here on belongs to the main unit)
namespace {
template <int MT, int NTW, int DEPTH, int KW>
int launch_skinny(const GemmParams& p, hipStream_t stream) {
  constexpr size_t lds_bytes = (size_t)KW * (NTW + MT) * 16 * kStepK;
  static_assert(lds_bytes <= 160 * 1024, "transpose buffers must fit the 160 KB LDS");
  constexpr auto kern = gemm_skinny_kernel<MT, NTW, DEPTH, KW>;
  (void)LdsLimit<kern, lds_bytes>::registered;
  if (const int st = ready_device()) return st;
  const unsigned grid = (unsigned)((p.N + 16 * NTW - 1) / (16 * NTW));
  hipLaunchKernelGGL(kern, dim3(grid), dim3(KW * 64), lds_bytes, stream, p);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(MI355X_FP8_ELAUNCH, "skinny kernel launch: %s", hipGetErrorString(e));
  return MI355X_FP8_OK;
}

// ---- built-in scratch of the entry point that allocates nothing
// Split-K plans park their fp32 partial sums in device memory between the two launches. Callers
// that cannot bring a workspace (HIP graph capture, serving loops that may not allocate) get this
// array instead: every device the library is loaded on holds its own copy until the process
// ends. In host code the array's name is only a handle for the symbol look-up in setup_device();
// kernels, fills and copies take the per-device address that look-up returns.
constexpr size_t kScratchBytes = (size_t)MI355X_FP8_NOALLOC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[kScratchBytes];

// Sets the current device `dev` up: checks its shape, raises the dynamic-LDS limit of every
// registered kernel on it and looks up the address of its copy of `scratch`. None of this is an
// enqueue, so it belongs in front of any graph capture: mi355x_fp8_rowwise_init() does it by name,
// and a first call on a device that was never initialised does it on the way.
int setup_device(int dev) {
  if (g_device_state[dev].load(std::memory_order_acquire) < 0)
    return fail(MI355X_FP8_ENOTSUP, "device %d does not report the %d compute units these kernels are scheduled for "
                "(a partitioned mode or another part)", dev, kNumCu);
  if (mi355x_shared::lds_table_overflow) return fail(MI355X_FP8_ELAUNCH, "kernel table overflow (more than %d instantiations)", mi355x_shared::kMaxLdsKernels);
  if (const int st = check_device_shape(dev)) {
    if (st == MI355X_FP8_ENOTSUP) g_device_state[dev].store(-1, std::memory_order_release);
    return st;
  }
  for (int i = 0; i < mi355x_shared::num_lds_kernels; ++i) {
    const hipError_t e = hipFuncSetAttribute(mi355x_shared::lds_kernels[i].kernel, hipFuncAttributeMaxDynamicSharedMemorySize,
                                             (int)mi355x_shared::lds_kernels[i].lds_bytes);
    if (e != hipSuccess) return fail(MI355X_FP8_ELAUNCH, "hipFuncSetAttribute: %s", hipGetErrorString(e));
  }
  void* ptr = nullptr;
  const hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
  if (e != hipSuccess || !ptr) return fail(MI355X_FP8_ELAUNCH, "hipGetSymbolAddress(scratch): %s", hipGetErrorString(e));
  g_scratch_ptr[dev].store(ptr, std::memory_order_release);  // every thread finds the same address
  g_device_state[dev].store(1, std::memory_order_release);
  return MI355X_FP8_OK;
}

// Address of the current device's copy of `scratch`.
int scratch_of_current_device(void** out) {
  int dev = 0;
  if (const int st = ready_device(&dev)) return st;
  *out = g_scratch_ptr[dev].load(std::memory_order_acquire);
  return MI355X_FP8_OK;
}

// The persistent skinny kernel takes N a multiple of 16 and K of 2048 up to 8192 with M <= 16,
// and K = 4096 with M <= 32. (Two blocks of A in registers leave room for two steps of B in
// flight per wave. At K = 4096 that is a whole tile ahead and the form wins: M=32, N=8192 9.9 us
// against 11.4 us for the one-tile kernel. At K = 8192 it is half a tile and loses, 20.6 against
// 17.9 us; four steps in flight do not fit the 128 registers of a 16-wave workgroup.)
inline bool persistent_skinny_fits(int64_t M, int64_t N, int64_t K) {
  if (N % 16 != 0 || K % (kPersistWaves * kStepK) != 0) return false;
  const int64_t spw = K / (kPersistWaves * kStepK);
  return (M <= 16 && spw <= 4) || (M <= 32 && spw == 2);
}

template <int SPW, int MT, int LAG, bool VEC>
int launch_skinny_persistent(const GemmParams& p, hipStream_t stream) {
  constexpr size_t lds_bytes = persistent_lds_bytes(MT);
  constexpr auto kern = gemm_skinny_persistent_kernel<SPW, MT, LAG, VEC>;
  (void)LdsLimit<kern, lds_bytes>::registered;
  if (const int st = ready_device()) return st;
  const long ntiles = p.N / 16;
  const unsigned grid = (unsigned)(ntiles < kNumCu ? ntiles : kNumCu);
  GemmParams q = p;
  q.tiles_m = (int)(ntiles / grid);  // tiles per workgroup ...
  q.tiles_n = (int)(ntiles % grid);  // ... and how many workgroups take one more
  hipLaunchKernelGGL(kern, dim3(grid), dim3(kPersistWaves * 64), lds_bytes, stream, q);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(MI355X_FP8_ELAUNCH, "persistent skinny kernel launch: %s", hipGetErrorString(e));
  return MI355X_FP8_OK;
}

template <int SPW, bool VEC, bool KTAIL, bool HAS_BIAS>
int launch_skinny_pair(const GemmParams& p, hipStream_t stream) {
  constexpr size_t lds_bytes = pair_lds_bytes(SPW);
  static_assert(lds_bytes <= 160 * 1024, "A's steps, the transpose buffers and the partial results must fit the LDS");
  constexpr auto kern = gemm_skinny_pair_kernel<SPW, VEC, KTAIL, HAS_BIAS>;
  (void)LdsLimit<kern, lds_bytes>::registered;
  if (const int st = ready_device()) return st;
  const long ntiles = p.N / 16;
  const unsigned grid = (unsigned)(ntiles < kNumCu ? ntiles : kNumCu);
  GemmParams q = p;
  q.tiles_m = (int)(ntiles / grid);  // tiles per workgroup ...
  q.tiles_n = (int)(ntiles % grid);  // ... and how many workgroups take one more
  hipLaunchKernelGGL(kern, dim3(grid), dim3(kPersistWaves * 64), lds_bytes, stream, q);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(MI355X_FP8_ELAUNCH, "pair skinny kernel launch: %s", hipGetErrorString(e));
  return MI355X_FP8_OK;
}

template <bool VEC, bool KTAIL, bool HAS_BIAS>
int launch_skinny_pair_steps(const GemmParams& p, hipStream_t s) {
  const int steps = (p.K + kStepK - 1) / kStepK;
  const int spw = (steps + kPersistWaves - 1) / kPersistWaves;
  switch (spw) {
    case 1: return launch_skinny_pair<1, VEC, KTAIL, HAS_BIAS>(p, s);
    case 2: return launch_skinny_pair<2, VEC, KTAIL, HAS_BIAS>(p, s);
    case 3: return launch_skinny_pair<3, VEC, KTAIL, HAS_BIAS>(p, s);
    default: return launch_skinny_pair<4, VEC, KTAIL, HAS_BIAS>(p, s);
  }
}
template <bool VEC>
int launch_skinny_pair_form(const GemmParams& p, hipStream_t s) {
  const bool ktail = p.K % (kPersistWaves * kStepK) != 0;
  if (p.bias) return ktail ? launch_skinny_pair_steps<VEC, true, true>(p, s) : launch_skinny_pair_steps<VEC, false, true>(p, s);
  return ktail ? launch_skinny_pair_steps<VEC, true, false>(p, s) : launch_skinny_pair_steps<VEC, false, false>(p, s);
}

template <bool VEC>
int launch_skinny_persistent_steps(const GemmParams& p, hipStream_t s) {
  const int spw = p.K / (kPersistWaves * kStepK);
  if (p.M > 16) return launch_skinny_persistent<2, 2, 2, VEC>(p, s);
  switch (spw) {
    case 1: return launch_skinny_persistent<1, 1, 1, VEC>(p, s);
    case 2: return launch_skinny_persistent<2, 1, 2, VEC>(p, s);
    case 3: return launch_skinny_persistent<3, 1, 3, VEC>(p, s);
    default: return launch_skinny_persistent<4, 1, 4, VEC>(p, s);
  }
}

template <int MB, int NB>
int launch_narrow(const GemmParams& p, hipStream_t stream) {
  constexpr size_t lds_bytes = narrow_lds_bytes(MB, NB);
  constexpr auto kern = gemm_narrow_kernel<MB, NB>;
  (void)LdsLimit<kern, lds_bytes>::registered;
  if (const int st = ready_device()) return st;
  const unsigned row_blocks = (unsigned)((p.M + 32 * MB - 1) / (32 * MB));
  GemmParams q = p;
  q.tiles_n = row_blocks == 1 ? narrow_tile_cols(p.N) : 32 * NB;  // columns per tile
  if (q.tiles_n > 32 * NB) return fail(MI355X_FP8_ELAUNCH, "narrow-tile form and tile width disagree");
  const unsigned tiles = (unsigned)((p.N + q.tiles_n - 1) / q.tiles_n);
  // (with row blocks the kernel deals tiles out per XCD: whole rounds of the XCDs)
  const unsigned grid = row_blocks == 1 ? tiles : (tiles + kNumXcd - 1) / kNumXcd * kNumXcd * row_blocks;
  hipLaunchKernelGGL(kern, dim3(grid), dim3(512), lds_bytes, stream, q);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(MI355X_FP8_ELAUNCH, "narrow-tile kernel launch: %s", hipGetErrorString(e));
  return MI355X_FP8_OK;
}

// the narrow-tile instantiation for a shape
int launch_narrow_for(const GemmParams& p, hipStream_t s) {
  const NarrowForm f = narrow_form(p.M, p.N);
  if (f.mb == 1) return f.nb == 1 ? launch_narrow<1, 1>(p, s) : launch_narrow<1, 2>(p, s);
  return f.nb == 1 ? launch_narrow<2, 1>(p, s) : launch_narrow<2, 2>(p, s);
}

int run_gemm(const void* a, const void* b, const float* a_scale, const float* b_scale, const void* bias, void* c,
             int out_type, int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb, int64_t ldc, void* workspace,
             size_t workspace_bytes, int variant, void* stream, unsigned long long* stamps);

}  // namespace

extern "C" {

int mi355x_fp8_rowwise_abi_version(void) { return MI355X_FP8_ABI_VERSION; }

int mi355x_fp8_rowwise_init(void) { return ready_device(); }

const char* mi355x_fp8_rowwise_last_error(void) { return mi355x_shared::err; }

int mi355x_fp8_rowwise_select_variant(int64_t M, int64_t N, int64_t K) {
  const int st = check_shape(M, N, K);
  if (st != MI355X_FP8_OK) return st;
  if (K % 16 != 0) return MI355X_FP8_VARIANT_GENERIC;
  // M <= 64: the streaming kernel, unless a tiled plan (64- or 128-row tiles that stream B, split
  // K where the tiles are few) is expected to beat it: from two 16-row blocks of A up on most
  // shapes, with one block on the longest weight panels. Up to 8 rows the streaming kernel was
  // behind on one kind of shape only, few columns with very long rows, where a handful of workgroups
  // each stream a long tile and split tiles put the whole chip to work (8 x 1024 x 28672: 16.2 us
  // against 14.5); there a tiled plan has to be expected ahead by a tenth to be taken.
  // (above 64 rows the family's only member is the narrow-tile kernel in row blocks, where it fits)
  if (M > kSkinnyMaxM && !narrow_fits(M, N, K)) return MI355X_FP8_VARIANT_TILED;
  const float margin = M <= 8 ? 0.9f : 1.0f;
  return plan_tiled(M, N, K, -1, 0, kMaxSplits).cost_us < margin * skinny_cost_us(M, N, K) ? MI355X_FP8_VARIANT_TILED
                                                                                          : MI355X_FP8_VARIANT_SKINNY;
}

size_t mi355x_fp8_rowwise_workspace_bytes(int64_t M, int64_t N, int64_t K, int variant) {
  if (check_shape(M, N, K) != MI355X_FP8_OK) return 0;
  if ((variant & 0xff) == MI355X_FP8_VARIANT_AUTO)
    variant = (variant & ~0xff) | mi355x_fp8_rowwise_select_variant(M, N, K);
  // (the skinny kernels reduce on chip, the generic kernel does not split)
  if ((variant & 0xff) != MI355X_FP8_VARIANT_TILED || K % 16 != 0) return 0;
  const TiledPlan plan = plan_from_variant(M, N, K, variant, kMaxSplits);
  return plan.splits > 1 ? (size_t)plan.splits * (size_t)M * (size_t)N * sizeof(float) : 0;
}

int mi355x_fp8_rowwise_gemm(const void* a, const void* b, const float* a_scale, const float* b_scale,
                            const void* bias, void* c, int64_t M, int64_t N, int64_t K, int64_t lda,
                            int64_t ldb, int64_t ldc, void* workspace, size_t workspace_bytes,
                            int variant, void* stream) {
  return mi355x_fp8_rowwise_gemm_ex(a, b, a_scale, b_scale, bias, c, MI355X_FP8_OUT_BF16, M, N, K, lda, ldb, ldc,
                                    workspace, workspace_bytes, variant, stream);
}

int mi355x_fp8_rowwise_gemm_ex(const void* a, const void* b, const float* a_scale, const float* b_scale,
                               const void* bias, void* c, int out_type, int64_t M, int64_t N, int64_t K,
                               int64_t lda, int64_t ldb, int64_t ldc, void* workspace, size_t workspace_bytes,
                               int variant, void* stream) {
  return run_gemm(a, b, a_scale, b_scale, bias, c, out_type, M, N, K, lda, ldb, ldc, workspace, workspace_bytes, variant,
                  stream, nullptr);
}

int mi355x_fp8_rowwise_gemm_stamped(const void* a, const void* b, const float* a_scale, const float* b_scale,
                                    const void* bias, void* c, int64_t M, int64_t N, int64_t K, int64_t lda,
                                    int64_t ldb, int64_t ldc, void* workspace, size_t workspace_bytes, int variant,
                                    uint64_t* stamps, size_t stamp_entries, void* stream) {
  if (!stamps || stamp_entries < (size_t)MI355X_FP8_STAMP_ENTRIES)
    return fail(MI355X_FP8_EINVAL, "stamps must hold %d entries (got %zu)", MI355X_FP8_STAMP_ENTRIES, stamps ? stamp_entries : (size_t)0);
  if (reinterpret_cast<uintptr_t>(stamps) & 7) return fail(MI355X_FP8_EINVAL, "misaligned stamps pointer");
  return run_gemm(a, b, a_scale, b_scale, bias, c, MI355X_FP8_OUT_BF16, M, N, K, lda, ldb, ldc, workspace, workspace_bytes,
                  variant, stream, reinterpret_cast<unsigned long long*>(stamps));
}

}  // extern "C"

namespace {
int run_gemm(const void* a, const void* b, const float* a_scale, const float* b_scale, const void* bias, void* c,
             int out_type, int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb, int64_t ldc, void* workspace,
             size_t workspace_bytes, int variant, void* stream, unsigned long long* stamps) {
  if (out_type != MI355X_FP8_OUT_BF16 && out_type != MI355X_FP8_OUT_F16)
    return fail(MI355X_FP8_EINVAL, "unknown output type %d", out_type);
  int st = check_shape(M, N, K);
  if (st != MI355X_FP8_OK) return st;
  if (!a || !b || !a_scale || !b_scale || !c) return fail(MI355X_FP8_EINVAL, "null operand pointer");
  if (lda < K || ldb < K || ldc < N) return fail(MI355X_FP8_EINVAL, "leading dimension smaller than the row length");
  if ((reinterpret_cast<uintptr_t>(a_scale) & 3) || (reinterpret_cast<uintptr_t>(b_scale) & 3) ||
      (reinterpret_cast<uintptr_t>(c) & 1) || (reinterpret_cast<uintptr_t>(bias) & 1))
    return fail(MI355X_FP8_EINVAL, "misaligned scale, bias or output pointer");
  if (variant < 0 || (variant >> 24) || ((variant >> 8) & 0xff) > kNumTileConfigs)
    return fail(MI355X_FP8_EINVAL, "unknown variant 0x%x", variant);
  const int plan_bits = variant & ~0xff;
  variant &= 0xff;
  // What the MFMA families ask of the operands; the generic family takes whatever is left, and AUTO
  // sends it there.
  const char* unfit = nullptr;
  if (K % 16 != 0) unfit = "K must be a multiple of 16";
  else if (lda % 16 || ldb % 16) unfit = "lda and ldb must be multiples of 16";
  else if ((reinterpret_cast<uintptr_t>(a) & 15) || (reinterpret_cast<uintptr_t>(b) & 15)) unfit = "a and b must be 16-byte aligned";
  // (a tile's rows are addressed with 32-bit byte offsets that must stay below 2^31)
  else if (lda * 256 > (int64_t)INT32_MAX || ldb * 256 > (int64_t)INT32_MAX || ldc * 512 > (int64_t)INT32_MAX)
    unfit = "leading dimension too large";
  if (unfit && variant == MI355X_FP8_VARIANT_AUTO) variant = MI355X_FP8_VARIANT_GENERIC;
  if (unfit && variant != MI355X_FP8_VARIANT_GENERIC)
    return fail(MI355X_FP8_ENOTSUP, "%s for this kernel family (lda %lld, ldb %lld, ldc %lld, K %lld); the generic family or "
                "the automatic choice takes such operands", unfit, (long long)lda, (long long)ldb, (long long)ldc, (long long)K);
  if (variant == MI355X_FP8_VARIANT_GENERIC && stamps)
    return fail(MI355X_FP8_ENOTSUP, "the stamped entry point runs the tiled family only");
  if (variant == MI355X_FP8_VARIANT_AUTO) {
    variant = mi355x_fp8_rowwise_select_variant(M, N, K);
    if (variant == MI355X_FP8_VARIANT_TILED && (M <= kSkinnyMaxM || narrow_fits(M, N, K))) {
      // the choice assumed the plan's workspace; without it the plan changes and may lose
      const TiledPlan plan = plan_from_variant(M, N, K, plan_bits, kMaxSplits);
      const size_t need = plan.splits > 1 ? (size_t)plan.splits * M * N * sizeof(float) : 0;
      if (need && (!workspace || workspace_bytes < need) &&
          plan_from_variant(M, N, K, plan_bits, 1).cost_us >= skinny_cost_us(M, N, K))
        variant = MI355X_FP8_VARIANT_SKINNY;
    }
  }
  if (variant == MI355X_FP8_VARIANT_SKINNY && M > kSkinnyMaxM && !narrow_fits(M, N, K))
    return fail(MI355X_FP8_ENOTSUP,
                "skinny variant handles M <= %d, and M <= %d where 64x64 tiles give every CU at most one (got %lldx%lld)",
                kSkinnyMaxM, kNarrowMaxM, (long long)M, (long long)N);

  GemmParams p;
  p.a = (const uint8_t*)a; p.b = (const uint8_t*)b;
  p.a_scale = a_scale; p.b_scale = b_scale;
  p.bias = (const uint16_t*)bias; p.c = (uint16_t*)c;
  p.M = (int)M; p.N = (int)N; p.K = (int)K;
  p.lda = lda; p.ldb = ldb; p.ldc = ldc;
  p.tiles_m = p.tiles_n = 0; p.group_m = 1;
  p.splits = 1; p.steps_per_split = k_steps_of(K); p.partial = nullptr;
  p.m_sizes = nullptr; p.groups = 0; p.out_f16 = out_type == MI355X_FP8_OUT_F16;
  p.div_tiles_mul = p.div_tiles_shift = p.div_group_mul = p.div_group_shift = 0; p.stamps = stamps;
  hipStream_t s = (hipStream_t)stream;

  switch (variant) {
    case MI355X_FP8_VARIANT_TILED:
      {
        // A caller that brought no (or too little) workspace gets the best plan that needs none,
        // unless it asked for a split factor by name.
        TiledPlan plan = plan_from_variant(M, N, K, plan_bits, kMaxSplits);
        const size_t need = plan.splits > 1 ? (size_t)plan.splits * M * N * sizeof(float) : 0;
        if (need && (!workspace || workspace_bytes < need)) {
          if ((plan_bits >> 16) & 0xff)
            return fail(MI355X_FP8_EINVAL, "split-K factor %d needs %zu bytes of workspace (got %zu)",
                        plan.splits, need, workspace ? workspace_bytes : (size_t)0);
          // the cheapest plan whose partial planes fit what the caller brought (none: the unsplit plans)
          const size_t plane = (size_t)M * (size_t)N * sizeof(float);
          const size_t fit = workspace ? workspace_bytes / plane : 0;
          plan = plan_from_variant(M, N, K, plan_bits, fit < 1 ? 1 : fit > (size_t)kMaxSplits ? kMaxSplits : (int)fit);
        }
        // (the partial sums of a tile are addressed with 32-bit byte offsets that must stay below 2^31)
        if (plan.splits > 1 && N * 512 > (int64_t)INT32_MAX) plan = plan_from_variant(M, N, K, plan_bits & 0xff00, 1);
        if (plan.splits > 1 && (reinterpret_cast<uintptr_t>(workspace) & 15))
          return fail(MI355X_FP8_EINVAL, "workspace must be 16-byte aligned");
        p.splits = plan.splits;
        p.steps_per_split = plan.steps_per_split;
        p.partial = plan.splits > 1 ? (float*)workspace : nullptr;
        switch (plan.config) {
          case 0: return mi355x_shared::tiled_config_0(p, s);
          case 1: return mi355x_shared::tiled_config_1(p, s);
          case 2: return mi355x_shared::tiled_config_2(p, s);
          case 3: return mi355x_shared::tiled_config_3(p, s);
          case 4: return mi355x_shared::tiled_config_4(p, s);
          case 5: return mi355x_shared::tiled_config_5(p, s);
          case 6: return mi355x_shared::tiled_config_6(p, s);
          default: return fail(MI355X_FP8_EINVAL, "unknown tile configuration %d", plan.config);
        }
      }
    case MI355X_FP8_VARIANT_SKINNY:
      // 16-row blocks of A | B tiles per wave | steps in flight per wave (sized to 128 VGPRs) | waves.
      // (Measured alternatives at M = 16: two B tiles per wave with 4, 6 or 8 steps in flight 17.8-19.9 us,
      // four waves 14.7-15.0 us, six steps in flight 16.4 us, against 14.4 us for this one.)
      if (plan_bits & MI355X_FP8_SKINNY_NARROW) {
        if (!narrow_fits(M, N, K))
          return fail(MI355X_FP8_ENOTSUP,
                      "the narrow-tile kernel takes M <= %d, and M <= %d where 64x64 tiles give every CU at most one (got %lldx%lld)",
                      kSkinnyMaxM, kNarrowMaxM, (long long)M, (long long)N);
        return launch_narrow_for(p, s);
      }
      if (M > kSkinnyMaxM) {
        if (plan_bits & MI355X_FP8_SKINNY_ONE_TILE)
          return fail(MI355X_FP8_ENOTSUP, "the one-tile-per-workgroup form takes M <= %d (got M=%lld)", kSkinnyMaxM, (long long)M);
        return launch_narrow_for(p, s);
      }
      if (!(plan_bits & (MI355X_FP8_SKINNY_ONE_TILE | MI355X_FP8_SKINNY_RESIDENT)) && narrow_preferred(M, N, K))
        return launch_narrow_for(p, s);
      if ((plan_bits & MI355X_FP8_SKINNY_RESIDENT) && !pair_skinny_fits(M, N, K) && !persistent_skinny_fits(M, N, K))
        return fail(MI355X_FP8_ENOTSUP, "neither form that keeps A on chip takes %lldx%lldx%lld", (long long)M, (long long)N, (long long)K);
      if ((pair_skinny_fits(M, N, K) || persistent_skinny_fits(M, N, K)) && !(plan_bits & MI355X_FP8_SKINNY_ONE_TILE)) {
        // 16-byte loads of b_scale, 8-byte loads of bias and 8-byte stores of C when everything is aligned for them
        const bool vec = (reinterpret_cast<uintptr_t>(b_scale) & 15) == 0 && (reinterpret_cast<uintptr_t>(bias) & 7) == 0 &&
                         (reinterpret_cast<uintptr_t>(c) & 7) == 0 && (ldc & 3) == 0;
        // (pinned, the forms that keep A on chip run wherever they fit; left to the library, where they are expected ahead)
        const bool resident = (plan_bits & MI355X_FP8_SKINNY_RESIDENT) || skinny_streaming_choice(M, N, K) != kStreamOneTile;
        // (the pair kernel addresses a workgroup's rows of B with 32-bit offsets below 2^31)
        if (resident && pair_skinny_fits(M, N, K) && ldb * 32 <= (int64_t)INT32_MAX)
          return vec ? launch_skinny_pair_form<true>(p, s) : launch_skinny_pair_form<false>(p, s);
        if (resident && persistent_skinny_fits(M, N, K))
          return vec ? launch_skinny_persistent_steps<true>(p, s) : launch_skinny_persistent_steps<false>(p, s);
      }
      if (M <= 16) return launch_skinny<1, 1, 4, 8>(p, s);
      if (M <= 32) return launch_skinny<2, 1, 2, 8>(p, s);
      if (M <= 48) return launch_skinny<3, 1, 2, 8>(p, s);
      return launch_skinny<4, 2, 2, 8>(p, s);  // 32 rows of B per workgroup: A passes L1 half as often
    case MI355X_FP8_VARIANT_GENERIC: {
      if (const int gs = ready_device()) return gs;
      const dim3 grid((unsigned)((N + kGenericTile - 1) / kGenericTile), (unsigned)((M + kGenericTile - 1) / kGenericTile));
      if (grid.y > 65535) return fail(MI355X_FP8_ENOTSUP, "the generic family takes M <= %d", 65535 * kGenericTile);
      hipLaunchKernelGGL(gemm_generic_kernel, grid, dim3(256), 0, s, p);
      const hipError_t e = hipGetLastError();
      if (e != hipSuccess) return fail(MI355X_FP8_ELAUNCH, "generic kernel launch: %s", hipGetErrorString(e));
      return MI355X_FP8_OK;
    }
    default:
      return fail(MI355X_FP8_EINVAL, "unknown variant %d", variant);
  }
}
}  // namespace

extern "C" {

int mi355x_fp8_rowwise_gemm_noalloc(const void* a, const void* b, const float* a_scale, const float* b_scale,
                                    const void* bias, void* c, int64_t M, int64_t N, int64_t K, int64_t lda,
                                    int64_t ldb, int64_t ldc, int variant, void* stream) {
  const int st = check_shape(M, N, K);
  if (st != MI355X_FP8_OK) return st;
  if (variant < 0 || (variant >> 24) || ((variant >> 8) & 0xff) > kNumTileConfigs)
    return fail(MI355X_FP8_EINVAL, "unknown variant 0x%x", variant);
  // host arithmetic only up to here: an oversized request is turned away before any device call
  const size_t need = mi355x_fp8_rowwise_workspace_bytes(M, N, K, variant);
  // A plan the buffer cannot hold is refused only when the caller named its split factor; left to
  // the library, the call runs the cheapest plan whose partial sums fit the buffer, as the workspace
  // form does with a workspace that is too small.
  if (need > kScratchBytes && ((variant >> 16) & 0xff))
    return fail(MI355X_FP8_ENOTSUP,
                "split-K factor %d on %lldx%lldx%lld needs %zu bytes of scratch, the built-in buffer holds %zu; "
                "call mi355x_fp8_rowwise_gemm with a workspace of that size instead",
                (variant >> 16) & 0xff, (long long)M, (long long)N, (long long)K, need, kScratchBytes);
  void* ws = nullptr;
  if (need) {
    if (const int ss = scratch_of_current_device(&ws)) return ss;
  }
  // Nothing in the buffer has to start at zero: every split stores its whole plane of partial sums
  // before the finalize kernel (stream-ordered behind it) reads any of it.
  return mi355x_fp8_rowwise_gemm_ex(a, b, a_scale, b_scale, bias, c, MI355X_FP8_OUT_BF16, M, N, K, lda, ldb, ldc,
                                    ws, need ? kScratchBytes : 0, variant, stream);
}

int mi355x_fp8_rowwise_grouped_gemm(const void* a, const void* b, const float* a_scale, const float* b_scale,
                                    const int32_t* m_sizes, void* c, int64_t G, int64_t M, int64_t N,
                                    int64_t K, int64_t lda, int64_t ldb, int64_t ldc, int tile_config,
                                    void* stream) {
  int st = check_shape(M, N, K);
  if (st == MI355X_FP8_OK) st = check_fast_shape(K);
  if (st != MI355X_FP8_OK) return st;
  if (G < 1 || G > 65536) return fail(MI355X_FP8_EINVAL, "G must be in 1..65536 (got %lld)", (long long)G);
  if (G * N > INT32_MAX) return fail(MI355X_FP8_ENOTSUP, "G*N exceeds 2^31-1");
  if (!a || !b || !a_scale || !b_scale || !m_sizes || !c) return fail(MI355X_FP8_EINVAL, "null operand pointer");
  if (lda < K || ldb < K || ldc < N) return fail(MI355X_FP8_EINVAL, "leading dimension smaller than the row length");
  if (lda % 16 || ldb % 16) return fail(MI355X_FP8_ENOTSUP, "lda and ldb must be multiples of 16");
  if ((reinterpret_cast<uintptr_t>(a) & 15) || (reinterpret_cast<uintptr_t>(b) & 15))
    return fail(MI355X_FP8_ENOTSUP, "a and b must be 16-byte aligned");
  if ((reinterpret_cast<uintptr_t>(a_scale) & 3) || (reinterpret_cast<uintptr_t>(b_scale) & 3) ||
      (reinterpret_cast<uintptr_t>(c) & 1) || (reinterpret_cast<uintptr_t>(m_sizes) & 3))
    return fail(MI355X_FP8_EINVAL, "misaligned scale, size or output pointer");
  // (a tile's rows are addressed with 32-bit byte offsets that must stay below 2^31)
  if (lda * 256 > (int64_t)INT32_MAX || ldb * 256 > (int64_t)INT32_MAX || ldc * 512 > (int64_t)INT32_MAX)
    return fail(MI355X_FP8_ENOTSUP, "leading dimension too large");
  if (tile_config < -1 || tile_config >= kNumGroupedTileConfigs)
    return fail(MI355X_FP8_EINVAL, "unknown tile configuration %d", tile_config);

  GemmParams p;
  p.a = (const uint8_t*)a; p.b = (const uint8_t*)b;
  p.a_scale = a_scale; p.b_scale = b_scale;
  p.bias = nullptr; p.c = (uint16_t*)c;
  p.M = (int)M; p.N = (int)N; p.K = (int)K;
  p.lda = lda; p.ldb = ldb; p.ldc = ldc;
  p.tiles_m = p.tiles_n = 0; p.group_m = 1;
  p.splits = 1; p.steps_per_split = k_steps_of(K); p.partial = nullptr;
  p.m_sizes = m_sizes; p.groups = (int)G; p.out_f16 = 0;
  p.div_tiles_mul = p.div_tiles_shift = p.div_group_mul = p.div_group_shift = 0; p.stamps = nullptr;
  hipStream_t s = (hipStream_t)stream;
  // Large tiles when an average group fills most of one and there are enough of them for every
  // CU, small tiles otherwise (the group sizes themselves are on the device; M / G is what the
  // host knows). Where 256x256 tiles are too few and 256x128 tiles come to about one round of workgroups,
  // those, on rows long enough for their deeper ring to pay (measured, equal groups: G = 4, M = 1024,
  // N = K = 8192 78.8 -> 60.9 us; G = 2 ... 16, M = 4096, N = 2048, K = 7168 52-65 -> 49-60; at K = 2048
  // they are 1-3 % behind the small tiles).
  if (tile_config < 0) {
    const bool rows_fill = M / G >= 192;
    const int64_t tiles_256 = (M / 256) * (N / 256), tiles_128 = (M / 256) * (N / 128);
    tile_config = rows_fill && tiles_256 >= 192 ? 0 : rows_fill && tiles_128 >= 192 && tiles_128 <= 288 && K >= 4096 ? 2 : 1;
  }
  const bool ktail = K % kStepK;
  if (tile_config == 0)
    return ktail ? launch_tiled<256, 256, 2, 2, true, kEpiPlain, true>(p, s)
                 : launch_tiled<256, 256, 2, 2, false, kEpiPlain, true>(p, s);
  if (tile_config == 2)
    return ktail ? launch_tiled<256, 128, 2, 2, true, kEpiPlain, true, false, 3>(p, s)
                 : launch_tiled<256, 128, 2, 2, false, kEpiPlain, true, false, 3>(p, s);
  return ktail ? launch_tiled<128, 128, 2, 2, true, kEpiPlain, true>(p, s)
               : launch_tiled<128, 128, 2, 2, false, kEpiPlain, true>(p, s);
}

int mi355x_fp8_blockwise_gemm(const void* a, const void* b, const float* a_scale, const float* b_scale,
                              void* c, int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb,
                              int64_t ldc, void* stream) {
  int st = check_shape(M, N, K);
  if (st == MI355X_FP8_OK) st = check_fast_shape(K);
  if (st != MI355X_FP8_OK) return st;
  if (K > 256 * kStepK) return fail(MI355X_FP8_ENOTSUP, "block-scaled form handles K <= %d (got %lld)",
                                    256 * kStepK, (long long)K);
  if (!a || !b || !a_scale || !b_scale || !c) return fail(MI355X_FP8_EINVAL, "null operand pointer");
  if (lda < K || ldb < K || ldc < N) return fail(MI355X_FP8_EINVAL, "leading dimension smaller than the row length");
  if (lda % 16 || ldb % 16) return fail(MI355X_FP8_ENOTSUP, "lda and ldb must be multiples of 16");
  if ((reinterpret_cast<uintptr_t>(a) & 15) || (reinterpret_cast<uintptr_t>(b) & 15))
    return fail(MI355X_FP8_ENOTSUP, "a and b must be 16-byte aligned");
  if ((reinterpret_cast<uintptr_t>(a_scale) & 3) || (reinterpret_cast<uintptr_t>(b_scale) & 3) ||
      (reinterpret_cast<uintptr_t>(c) & 1))
    return fail(MI355X_FP8_EINVAL, "misaligned scale or output pointer");
  // (a tile's rows are addressed with 32-bit byte offsets that must stay below 2^31)
  if (lda * 256 > (int64_t)INT32_MAX || ldb * 256 > (int64_t)INT32_MAX || ldc * 512 > (int64_t)INT32_MAX)
    return fail(MI355X_FP8_ENOTSUP, "leading dimension too large");
  GemmParams p;
  p.a = (const uint8_t*)a; p.b = (const uint8_t*)b;
  p.a_scale = a_scale; p.b_scale = b_scale;
  p.bias = nullptr; p.c = (uint16_t*)c;
  p.M = (int)M; p.N = (int)N; p.K = (int)K;
  p.lda = lda; p.ldb = ldb; p.ldc = ldc;
  p.tiles_m = p.tiles_n = 0; p.group_m = 1;
  p.splits = 1; p.steps_per_split = k_steps_of(K); p.partial = nullptr;
  p.m_sizes = nullptr; p.groups = 0; p.out_f16 = 0;
  p.div_tiles_mul = p.div_tiles_shift = p.div_group_mul = p.div_group_shift = 0; p.stamps = nullptr;
  hipStream_t s = (hipStream_t)stream;
  // 128x128 tiles: with 256x128 tiles (64 more accumulators and 64 more partial products per
  // lane) the fold no longer fits the 256 registers VALU instructions can address
  return (K % kStepK) ? launch_tiled<128, 128, 2, 2, true, kEpiPlain, false, true>(p, s)
                      : launch_tiled<128, 128, 2, 2, false, kEpiPlain, false, true>(p, s);
}

namespace {
// Rows of at most 64 x 8 16-byte chunks are quantised by one wave each, kWaveRows rows per workgroup:
// the number of chunks a lane keeps in registers (4 or 8), or 0 for longer rows. (Measured, bf16 rows,
// workgroup per row -> wave per row: 16384 x 2048 quantiser 28.7 -> 19.9 us, RMSNorm form 40.8 -> 21.0,
// SiLU-mul form 49.0 -> 27.9; 65536 x 512 75 -> 27, 132 -> 29, 170 -> 32; eight rows per workgroup
// instead of four changed nothing.)
constexpr int kWaveRows = 4;
inline int row_chunks_per_lane(int64_t chunks) { return chunks <= 64 * 4 ? 4 : chunks <= 64 * 8 ? 8 : 0; }
// (bf16 rows of up to 1024 elements: two rounds per lane instead of four, of which at least two would be idle)
inline int bf16_row_chunks_per_lane(int64_t chunks) { return chunks <= 64 * 2 ? 2 : row_chunks_per_lane(chunks); }
}  // namespace

int mi355x_fp8_rowwise_quantize(const void* x, int src_type, void* xq, float* inv_scale, int64_t R,
                                int64_t K, int64_t ldx, int64_t ldq, void* stream) {
  if (!x || !xq || !inv_scale) return fail(MI355X_FP8_EINVAL, "null pointer");
  if (R < 1 || K < 1 || ldx < K || ldq < K) return fail(MI355X_FP8_EINVAL, "bad shape or leading dimension");
  if (R > INT32_MAX || K > INT32_MAX) return fail(MI355X_FP8_ENOTSUP, "dimension exceeds 2^31-1");
  hipStream_t s = (hipStream_t)stream;
  // source and destination rows that start 16-byte aligned and hold whole 16-byte source
  // chunks take the vector kernel
  const int esz = src_type == MI355X_FP8_SRC_BF16 ? 2 : 4;
  const int epv = 16 / esz;
  const bool vec = (reinterpret_cast<uintptr_t>(x) & 15) == 0 && (ldx * esz) % 16 == 0 && K % epv == 0 &&
                   (reinterpret_cast<uintptr_t>(xq) & 15) == 0 && ldq % 16 == 0;
  const bool long_row = K / epv > 8 * 256;  // more chunks than 256 lanes keep in registers
  const bool short_row = K / epv <= 4 * 256;  // (bf16 source: half the registers, more workgroups per CU)
  const int wave_cache = row_chunks_per_lane(K / epv);  // > 0: a wave per row, that many chunks per lane
  const unsigned wave_grid = (unsigned)((R + kWaveRows - 1) / kWaveRows);
  if (vec && src_type == MI355X_FP8_SRC_F32) {
    if (wave_cache) {
      auto kern = wave_cache == 4 ? quantize_rows_vec_kernel<float, 4, 64, kWaveRows> : quantize_rows_vec_kernel<float, 8, 64, kWaveRows>;
      hipLaunchKernelGGL(kern, dim3(wave_grid), dim3(64 * kWaveRows), 0, s, (const float*)x, (uint8_t*)xq, inv_scale, (int)K,
                         (long)ldx, (long)ldq, (long)R);
    } else {
      auto kern = long_row ? quantize_rows_vec_kernel<float, 8, 1024> : quantize_rows_vec_kernel<float, 8, 256>;
      hipLaunchKernelGGL(kern, dim3((unsigned)R), dim3(long_row ? 1024 : 256), 0, s, (const float*)x,
                         (uint8_t*)xq, inv_scale, (int)K, (long)ldx, (long)ldq, (long)R);
    }
  } else if (vec && src_type == MI355X_FP8_SRC_BF16) {
    // (A wave per row is the form for many rows. With few, a row spread over a workgroup's 256 lanes is back sooner:
    // 16 x 4096 3.3 us against 5.2, 2048 x 4096 9.2 against 10.2, 512 x 2048 3.3 against 3.9; from 8192 rows up the wave
    // form is ahead, 16384 x 4096 37.4 against 40.1.)
    const int lanes_cache = bf16_row_chunks_per_lane(K / epv);
    const bool few_rows = (lanes_cache == 8 && R <= 2048) || (lanes_cache == 4 && R <= 512);
    if (const int wave_cache = few_rows ? 0 : lanes_cache) {
      auto kern = wave_cache == 2   ? quantize_rows_vec_kernel<uint16_t, 2, 64, kWaveRows>
                  : wave_cache == 4 ? quantize_rows_vec_kernel<uint16_t, 4, 64, kWaveRows>
                                    : quantize_rows_vec_kernel<uint16_t, 8, 64, kWaveRows>;
      hipLaunchKernelGGL(kern, dim3(wave_grid), dim3(64 * kWaveRows), 0, s, (const uint16_t*)x, (uint8_t*)xq, inv_scale, (int)K,
                         (long)ldx, (long)ldq, (long)R);
    } else {
      // (Long rows: 512 lanes with 8 chunks each up to 4096 chunks, 1024 lanes with 4 beyond. 1024 lanes with 8 chunks
      // each, the f32 form, reach half the rate here: 16384 x 28672 397.6 us against 235.4, 4096 x 28672 104.6 against 64.0;
      // 16384 x 53248 600 against 469.)
      const bool very_long_row = K / epv > 8 * 512;
      auto kern = very_long_row ? quantize_rows_vec_kernel<uint16_t, 4, 1024>
                  : long_row    ? quantize_rows_vec_kernel<uint16_t, 8, 512>
                  : short_row   ? quantize_rows_vec_kernel<uint16_t, 4, 256>
                                : quantize_rows_vec_kernel<uint16_t, 8, 256>;
      hipLaunchKernelGGL(kern, dim3((unsigned)R), dim3(very_long_row ? 1024 : long_row ? 512 : 256), 0, s,
                         (const uint16_t*)x, (uint8_t*)xq, inv_scale, (int)K, (long)ldx, (long)ldq, (long)R);
    }
  } else if (src_type == MI355X_FP8_SRC_F32) {
    hipLaunchKernelGGL(quantize_rows_kernel<float>, dim3((unsigned)R), dim3(256), 0, s, (const float*)x,
                       (uint8_t*)xq, inv_scale, (int)K, (long)ldx, (long)ldq);
  } else if (src_type == MI355X_FP8_SRC_BF16) {
    hipLaunchKernelGGL(quantize_rows_kernel<uint16_t>, dim3((unsigned)R), dim3(256), 0, s,
                       (const uint16_t*)x, (uint8_t*)xq, inv_scale, (int)K, (long)ldx, (long)ldq);
  } else {
    return fail(MI355X_FP8_EINVAL, "unknown src_type %d", src_type);
  }
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(MI355X_FP8_ELAUNCH, "quantize kernel launch: %s", hipGetErrorString(e));
  return MI355X_FP8_OK;
}

int mi355x_fp8_blockwise_quantize(const void* x, int src_type, void* xq, float* inv_scale, int64_t M, int64_t K,
                                  int64_t ldx, int64_t ldq, void* stream) {
  if (!x || !xq || !inv_scale) return fail(MI355X_FP8_EINVAL, "null pointer");
  if (M < 1 || K < 1 || ldx < K || ldq < K) return fail(MI355X_FP8_EINVAL, "bad shape or leading dimension");
  if (M > INT32_MAX || K > INT32_MAX) return fail(MI355X_FP8_ENOTSUP, "dimension exceeds 2^31-1");
  if (src_type != MI355X_FP8_SRC_F32 && src_type != MI355X_FP8_SRC_BF16)
    return fail(MI355X_FP8_EINVAL, "unknown src_type %d", src_type);
  const int64_t grid_m = (M + kQuantBlock - 1) / kQuantBlock, grid_k = (K + kQuantBlock - 1) / kQuantBlock;
  if (grid_m > 65535) return fail(MI355X_FP8_ENOTSUP, "more than 65535 block rows");
  hipStream_t s = (hipStream_t)stream;
  const int esz = src_type == MI355X_FP8_SRC_BF16 ? 2 : 4;
  const int epv = 16 / esz;
  // whole 16-byte source chunks from 16-byte aligned rows, and stores of a chunk's codes (4 or 8 bytes) aligned
  const bool vec = (reinterpret_cast<uintptr_t>(x) & 15) == 0 && (ldx * esz) % 16 == 0 && K % epv == 0 &&
                   (reinterpret_cast<uintptr_t>(xq) & (epv - 1)) == 0 && ldq % epv == 0;
  const dim3 grid((unsigned)grid_k, (unsigned)grid_m);
  if (src_type == MI355X_FP8_SRC_F32) {
    auto kern = vec ? quantize_blocks_kernel<float, true> : quantize_blocks_kernel<float, false>;
    hipLaunchKernelGGL(kern, grid, dim3(256), 0, s, (const float*)x, (uint8_t*)xq, inv_scale, (int)M, (int)K, (long)ldx,
                       (long)ldq, (int)grid_k);
  } else {
    auto kern = vec ? quantize_blocks_kernel<uint16_t, true> : quantize_blocks_kernel<uint16_t, false>;
    hipLaunchKernelGGL(kern, grid, dim3(256), 0, s, (const uint16_t*)x, (uint8_t*)xq, inv_scale, (int)M, (int)K,
                       (long)ldx, (long)ldq, (int)grid_k);
  }
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(MI355X_FP8_ELAUNCH, "block quantize kernel launch: %s", hipGetErrorString(e));
  return MI355X_FP8_OK;
}

namespace {
int launch_fused_quant(int op, const void* x1, const void* x2, float eps, void* xq, float* inv_scale, int64_t R,
                       int64_t K, int64_t ld1, int64_t ld2, int64_t ldq, void* stream) {
  if (!x1 || !x2 || !xq || !inv_scale) return fail(MI355X_FP8_EINVAL, "null pointer");
  if (R < 1 || K < 1 || ld1 < K || ldq < K || (op == kFusedSiluMul && ld2 < K))
    return fail(MI355X_FP8_EINVAL, "bad shape or leading dimension");
  if (R > INT32_MAX || K > INT32_MAX) return fail(MI355X_FP8_ENOTSUP, "dimension exceeds 2^31-1");
  // whole 16-byte chunks of bf16, rows that start 16-byte aligned (the GEMM that follows wants K a
  // multiple of 16 and 16-byte aligned rows of codes anyway)
  if (K % 8 || ld1 % 8 || (op == kFusedSiluMul && ld2 % 8) || ldq % 16 || (reinterpret_cast<uintptr_t>(x1) & 15) ||
      (reinterpret_cast<uintptr_t>(x2) & 15) || (reinterpret_cast<uintptr_t>(xq) & 15))
    return fail(MI355X_FP8_ENOTSUP, "rows must hold whole 16-byte chunks and start 16-byte aligned");
  if (!(eps >= 0.0f)) return fail(MI355X_FP8_EINVAL, "eps must be >= 0");
  hipStream_t s = (hipStream_t)stream;
  // chunks a lane keeps in registers: 4 for rows up to 8192 elements (half the registers, twice the
  // workgroups per CU), 8 up to 16384, beyond that 1024 lanes per row
  const int64_t chunks = K / 8;
  const bool long_row = chunks > 8 * 256;
  const bool short_row = chunks <= 4 * 256;
  // > 0: a wave per row, that many chunks per lane (RMSNorm with eight chunks and their weights per lane
  // measured behind the workgroup-per-row form: 50.1 against 47.8 us on 16384 x 4096)
  int wave_cache = bf16_row_chunks_per_lane(chunks);
  if (op == kFusedRmsNorm && wave_cache == 8) wave_cache = 0;
  const dim3 grid(wave_cache ? (unsigned)((R + kWaveRows - 1) / kWaveRows) : (unsigned)R);
  // (Long rows up to 32768 elements: 512 lanes with 8 chunks each. With 1024 lanes they reach two thirds of that rate:
  // SiLU-mul 4096 x 28672 146.6 -> 100.6 us, 1024 x 28672 44.5 -> 29.5; RMSNorm 4096 x 28672 115.8 -> 83.8. Beyond,
  // 1024 lanes: 4096 x 53248 199.5 us against 218.)
  const bool mid_row = long_row && chunks <= 8 * 512;
  // (Rows of 8193 to 16384 elements: 512 lanes with 4 chunks each instead of 256 with 8. RMSNorm 8192 x 16384 96.0 ->
  // 78.6 us, 32768 x 16384 370 -> 302, 8192 x 11008 85.1 -> 67.1; SiLU-mul 8192 x 11008 80.6 -> 79.6, 8192 x 16384
  // 109.1 -> 107.6.)
  const bool half_row = !wave_cache && !long_row && !short_row;
  const dim3 block(wave_cache ? 64 * kWaveRows : mid_row || half_row ? 512 : long_row ? 1024 : 256);
  const uint16_t* a = (const uint16_t*)x1;
  const uint16_t* b = (const uint16_t*)x2;
  if (op == kFusedRmsNorm) {
    auto kern = wave_cache == 2 ? fused_rowwise_quant_kernel<kFusedRmsNorm, 2, 64, kWaveRows>
                : wave_cache == 4 ? fused_rowwise_quant_kernel<kFusedRmsNorm, 4, 64, kWaveRows>
                : wave_cache  ? fused_rowwise_quant_kernel<kFusedRmsNorm, 8, 64, kWaveRows>
                : mid_row     ? fused_rowwise_quant_kernel<kFusedRmsNorm, 8, 512>
                : long_row    ? fused_rowwise_quant_kernel<kFusedRmsNorm, 8, 1024>
                : chunks <= 2 * 256 ? fused_rowwise_quant_kernel<kFusedRmsNorm, 2, 256>  // (no idle rounds: 16384 x 4096 47.8 -> 35.5 us)
                : short_row   ? fused_rowwise_quant_kernel<kFusedRmsNorm, 4, 256> : fused_rowwise_quant_kernel<kFusedRmsNorm, 4, 512>;
    hipLaunchKernelGGL(kern, grid, block, 0, s, a, b, eps, (uint8_t*)xq, inv_scale, (int)K, (long)ld1, (long)ld2, (long)ldq, (long)R);
  } else {
    auto kern = wave_cache == 2 ? fused_rowwise_quant_kernel<kFusedSiluMul, 2, 64, kWaveRows>
                : wave_cache == 4 ? fused_rowwise_quant_kernel<kFusedSiluMul, 4, 64, kWaveRows>
                : wave_cache  ? fused_rowwise_quant_kernel<kFusedSiluMul, 8, 64, kWaveRows>
                : mid_row     ? fused_rowwise_quant_kernel<kFusedSiluMul, 8, 512>
                : long_row    ? fused_rowwise_quant_kernel<kFusedSiluMul, 8, 1024>
                : short_row   ? fused_rowwise_quant_kernel<kFusedSiluMul, 4, 256> : fused_rowwise_quant_kernel<kFusedSiluMul, 4, 512>;
    hipLaunchKernelGGL(kern, grid, block, 0, s, a, b, eps, (uint8_t*)xq, inv_scale, (int)K, (long)ld1, (long)ld2, (long)ldq, (long)R);
  }
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(MI355X_FP8_ELAUNCH, "fused quantise kernel launch: %s", hipGetErrorString(e));
  return MI355X_FP8_OK;
}
}  // namespace

int mi355x_fp8_rmsnorm_rowwise_quantize(const void* x, const void* weight, float eps, void* xq, float* inv_scale,
                                        int64_t R, int64_t K, int64_t ldx, int64_t ldq, void* stream) {
  return launch_fused_quant(kFusedRmsNorm, x, weight, eps, xq, inv_scale, R, K, ldx, K, ldq, stream);
}

int mi355x_fp8_silu_mul_rowwise_quantize(const void* x1, const void* x2, void* xq, float* inv_scale, int64_t R,
                                         int64_t K, int64_t ldx1, int64_t ldx2, int64_t ldq, void* stream) {
  return launch_fused_quant(kFusedSiluMul, x1, x2, 0.0f, xq, inv_scale, R, K, ldx1, ldx2, ldq, stream);
}

}  // extern "C"
#endif  // !MI355X_TILED_PART
