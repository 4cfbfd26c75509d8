// Row-wise scaled FP8 (e4m3fn) GEMM for MI355X (gfx950, CDNA4): kernels and C ABI.
//
//   C[M,N] bf16 = bf16( (sum_k A[m,k] * B[n,k]) * a_scale[m] * b_scale[n] + bias[n] )
//
// A is [M,K] and B is [N,K], both K-contiguous, one byte per element. The contraction runs
// on the gfx950 f8f6f4 MFMA instructions (full FP8 rate) with fp32 accumulation; scales and
// bias are applied in fp32 to the accumulator and the result is rounded to bf16 once.
//
// Two kernel families:
//   gemm_tiled_kernel   persistent workgroups, BM x BN x 128 tiles staged global->LDS with
//                       direct-to-LDS loads into two swizzled stages, 32x32x64 MFMA.
//   gemm_skinny_kernel  M <= 64: every workgroup owns 16 rows of B and all of K, its waves
//                       split K between them and reduce through LDS; B is streamed once.
//
// Operand roles inside the MFMA are swapped on purpose (rows of B feed the instruction's
// "A" port, rows of A its "B" port) so each lane ends up holding 4 consecutive columns n of
// one output row m and can store them as one 8-byte write.

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdarg.h>
#include <stdio.h>
#include <string.h>

#include "../../include/mi355x_fp8_rowwise.h"

namespace {

typedef int   v4i  __attribute__((ext_vector_type(4)));
typedef int   v8i  __attribute__((ext_vector_type(8)));
typedef float v4f  __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef unsigned short us4 __attribute__((ext_vector_type(4)));

constexpr int kNumXcd = 8;       // accelerator complex dies; workgroup ids round-robin over them
constexpr int kNumCu = 256;
constexpr int kBK = 128;         // bytes (= fp8 elements) of K per LDS stage
constexpr int kChunk = 16;       // bytes moved per lane per load

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

__device__ __forceinline__ void tile_coords(int t, int tiles_m, int tiles_n, int group_m,
                                            int& tm, int& tn) {
  const int per_group = group_m * tiles_n;
  const int g = t / per_group;
  const int first_m = g * group_m;
  const int gsz = min(tiles_m - first_m, group_m);
  const int in_g = t - g * per_group;
  tm = first_m + in_g % gsz;
  tn = in_g / gsz;
}

// ------------------------------------------------------------------------------------
// LDS tile layout. A stage holds BM rows of A then BN rows of B, 128 bytes per row, i.e. 8
// chunks of 16 bytes. Chunk c of row r is kept at chunk position c ^ swz(r) so that the
// MFMA operand reads (consecutive lanes = consecutive rows, same logical chunk) spread
// over all banks instead of piling onto one.
// ------------------------------------------------------------------------------------
template <int SWZ_SHIFT>
__device__ __forceinline__ int swz(int row) {
  return (row >> SWZ_SHIFT) & 7;
}

__device__ __forceinline__ void load_chunk_to_lds(const uint8_t* gsrc, uint8_t* lds_wave_base) {
  // Each lane fetches 16 bytes; the hardware deposits lane i's bytes at lds_wave_base + 16*i.
  __builtin_amdgcn_global_load_lds(
      (const __attribute__((address_space(1))) void*)gsrc,
      (__attribute__((address_space(3))) void*)lds_wave_base, 16, 0, 0);
}

template <int BM, int BN, int WAVES_M, int WAVES_N, int SWZ_SHIFT>
__global__ __launch_bounds__(WAVES_M* WAVES_N * 64) void gemm_tiled_kernel(GemmParams p) {
  constexpr int NW = WAVES_M * WAVES_N;
  constexpr int WTM = BM / WAVES_M;    // wave tile rows (m)
  constexpr int WTN = BN / WAVES_N;    // wave tile cols (n)
  constexpr int MT = WTM / 32, NT = WTN / 32;
  constexpr int STAGE = (BM + BN) * kBK;
  constexpr int A_GROUPS = BM / 8 / NW;  // 8-row groups of A each wave fetches per stage
  constexpr int B_GROUPS = BN / 8 / NW;
  static_assert(BM % (8 * NW) == 0 && BN % (8 * NW) == 0, "tile rows must split over waves");
  static_assert(WTM % 32 == 0 && WTN % 32 == 0, "wave tile must be a multiple of 32x32");

  extern __shared__ __attribute__((aligned(1024))) uint8_t lds[];

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int wm = wave / WAVES_N, wn = wave % WAVES_N;
  const int l32 = lane & 31, half = lane >> 5;

  // ---- per-lane constants of the global->LDS copy
  const int ld_row = lane >> 3;  // row inside an 8-row group
  const int ld_pc = lane & 7;    // physical chunk this lane's 16 bytes land in

  // ---- per-lane constants of the LDS->register operand reads
  // Lane (l32, half) takes, for K sub-step s (64 bytes) and j in {0,1}, logical chunk
  // 4*half + 2*s + j of its row. Any assignment is valid as long as A and B use the same
  // one; this one keeps the two halves of the wave in different 64-byte halves of a row.
  int rd_off[2][2];
#pragma unroll
  for (int s = 0; s < 2; ++s)
#pragma unroll
    for (int j = 0; j < 2; ++j)
      rd_off[s][j] = l32 * kBK + (((4 * half + 2 * s + j) ^ swz<SWZ_SHIFT>(l32)) * kChunk);
  const int a_rd_base = (wm * WTM) * kBK;
  const int b_rd_base = BM * kBK + (wn * WTN) * kBK;

  const int total_tiles = p.tiles_m * p.tiles_n;
  const TileWalk walk = make_walk(total_tiles);
  const int k_full = p.K / kBK;            // whole 128-byte steps
  const int k_tail = p.K - k_full * kBK;   // 0 or a multiple of 16
  const int k_steps = k_full + (k_tail ? 1 : 0);

  for (int li = walk.slot; li < walk.chunk_len; li += walk.slots) {
    int tm, tn;
    tile_coords(walk.chunk_begin + li, p.tiles_m, p.tiles_n, p.group_m, tm, tn);
    const int m0 = tm * BM, n0 = tn * BN;

    // Rows past the matrix edge are redirected to the last valid row: they are read but
    // never stored, so every load stays in bounds without predication.
    uint32_t a_off[A_GROUPS], b_off[B_GROUPS];
    const uint8_t* a_tile = p.a + (size_t)m0 * p.lda;
    const uint8_t* b_tile = p.b + (size_t)n0 * p.ldb;
#pragma unroll
    for (int i = 0; i < A_GROUPS; ++i) {
      const int r = (wave + NW * i) * 8 + ld_row;
      const int rc = min(r, p.M - 1 - m0);
      a_off[i] = (uint32_t)rc * (uint32_t)p.lda + ((ld_pc ^ swz<SWZ_SHIFT>(r)) * kChunk);
    }
#pragma unroll
    for (int i = 0; i < B_GROUPS; ++i) {
      const int r = (wave + NW * i) * 8 + ld_row;
      const int rc = min(r, p.N - 1 - n0);
      b_off[i] = (uint32_t)rc * (uint32_t)p.ldb + ((ld_pc ^ swz<SWZ_SHIFT>(r)) * kChunk);
    }

    auto issue_stage = [&](int kt, int stage) {
      uint8_t* sbase = lds + stage * STAGE;
      const size_t kb = (size_t)kt * kBK;
      if (kt < k_full) {
#pragma unroll
        for (int i = 0; i < A_GROUPS; ++i)
          load_chunk_to_lds(a_tile + kb + a_off[i], sbase + (wave + NW * i) * 1024);
#pragma unroll
        for (int i = 0; i < B_GROUPS; ++i)
          load_chunk_to_lds(b_tile + kb + b_off[i], sbase + BM * kBK + (wave + NW * i) * 1024);
      } else {
        // K tail: chunks past K are written as zeros (they would otherwise pollute the sums).
#pragma unroll
        for (int i = 0; i < A_GROUPS; ++i) {
          const int r = (wave + NW * i) * 8 + ld_row;
          const int c = ld_pc ^ swz<SWZ_SHIFT>(r);
          v4i v = {0, 0, 0, 0};
          if (c * kChunk < k_tail) v = *(const v4i*)(a_tile + kb + a_off[i]);
          *(v4i*)(sbase + (wave + NW * i) * 1024 + lane * kChunk) = v;
        }
#pragma unroll
        for (int i = 0; i < B_GROUPS; ++i) {
          const int r = (wave + NW * i) * 8 + ld_row;
          const int c = ld_pc ^ swz<SWZ_SHIFT>(r);
          v4i v = {0, 0, 0, 0};
          if (c * kChunk < k_tail) v = *(const v4i*)(b_tile + kb + b_off[i]);
          *(v4i*)(sbase + BM * kBK + (wave + NW * i) * 1024 + lane * kChunk) = v;
        }
      }
    };

    v16f acc[MT][NT];
#pragma unroll
    for (int i = 0; i < MT; ++i)
#pragma unroll
      for (int j = 0; j < NT; ++j)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;

    __syncthreads();  // previous tile's readers are done with both stages
    issue_stage(0, 0);

    for (int kt = 0; kt < k_steps; ++kt) {
      const int stage = kt & 1;
      __syncthreads();  // stage `stage` has landed everywhere; the other stage is free
      if (kt + 1 < k_steps) issue_stage(kt + 1, stage ^ 1);

      const uint8_t* sa = lds + stage * STAGE + a_rd_base;
      const uint8_t* sb = lds + stage * STAGE + b_rd_base;
#pragma unroll
      for (int s = 0; s < 2; ++s) {
        v8i af[MT], bf[NT];
#pragma unroll
        for (int i = 0; i < MT; ++i) {
          const v4i lo = *(const v4i*)(sa + i * 32 * kBK + rd_off[s][0]);
          const v4i hi = *(const v4i*)(sa + i * 32 * kBK + rd_off[s][1]);
          af[i] = (v8i){lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
        }
#pragma unroll
        for (int j = 0; j < NT; ++j) {
          const v4i lo = *(const v4i*)(sb + j * 32 * kBK + rd_off[s][0]);
          const v4i hi = *(const v4i*)(sb + j * 32 * kBK + rd_off[s][1]);
          bf[j] = (v8i){lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
        }
#pragma unroll
        for (int i = 0; i < MT; ++i)
#pragma unroll
          for (int j = 0; j < NT; ++j)
            acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(
                bf[j], af[i], acc[i][j], 0, 0, 0, 0, 0, 0);
      }
    }

    // ---- epilogue: lane holds, for every (i, j) sub-tile, row m = .. + l32 and the columns
    // n = .. + 8*q + 4*half + e (register v = 4*q + e).
    const bool full = (m0 + BM <= p.M) && (n0 + BN <= p.N) && ((p.ldc & 3) == 0) &&
                      ((reinterpret_cast<uintptr_t>(p.c) & 7) == 0);
#pragma unroll
    for (int i = 0; i < MT; ++i) {
      const int m = m0 + wm * WTM + i * 32 + l32;
      const float sa_m = p.a_scale[min(m, p.M - 1)];
      uint16_t* crow = p.c + (size_t)m * p.ldc;
#pragma unroll
      for (int j = 0; j < NT; ++j) {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int n = n0 + wn * WTN + j * 32 + 8 * q + 4 * half;
          if (full) {
            const v4f sb4 = *(const v4f*)(p.b_scale + n);
            float r[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) r[e] = acc[i][j][4 * q + e] * sa_m * sb4[e];
            if (p.bias) {
              const us4 b4 = *(const us4*)(p.bias + n);
#pragma unroll
              for (int e = 0; e < 4; ++e) r[e] += bf16_to_f32(b4[e]);
            }
            us4 o;
#pragma unroll
            for (int e = 0; e < 4; ++e) o[e] = f32_to_bf16_rne(r[e]);
            *(us4*)(crow + n) = o;
          } else if (m < p.M) {
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              if (n + e < p.N) {
                float r = acc[i][j][4 * q + e] * sa_m * p.b_scale[n + e];
                if (p.bias) r += bf16_to_f32(p.bias[n + e]);
                crow[n + e] = f32_to_bf16_rne(r);
              }
            }
          }
        }
      }
    }
  }
}

// ------------------------------------------------------------------------------------
// Skinny kernel (M <= 16*MT). Workgroup = KW waves sharing one 16-row panel of B; wave w
// takes the 128-byte K steps w, w+KW, ... so that per iteration the workgroup reads one
// contiguous KW*128-byte run of every row. Lane (r = lane%16, g = lane/16) loads, per
// step, bytes [g*16, g*16+16) and [64+g*16, 64+g*16+16) of its row: each load
// instruction then covers 64 contiguous bytes per row. A is read with the same mapping
// straight from L2. Partial 16x16 tiles are summed across waves through LDS.
// ------------------------------------------------------------------------------------
template <int MT, int KW>
__global__ __launch_bounds__(KW * 64) void gemm_skinny_kernel(GemmParams p) {
  __shared__ v4f red[KW][MT][64];

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int r = lane & 15, g = lane >> 4;
  const int n0 = blockIdx.x * 16;

  const uint8_t* bp = p.b + (size_t)min(n0 + r, p.N - 1) * p.ldb + g * kChunk;
  const uint8_t* ap[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t)
    ap[t] = p.a + (size_t)min(t * 16 + r, p.M - 1) * p.lda + g * kChunk;

  v4f acc[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) acc[t] = (v4f){0.f, 0.f, 0.f, 0.f};

  const int k_full = p.K / kBK;
  const int k_tail = p.K - k_full * kBK;

  constexpr int UNROLL = (MT == 1) ? 4 : 2;
  int it = wave;
  for (; it + (UNROLL - 1) * KW < k_full; it += UNROLL * KW) {
    v4i b0[UNROLL], b1[UNROLL], a0[UNROLL][MT], a1[UNROLL][MT];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      const size_t kb = (size_t)(it + u * KW) * kBK;
      b0[u] = __builtin_nontemporal_load((const v4i*)(bp + kb));
      b1[u] = __builtin_nontemporal_load((const v4i*)(bp + kb + 64));
    }
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      const size_t kb = (size_t)(it + u * KW) * kBK;
#pragma unroll
      for (int t = 0; t < MT; ++t) {
        a0[u][t] = *(const v4i*)(ap[t] + kb);
        a1[u][t] = *(const v4i*)(ap[t] + kb + 64);
      }
    }
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      const v8i bf = {b0[u][0], b0[u][1], b0[u][2], b0[u][3], b1[u][0], b1[u][1], b1[u][2], b1[u][3]};
#pragma unroll
      for (int t = 0; t < MT; ++t) {
        const v8i af = {a0[u][t][0], a0[u][t][1], a0[u][t][2], a0[u][t][3],
                        a1[u][t][0], a1[u][t][1], a1[u][t][2], a1[u][t][3]};
        acc[t] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(bf, af, acc[t], 0, 0, 0, 0, 0, 0);
      }
    }
  }
  // leftover whole steps, then the partial step (taken by the wave whose turn it is)
  for (; it < k_full + (k_tail ? 1 : 0); it += KW) {
    const size_t kb = (size_t)it * kBK;
    const int lim = (it < k_full) ? kBK : k_tail;
    const bool in0 = g * kChunk < lim, in1 = 64 + g * kChunk < lim;
    const v4i z = {0, 0, 0, 0};
    const v4i b0 = in0 ? *(const v4i*)(bp + kb) : z;
    const v4i b1 = in1 ? *(const v4i*)(bp + kb + 64) : z;
    const v8i bf = {b0[0], b0[1], b0[2], b0[3], b1[0], b1[1], b1[2], b1[3]};
#pragma unroll
    for (int t = 0; t < MT; ++t) {
      const v4i a0 = in0 ? *(const v4i*)(ap[t] + kb) : z;
      const v4i a1 = in1 ? *(const v4i*)(ap[t] + kb + 64) : z;
      const v8i af = {a0[0], a0[1], a0[2], a0[3], a1[0], a1[1], a1[2], a1[3]};
      acc[t] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(bf, af, acc[t], 0, 0, 0, 0, 0, 0);
    }
  }

#pragma unroll
  for (int t = 0; t < MT; ++t) red[wave][t][lane] = acc[t];
  __syncthreads();

  // Lane layout of a 16x16 result: m = t*16 + lane%16, n = n0 + 4*(lane/16) + e.
  for (int idx = threadIdx.x; idx < MT * 64; idx += KW * 64) {
    const int t = idx >> 6, l = idx & 63;
    v4f s = red[0][t][l];
#pragma unroll
    for (int w = 1; w < KW; ++w) s += red[w][t][l];
    const int m = t * 16 + (l & 15);
    const int n = n0 + 4 * (l >> 4);
    if (m >= p.M) continue;
    const float sa_m = p.a_scale[m];
    uint16_t* crow = p.c + (size_t)m * p.ldc;
    uint16_t o[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int ne = min(n + e, p.N - 1);
      float v = s[e] * sa_m * p.b_scale[ne];
      if (p.bias) v += bf16_to_f32(p.bias[ne]);
      o[e] = f32_to_bf16_rne(v);
    }
    if (n + 3 < p.N && ((p.ldc & 3) == 0) && ((reinterpret_cast<uintptr_t>(p.c) & 7) == 0)) {
      *(us4*)(crow + n) = (us4){o[0], o[1], o[2], o[3]};
    } else {
#pragma unroll
      for (int e = 0; e < 4; ++e)
        if (n + e < p.N) crow[n + e] = o[e];
    }
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
  for (int k = threadIdx.x; k < K; k += 256) amax = fmaxf(amax, fabsf(T::load(xr + k)));
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) amax = fmaxf(amax, __shfl_xor(amax, o));
  if ((threadIdx.x & 63) == 0) wave_max[threadIdx.x >> 6] = amax;
  __syncthreads();
  amax = fmaxf(fmaxf(wave_max[0], wave_max[1]), fmaxf(wave_max[2], wave_max[3]));

  // `448.0 / tensor` in the PyTorch program this replaces evaluates as reciprocal * 448
  const float recip = T::round(1.0f / fmaxf(amax, T::round(1e-12f)));
  const float scale = T::round(recip * 448.0f);
  if (threadIdx.x == 0) inv_scale[row] = T::round(1.0f / scale);
  for (int k = threadIdx.x; k < K; k += 256) {
    float v = T::round(T::load(xr + k) * scale);
    v = fminf(fmaxf(v, -448.0f), 448.0f);
    qr[k] = f32_to_e4m3fn_rne(v);
  }
}

// ------------------------------------------------------------------------------------
// Host side
// ------------------------------------------------------------------------------------
thread_local char g_err[512] = "";

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

constexpr int kSkinnyMaxM = 64;

int check_shape(int64_t M, int64_t N, int64_t K) {
  if (M < 1 || N < 1 || K < 1) return fail(MI355X_FP8_EINVAL, "M, N, K must be >= 1 (got %lld, %lld, %lld)",
                                           (long long)M, (long long)N, (long long)K);
  if (M > INT32_MAX || N > INT32_MAX || K > INT32_MAX)
    return fail(MI355X_FP8_ENOTSUP, "dimension exceeds 2^31-1");
  if (K % 16 != 0) return fail(MI355X_FP8_ENOTSUP, "K must be a multiple of 16 (got %lld)", (long long)K);
  return MI355X_FP8_OK;
}

template <int BM, int BN, int WAVES_M, int WAVES_N, int SWZ_SHIFT>
int launch_tiled(GemmParams p, hipStream_t stream) {
  constexpr int threads = WAVES_M * WAVES_N * 64;
  constexpr size_t lds_bytes = 2 * (size_t)(BM + BN) * kBK;
  p.tiles_m = (p.M + BM - 1) / BM;
  p.tiles_n = (p.N + BN - 1) / BN;
  p.group_m = 4;
  const long total = (long)p.tiles_m * p.tiles_n;
  long grid = total < kNumCu ? ((total + kNumXcd - 1) / kNumXcd) * kNumXcd : kNumCu;
  auto kern = gemm_tiled_kernel<BM, BN, WAVES_M, WAVES_N, SWZ_SHIFT>;
  static bool attr_set = false;  // raising the dynamic LDS limit is idempotent; races are harmless
  if (!attr_set) {
    hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize,
                                       (int)lds_bytes);
    if (e != hipSuccess) return fail(MI355X_FP8_ELAUNCH, "hipFuncSetAttribute: %s", hipGetErrorString(e));
    attr_set = true;
  }
  hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(threads), lds_bytes, stream, p);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(MI355X_FP8_ELAUNCH, "tiled kernel launch: %s", hipGetErrorString(e));
  return MI355X_FP8_OK;
}

template <int MT>
int launch_skinny(const GemmParams& p, hipStream_t stream) {
  constexpr int KW = 8;
  const unsigned grid = (unsigned)((p.N + 15) / 16);
  hipLaunchKernelGGL((gemm_skinny_kernel<MT, KW>), dim3(grid), dim3(KW * 64), 0, stream, p);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(MI355X_FP8_ELAUNCH, "skinny kernel launch: %s", hipGetErrorString(e));
  return MI355X_FP8_OK;
}

}  // namespace

extern "C" {

int mi355x_fp8_rowwise_abi_version(void) { return MI355X_FP8_ABI_VERSION; }

const char* mi355x_fp8_rowwise_last_error(void) { return g_err; }

int mi355x_fp8_rowwise_select_variant(int64_t M, int64_t N, int64_t K) {
  const int st = check_shape(M, N, K);
  if (st != MI355X_FP8_OK) return st;
  return M <= kSkinnyMaxM ? MI355X_FP8_VARIANT_SKINNY : MI355X_FP8_VARIANT_TILED;
}

size_t mi355x_fp8_rowwise_workspace_bytes(int64_t M, int64_t N, int64_t K, int variant) {
  (void)M; (void)N; (void)K; (void)variant;
  return 0;  // both kernel families reduce on chip
}

int mi355x_fp8_rowwise_gemm(const void* a, const void* b, const float* a_scale, const float* b_scale,
                            const void* bias, void* c, int64_t M, int64_t N, int64_t K, int64_t lda,
                            int64_t ldb, int64_t ldc, void* workspace, size_t workspace_bytes,
                            int variant, void* stream) {
  (void)workspace; (void)workspace_bytes;
  int st = check_shape(M, N, K);
  if (st != MI355X_FP8_OK) return st;
  if (!a || !b || !a_scale || !b_scale || !c) return fail(MI355X_FP8_EINVAL, "null operand pointer");
  if (lda < K || ldb < K || ldc < N) return fail(MI355X_FP8_EINVAL, "leading dimension smaller than the row length");
  if (lda % 16 || ldb % 16) return fail(MI355X_FP8_ENOTSUP, "lda and ldb must be multiples of 16");
  if ((reinterpret_cast<uintptr_t>(a) & 15) || (reinterpret_cast<uintptr_t>(b) & 15))
    return fail(MI355X_FP8_ENOTSUP, "a and b must be 16-byte aligned");
  if ((reinterpret_cast<uintptr_t>(a_scale) & 3) || (reinterpret_cast<uintptr_t>(b_scale) & 3) ||
      (reinterpret_cast<uintptr_t>(c) & 1) || (reinterpret_cast<uintptr_t>(bias) & 1))
    return fail(MI355X_FP8_EINVAL, "misaligned scale, bias or output pointer");
  if (lda * 256 > (int64_t)UINT32_MAX || ldb * 256 > (int64_t)UINT32_MAX)
    return fail(MI355X_FP8_ENOTSUP, "leading dimension too large");
  if (variant == MI355X_FP8_VARIANT_AUTO) variant = mi355x_fp8_rowwise_select_variant(M, N, K);
  if (variant == MI355X_FP8_VARIANT_SKINNY && M > kSkinnyMaxM)
    return fail(MI355X_FP8_ENOTSUP, "skinny variant handles M <= %d (got %lld)", kSkinnyMaxM, (long long)M);

  GemmParams p;
  p.a = (const uint8_t*)a; p.b = (const uint8_t*)b;
  p.a_scale = a_scale; p.b_scale = b_scale;
  p.bias = (const uint16_t*)bias; p.c = (uint16_t*)c;
  p.M = (int)M; p.N = (int)N; p.K = (int)K;
  p.lda = lda; p.ldb = ldb; p.ldc = ldc;
  p.tiles_m = p.tiles_n = 0; p.group_m = 1;
  hipStream_t s = (hipStream_t)stream;

  switch (variant) {
    case MI355X_FP8_VARIANT_TILED:
      // b_scale is read 16 bytes at a time on full tiles
      if (reinterpret_cast<uintptr_t>(b_scale) & 15 || (bias && (reinterpret_cast<uintptr_t>(bias) & 7)))
        return fail(MI355X_FP8_ENOTSUP, "tiled variant needs b_scale 16-byte and bias 8-byte aligned");
      return launch_tiled<256, 256, 2, 2, 0>(p, s);
    case MI355X_FP8_VARIANT_SKINNY:
      if (M <= 16) return launch_skinny<1>(p, s);
      if (M <= 32) return launch_skinny<2>(p, s);
      if (M <= 48) return launch_skinny<3>(p, s);
      return launch_skinny<4>(p, s);
    default:
      return fail(MI355X_FP8_EINVAL, "unknown variant %d", variant);
  }
}

int mi355x_fp8_rowwise_quantize(const void* x, int src_type, void* xq, float* inv_scale, int64_t R,
                                int64_t K, int64_t ldx, int64_t ldq, void* stream) {
  if (!x || !xq || !inv_scale) return fail(MI355X_FP8_EINVAL, "null pointer");
  if (R < 1 || K < 1 || ldx < K || ldq < K) return fail(MI355X_FP8_EINVAL, "bad shape or leading dimension");
  if (R > INT32_MAX || K > INT32_MAX) return fail(MI355X_FP8_ENOTSUP, "dimension exceeds 2^31-1");
  hipStream_t s = (hipStream_t)stream;
  if (src_type == MI355X_FP8_SRC_F32) {
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

}  // extern "C"
