// bf16 GEMM for k-contiguous operands (C[m][n] = sum_k A[m][k] * B[n][k]) with an LDS ring
// filled by direct global->LDS loads (global_load_lds_dwordx4, gfx950), so that several
// K-slabs are in flight per workgroup without passing through registers.
//
// Replaces, for the layouts that qualify, the reference's dot_general lowering to mlx
// matmul (src/pjrt_plugin/ops/linalg.cc:89-250).
//
// Layout of one ring stage: BM rows of A then BN rows of B, each row 64 k = 128 bytes = 8
// slots of 16 bytes.  A direct load writes lane i of a wavefront at (LDS base + 16*i), i.e.
// a wavefront instruction fills 8 whole rows; which 16 bytes of global memory a lane fetches
// is free, so the logical slot kv of row r is kept at physical slot kv ^ ((r >> 1) & 7).
// With that swizzle the MFMA operand read (32 rows x one slot, ds_read_b128) touches every
// bank once per 16 lanes.
//
// B may also be given n-contiguous ([K][N] rows, the layout of a dense layer's weights): its
// stage then holds 64 k-rows of BN columns, and the MFMA operand (8 consecutive k per lane) is
// assembled by two transposing LDS reads (ds_read_b64_tr_b16: within 16 lanes, lane d receives
// element d%4 of the 8 bytes addressed by lanes d/4, d/4+4, d/4+8, d/4+12), so no transposed
// copy of the weights is made.  The 16-byte slots of a k-row are XOR-swizzled by the row number
// so that the four rows one such read touches fall into different banks.
//
// Pipeline per iteration: wait until the oldest stage has landed (vmcnt), barrier, start the
// loads that refill the stage consumed one iteration ago, multiply the landed stage.  One
// barrier per 64-wide K-slab; loads are (STAGES-1) slabs ahead of the math.
//
// Every ring stage is an LDS array of its own and the K loop is unrolled by the ring length, so each
// direct load and each operand read names its stage at compile time.  The compiler has to order LDS
// reads after direct loads into LDS that may alias them; with one array for the whole ring it cannot
// tell the stage being refilled from the stage being read and waits for every outstanding load
// (vmcnt(0)) before the first operand read of each iteration, which serialises load and math.
#include <hip/hip_runtime.h>

#include <cstdint>
#include <cstdio>
#include <cstdlib>

#include "hip_abi.h"

namespace {

typedef unsigned short u16;
typedef unsigned int u32;
typedef float float16v __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef short short4v __attribute__((ext_vector_type(4)));
typedef short short8v __attribute__((ext_vector_type(8)));

#define GLOBAL_PTR(p) ((__attribute__((address_space(1))) void*)(p))
#define LDS_PTR(p) ((__attribute__((address_space(3))) void*)(p))

struct AsyncArgs {
  const u16* a;
  const u16* b;
  void* c;
  const void* bias;   // N values of the output type, or null
  long long M, N, K;
  long long aB0, aB1, aLd, bB0, bB1, bLd;
  int batch1;
  int outBf16;
  int tilesM, tilesN;
  long long total;
  int act;                 // 1: y = actA * x * (1 + tanh(actC * (x + actB * x^3))) on the stored value (bf16 results)
  float actA, actB, actC;
};

__device__ __forceinline__ u16 to_bf16(float f) { return __builtin_bit_cast(u16, (__bf16)f); }

// s_waitcnt immediate for "at most n vector-memory operations outstanding" (gfx9 encoding:
// vmcnt in bits 3:0 and 15:14, expcnt 6:4 and lgkmcnt 11:8 left at their maxima)
constexpr int vmcntImm(int n) { return (n & 15) | ((n >> 4) << 14) | (7 << 4) | (15 << 8); }

// slot swizzle of an n-contiguous B stage: rows k .. k+3 of one 32-column block land in distinct banks
template <int BN>
__device__ __forceinline__ int swzB(int k) { return BN == 64 ? ((k >> 1) & 1) << 2 : (k & 3) << 2; }

// one LDS array per (size, stage): distinct objects, so accesses to different stages provably do not alias
template <int BYTES, int S>
__device__ __forceinline__ unsigned char* stageBase() {
  __shared__ __attribute__((aligned(1024))) unsigned char buf[BYTES];
  return buf;
}

template <int N>
struct Const { static constexpr int value = N; };

// WM wavefront rows by 2 wavefront columns per workgroup: 2 x 2 for the tiles up to 256 x 128, 4 x 2 (512 lanes, two
// wavefronts per SIMD, each 64 x 128 of the result) for the 256 x 256 tile.  The large tile is what the matrix pipes
// need to stay fed: a stage of it carries 64 KB for 2048 cycles of products per compute unit (32 bytes a cycle through
// the vector memory path, half of what that path delivers), where a 128 x 64 tile asks for 24 KB per 256 cycles and
// three resident workgroups together saturate the path at under half of the matrix peak; and with two wavefronts on
// a SIMD one reads its operands from LDS while the other multiplies.  What it cannot do is keep more than one stage
// in flight (two stages fill 128 KB of LDS), so it waits for memory about 60 % of the time and pays only for long K.
template <int BM, int BN, int STAGES, bool BNN, int WM = 2>
__global__ void __launch_bounds__(WM * 128) gemm_bf16_async(AsyncArgs g) {
  constexpr int BK = 64;
  constexpr int NW = WM * 2;                  // wavefronts per workgroup
  constexpr int NT = NW * 64;
  constexpr int TM = BM / (32 * WM), TN = BN / 64;
  constexpr int STAGE_BYTES = (BM + BN) * 128;
  constexpr int NI = (BM + BN) / (8 * NW);    // direct loads per wavefront per stage (8 rows each)
  static_assert((STAGES - 2) * NI <= 63, "vmcnt range");
  static_assert(BM % (32 * WM) == 0 && (BM / 8) % NW == 0 && (BN / 8) % NW == 0, "tile split over the wavefronts");
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;

  // tile decode in 32-bit arithmetic (the launcher keeps the grid below 2^31): 64-bit divisions cost hundreds of cycles each
  unsigned id = blockIdx.x;
  const unsigned total = (unsigned)g.total;
  if ((total & 7u) == 0) id = (id & 7u) * (total >> 3) + (id >> 3);
  const unsigned perBatch = (unsigned)g.tilesM * (unsigned)g.tilesN;
  const unsigned bzu = id / perBatch;
  const unsigned t = id - bzu * perBatch;
  int tm, tn;
  if (WM == 4) {
    // eight tile rows are walked together, column by column: the 32 workgroups an XCD runs at a time then share 8 + 4
    // operand slabs per step of K in its L2 instead of 1 + 32
    const unsigned perGroup = 8u * (unsigned)g.tilesN;
    const unsigned group = t / perGroup, first = group * 8u;
    const unsigned rows = (unsigned)g.tilesM - first < 8u ? (unsigned)g.tilesM - first : 8u;
    const unsigned in = t - group * perGroup;
    tm = (int)(first + in % rows);
    tn = (int)(in / rows);
  } else {
    tm = (int)(t / (unsigned)g.tilesN);
    tn = (int)(t - (unsigned)tm * (unsigned)g.tilesN);
  }
  const long long bz = bzu;
  const long long b0 = bzu / (unsigned)g.batch1, b1 = bzu - (unsigned)b0 * (unsigned)g.batch1;
  const u16* A = g.a + b0 * g.aB0 + b1 * g.aB1;
  const u16* B = g.b + b0 * g.bB0 + b1 * g.bB1;
  const long long m0 = (long long)tm * BM, n0 = (long long)tn * BN;

  // per-lane source of each of this wavefront's direct loads (rows past the edge re-read the last row;
  // their products land in accumulator rows or columns that are never stored)
  const u16* src[NI];
#pragma unroll
  for (int j = 0; j < NI; ++j) {
    const int c = j * NW + wave;                      // 8-row group within the stage
    const int r = c * 8 + (lane >> 3);                // row within [A rows | B rows]
    const int kv = (lane & 7) ^ ((r >> 1) & 7);       // logical k-slot this lane fetches
    if (r < BM) {
      long long gm = m0 + r;
      if (gm > g.M - 1) gm = g.M - 1;
      src[j] = A + gm * g.aLd + kv * 8;
    } else if (BNN) {
      constexpr int PR = BN / 8;                      // 16-byte slots per k-row
      const int q = (c - BM / 8) * 64 + lane;         // physical slot within the B part
      const int k = q / PR;
      const int pcol = (q % PR) ^ swzB<BN>(k);        // logical slot kept there
      long long gn = n0 + pcol * 8;
      if (gn > g.N - 8) gn = g.N - 8;                 // columns past the edge are never stored
      src[j] = B + (long long)k * g.bLd + gn;
    } else {
      long long gn = n0 + (r - BM);
      if (gn > g.N - 1) gn = g.N - 1;
      src[j] = B + gn * g.bLd + kv * 8;
    }
  }
  const int nk = (int)(g.K / BK);
  auto issue = [&](auto stage, int slab) {   // stage == slab % STAGES, as a compile-time constant
    unsigned char* ring = stageBase<STAGE_BYTES, decltype(stage)::value>();
    const long long k0 = (long long)(slab < nk ? slab : nk - 1) * BK;   // past the end: harmless re-read keeps the count uniform
#pragma unroll
    for (int j = 0; j < NI; ++j) {
      unsigned char* dst = ring + (j * NW + wave) * 1024;
      // loads j >= BM / (8 NW) fill the B part; an n-contiguous B advances by rows
      const long long step = (BNN && j >= BM / (8 * NW)) ? k0 * g.bLd : k0;
      __builtin_amdgcn_global_load_lds(GLOBAL_PTR(src[j] + step), LDS_PTR(dst), 16, 0, 0);
    }
  };

  float16v acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

  // the bias values this lane adds at the end are fetched now, behind the first slabs
  float biasv[TN];
#pragma unroll
  for (int j = 0; j < TN; ++j) {
    const long long col = n0 + wn * (BN / 2) + j * 32 + (lane & 31);
    biasv[j] = 0.f;
    if (g.bias && col < g.N) biasv[j] = g.outBf16 ? __uint_as_float((u32)((const u16*)g.bias)[col] << 16) : ((const float*)g.bias)[col];
  }
  issue(Const<0>(), 0);
  if constexpr (STAGES > 2) issue(Const<1>(), 1);
  if constexpr (STAGES > 3) issue(Const<2>(), 2);
  static_assert(STAGES >= 2 && STAGES <= 4, "ring length");

  // fragment addresses: row-dependent part of the swizzle is fixed per lane
  const int arow = wm * (BM / WM) + (lane & 31);
  const int brow = BM + wn * (BN / 2) + (lane & 31);
  const int khalf = lane >> 5;
  // n-contiguous B: per-lane byte offset of its transposing reads inside a stage.  Lane d of a 16-lane group
  // addresses k-row khalf*8 + d/4 (+ a multiple of 4 per read, which leaves the swizzle unchanged) and
  // the 4 columns 4*(d%4) .. +3 of the group's 16.
  int bOff[TN];
  if (BNN) {
    const int d = lane & 15, nhalf = (lane >> 4) & 1;
    const int kLane = khalf * 8 + (d >> 2);
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const int slot = ((wn * (BN / 2) + j * 32) >> 3) + nhalf * 2 + ((d & 3) >> 1);
      bOff[j] = BM * 128 + kLane * (BN * 2) + ((slot ^ swzB<BN>(kLane)) << 4) + ((d & 1) << 3);
    }
  }
  auto step = [&](auto stage, int it) {
    constexpr int S = decltype(stage)::value;
    __builtin_amdgcn_s_waitcnt(vmcntImm((STAGES - 2) * NI));
    __builtin_amdgcn_s_barrier();
    issue(Const<(S + STAGES - 1) % STAGES>(), it + STAGES - 1);
    const unsigned char* st = stageBase<STAGE_BYTES, S>();
    // fragments of k-step kk+1 are requested before the products of k-step kk are issued
    bf16x8 av[2][TM], bv[2][TN];
    auto frags = [&](int kk, int p) {
#pragma unroll
      for (int i = 0; i < TM; ++i) {
        const int r = arow + i * 32;
        av[p][i] = *(const bf16x8*)(st + r * 128 + (((kk * 2 + khalf) ^ ((r >> 1) & 7)) << 4));
      }
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        if (BNN) {
          short4v h[2];
#pragma unroll
          for (int q = 0; q < 2; ++q)   // the step-dependent part of the address is a compile-time offset
            h[q] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) short4v*)(st + bOff[j] + (kk * 16 + q * 4) * (BN * 2)));
          short8v both = __builtin_shufflevector(h[0], h[1], 0, 1, 2, 3, 4, 5, 6, 7);
          bv[p][j] = __builtin_bit_cast(bf16x8, both);
        } else {
          const int r = brow + j * 32;
          bv[p][j] = *(const bf16x8*)(st + r * 128 + (((kk * 2 + khalf) ^ ((r >> 1) & 7)) << 4));
        }
      }
    };
    frags(0, 0);
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) {
      if (kk + 1 < 4) frags(kk + 1, (kk + 1) & 1);
      __builtin_amdgcn_sched_barrier(0);   // keep the reads ahead of the products: the scheduler would sink them to save registers
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(av[kk & 1][i], bv[kk & 1][j], acc[i][j], 0, 0, 0);
    }
    // every fragment read of this stage has returned before the next barrier lets a refill start
    __builtin_amdgcn_s_waitcnt((15) | (3 << 14) | (7 << 4) | (0 << 8));
  };
  int it = 0;
  for (; it + STAGES <= nk; it += STAGES) {   // whole turns of the ring, no branches inside
    step(Const<0>(), it);
    step(Const<1>(), it + 1);
    if constexpr (STAGES > 2) step(Const<2>(), it + 2);
    if constexpr (STAGES > 3) step(Const<3>(), it + 3);
  }
  // the last partial turn (nk is uniform, so every wavefront takes the same steps)
  if (it < nk) step(Const<0>(), it);
  if (it + 1 < nk) step(Const<1>(), it + 1);
  if constexpr (STAGES > 3) { if (it + 2 < nk) step(Const<2>(), it + 2); }
  __builtin_amdgcn_s_waitcnt(vmcntImm(0));   // drain the tail loads before the workgroup's LDS is released

  const long long cBase = bz * g.M * g.N;
  // value of accumulator element e of tile (i, j) as it is stored: bias added to the rounded product, then the activation
  auto finish16 = [&](float v, float bias) -> u16 {
    u16 r = to_bf16(v);
    if (g.bias) r = to_bf16(__uint_as_float((u32)r << 16) + bias);
    if (g.act == 1) {
      const float x = __uint_as_float((u32)r << 16);
      const float u = g.actC * (x + g.actB * (x * x * x));
      const float ex = __expf(2.f * fminf(u, 20.f));   // 1 + tanh(u) = 2 e^(2u) / (1 + e^(2u)): no cancellation for negative u
      r = to_bf16(g.actA * x * (2.f * ex * __builtin_amdgcn_rcpf(1.f + ex)));
    }
    return r;
  };
  if (g.outBf16 && (g.N & 7) == 0 && ((uintptr_t)g.c & 15) == 0) {
    // bf16 results leave through LDS: an accumulator lane holds 16 rows of one column, so direct stores are
    // 2-byte writes, 64 of them per instruction.  Each 64-row band of the tile is transposed through a ring
    // stage (free by now) and written as 16-byte row segments, whole cache lines per row.
    constexpr int LDW = BN + 8;   // staged row in elements: 16-byte aligned, consecutive rows 4 banks apart
    static_assert(64 * LDW * 2 <= STAGE_BYTES, "a band fits one stage");
    __syncthreads();              // every wavefront has read its last operands; all direct loads have landed
    // a band is 64 rows: the 32-row block i of two neighbouring wavefront rows (pair p)
#pragma unroll
    for (int b = 0; b < TM * (WM / 2); ++b) {
      const int i = b % TM, p = b / TM;
      u16* band = (u16*)((b & 1) ? stageBase<STAGE_BYTES, 1>() : stageBase<STAGE_BYTES, 0>());
      if ((wm >> 1) == p) {
#pragma unroll
        for (int j = 0; j < TN; ++j) {
          const int lc = wn * (BN / 2) + j * 32 + (lane & 31);
          const float bias = biasv[j];
#pragma unroll
          for (int e = 0; e < 16; ++e) {
            const int lr = (wm & 1) * 32 + (e >> 2) * 8 + (lane >> 5) * 4 + (e & 3);
            band[lr * LDW + lc] = finish16(acc[i][j][e], bias);
          }
        }
      }
      __syncthreads();   // also orders this band's reads of the other buffer's previous use before its next writes
      for (int sg = tid; sg < 64 * (BN / 8); sg += NT) {
        const int lr = sg / (BN / 8), cs = sg % (BN / 8);
        const long long row = m0 + (2 * p + (lr >> 5)) * (BM / WM) + i * 32 + (lr & 31);
        const long long col = n0 + cs * 8;
        if (row < g.M && col < g.N) *(uint4*)((u16*)g.c + cBase + row * g.N + col) = *(const uint4*)(band + lr * LDW + cs * 8);
      }
    }
  } else {
#pragma unroll
    for (int i = 0; i < TM; ++i) {
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        const long long col = n0 + wn * (BN / 2) + j * 32 + (lane & 31);
        if (col >= g.N) continue;
        // bias epilogue: the product is rounded to the output type first, as the separate add would see it
        const float bias = biasv[j];
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          const long long row = m0 + wm * (BM / WM) + i * 32 + (e >> 2) * 8 + (lane >> 5) * 4 + (e & 3);
          if (row >= g.M) continue;
          if (g.outBf16) ((u16*)g.c)[cBase + row * g.N + col] = finish16(acc[i][j][e], bias);
          else ((float*)g.c)[cBase + row * g.N + col] = acc[i][j][e] + bias;
        }
      }
    }
  }
}

template <int BM, int BN, int STAGES, bool BNN, int WM = 2>
int launch(const AsyncArgs& g, hipStream_t st) {
  gemm_bf16_async<BM, BN, STAGES, BNN, WM><<<dim3((unsigned)g.total), WM * 128, 0, st>>>(g);   // the ring is static LDS
  return hipGetLastError() == hipSuccess ? 0 : 3;
}

bool aligned16(const void* p) { return ((uintptr_t)p & 15) == 0; }

// out[b][x][k] = in[b0, b1][k][x]  (x contiguous in, k contiguous out), 64x64 tiles through LDS
struct TransposeArgs {
  const u16* in;
  u16* out;
  long long K, X, ld, inB0, inB1;
  int batch1;
};

__global__ void __launch_bounds__(256) transpose_bf16(TransposeArgs t) {
  __shared__ u16 tile[64][64 + 2];
  const int tid = threadIdx.x;
  const long long b0 = blockIdx.z / t.batch1, b1 = blockIdx.z % t.batch1;
  const u16* in = t.in + b0 * t.inB0 + b1 * t.inB1;
  u16* out = t.out + (long long)blockIdx.z * t.K * t.X;
  const long long k0 = (long long)blockIdx.y * 64, x0 = (long long)blockIdx.x * 64;
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int u = tid + 256 * i, k = u >> 3, xv = (u & 7) * 8;
    uint4 v = make_uint4(0, 0, 0, 0);
    if (k0 + k < t.K && x0 + xv < t.X) v = *(const uint4*)(in + (k0 + k) * t.ld + x0 + xv);
    const u16* e = (const u16*)&v;
#pragma unroll
    for (int q = 0; q < 8; ++q) tile[k][xv + q] = e[q];
  }
  __syncthreads();
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int u = tid + 256 * i, x = u >> 3, kv = (u & 7) * 8;
    if (x0 + x >= t.X || k0 + kv >= t.K) continue;
    uint4 v;
    u16* e = (u16*)&v;
#pragma unroll
    for (int q = 0; q < 8; ++q) e[q] = tile[kv + q][x];
    *(uint4*)(out + (x0 + x) * t.K + k0 + kv) = v;
  }
}

// How each operand reaches the k-contiguous layout the kernel needs.
struct OperandPlan {
  bool ok = false;
  bool copy = false;     // needs a transposed copy in the workspace
  bool rowsOfK = false;  // used in place as [K][rows] (B only): the kernel transposes while reading LDS
  long long ld = 0;      // row pitch when used in place
};

OperandPlan planOperand(long long rowStride, long long kStride, long long rows, long long K, long long other) {
  OperandPlan p;
  if (kStride == 1 && rowStride % 8 == 0) { p.ok = true; p.ld = rowStride; return p; }
  // laid out along the rows: worth a copy only when the other side is large enough to amortise it
  if (rowStride == 1 && kStride % 8 == 0 && rows % 8 == 0 && other >= 256) { p.ok = true; p.copy = true; p.ld = K; }
  return p;
}

bool qualifies(const mi355_gemm_desc* d, OperandPlan& pa, OperandPlan& pb) {
  if (d->in_dtype != 1 || (d->out_dtype != 0 && d->out_dtype != 1)) return false;
  const long long nb = d->batch0 * d->batch1;
  if (d->M <= 0 || d->N <= 0 || d->K <= 0 || nb <= 0 || nb > 65535) return false;
  if (d->K % 64 != 0) return false;
  pa = planOperand(d->aRow, d->aCol, d->M, d->K, d->N);
  pb = planOperand(d->bCol, d->bRow, d->N, d->K, d->M);
  // An n-contiguous B is read in place when that beats a transposed copy: the in-place kernel runs about a
  // sixth slower than the k-contiguous one on large products (measured), the copy costs a launch plus one pass over B.
  // MI355X_GEMM_NN=0 always copies, =2 never does.
  static const int nnMode = getenv("MI355X_GEMM_NN") ? atoi(getenv("MI355X_GEMM_NN")) : 1;
  if (nnMode != 0 && d->bCol == 1 && d->bRow % 8 == 0 && d->N % 8 == 0 && d->N >= 8 && d->bRow >= d->N) {
    const double nbd = (double)nb;
    const double gemmSeconds = 2.0 * nbd * (double)d->M * (double)d->N * (double)d->K / 450e12;
    const double copySeconds = 5e-6 + 4.0 * nbd * (double)d->N * (double)d->K / 5e12;
    if (nnMode == 2 || !pb.ok || 0.15 * gemmSeconds < copySeconds) {
      pb = OperandPlan();
      pb.ok = true; pb.rowsOfK = true; pb.ld = d->bRow;
    }
  }
  if (!pa.ok || !pb.ok) return false;
  if (d->batch0 > 1 && (d->aB0 % 8 || d->bB0 % 8)) return false;
  if (d->batch1 > 1 && (d->aB1 % 8 || d->bB1 % 8)) return false;
  return true;
}

size_t roundUp256(size_t b) { return (b + 255) / 256 * 256; }

int transposeInto(const u16* in, u16* out, long long K, long long X, long long ld, const mi355_gemm_desc* d, long long inB0, long long inB1,
                  hipStream_t st) {
  TransposeArgs t;
  t.in = in; t.out = out; t.K = K; t.X = X; t.ld = ld; t.inB0 = inB0; t.inB1 = inB1; t.batch1 = (int)d->batch1;
  dim3 grid((unsigned)((X + 63) / 64), (unsigned)((K + 63) / 64), (unsigned)(d->batch0 * d->batch1));
  transpose_bf16<<<grid, 256, 0, st>>>(t);
  return hipGetLastError() == hipSuccess ? 0 : 3;
}

}  // namespace

extern "C" size_t mi355_gemm_bf16_async_workspace_bytes(const mi355_gemm_desc* d) {
  OperandPlan pa, pb;
  if (!qualifies(d, pa, pb)) return 0;
  const size_t nb = (size_t)(d->batch0 * d->batch1);
  size_t bytes = 0;
  if (pa.copy) bytes += roundUp256(nb * (size_t)d->M * (size_t)d->K * 2);
  if (pb.copy) bytes += roundUp256(nb * (size_t)d->N * (size_t)d->K * 2);
  return bytes;
}

// 0 = launched, -1 = layout does not qualify, other = launch error.
extern "C" int mi355_gemm_bf16_async(const mi355_gemm_desc* d, const void* a, const void* b, void* c, const void* bias, void* workspace,
                                     size_t workspace_bytes, mi355_stream_t s) {
  OperandPlan pa, pb;
  if (!qualifies(d, pa, pb)) return -1;
  if (!aligned16(a) || !aligned16(b)) return -1;
  if ((pa.copy || pb.copy) && (workspace == nullptr || workspace_bytes < mi355_gemm_bf16_async_workspace_bytes(d) || !aligned16(workspace))) return -1;
  hipStream_t st = (hipStream_t)s;
  const long long nb = d->batch0 * d->batch1;
  AsyncArgs g;
  g.a = (const u16*)a; g.b = (const u16*)b; g.c = c;
  g.bias = bias;
  g.M = d->M; g.N = d->N; g.K = d->K;
  g.aB0 = d->aB0; g.aB1 = d->aB1; g.aLd = pa.ld;
  g.bB0 = d->bB0; g.bB1 = d->bB1; g.bLd = pb.ld;
  g.batch1 = (int)d->batch1;
  g.outBf16 = d->out_dtype == 1;
  if (d->act && !g.outBf16) return -1;
  g.act = d->act; g.actA = d->act_a; g.actB = d->act_b; g.actC = d->act_c;
  unsigned char* ws = (unsigned char*)workspace;
  if (pa.copy) {
    if (int r = transposeInto((const u16*)a, (u16*)ws, d->K, d->M, d->aCol, d, d->aB0, d->aB1, st)) return r;
    g.a = (const u16*)ws;
    g.aB1 = d->M * d->K; g.aB0 = g.aB1 * d->batch1;
    ws += roundUp256((size_t)nb * (size_t)d->M * (size_t)d->K * 2);
  }
  if (pb.copy) {
    if (int r = transposeInto((const u16*)b, (u16*)ws, d->K, d->N, d->bRow, d, d->bB0, d->bB1, st)) return r;
    g.b = (const u16*)ws;
    g.bB1 = d->N * d->K; g.bB0 = g.bB1 * d->batch1;
  }
  auto tiles = [&](int bm, int bn) { return ((d->M + bm - 1) / bm) * ((d->N + bn - 1) / bn) * nb; };
  // the largest tile that still leaves about three workgroups per compute unit
  int bm = 64, bn = 64;
  static const char* force = getenv("MI355X_GEMM_TILE");   // "256x128", "128x128", "128x64", "64x64": tuning aid
  if (force) sscanf(force, "%dx%d", &bm, &bn);
  else if (d->M > 128 && d->N > 64 && tiles(256, 128) >= 1024) { bm = 256; bn = 128; }
  // an in-place n-contiguous rhs wants twice as many 128x128 tiles before they pay (measured: 4096x768x3072 runs
  // 42 us on 128x64 tiles against 53 us on 768 tiles of 128x128)
  else if (d->M > 64 && d->N > 64 && tiles(128, 128) >= (pb.rowsOfK ? 1536 : 768)) { bm = 128; bn = 128; }
  else if (d->M > 64 && tiles(128, 64) >= 768) { bm = 128; bn = 64; }
  // The 256 x 256 tile (eight wavefronts) for large products with a long K.  Measured (k-contiguous / [K][N] rhs):
  // 8192^3 925 / 895 TFLOP/s against 857 / 818 on 256 x 128 tiles, 4096^3 864 / 821 against 719 / 694; with K = 768
  // (4096 x 2304 and 4096 x 3072 outputs) it is no faster or slower than the 128 x 64 tiles, and with fewer than 128 tiles
  // (N = 768) much slower.  One 64 KB stage in flight per compute unit does not cover the load latency (about 5 500
  // cycles per 64 of K against 2 048 of products), and the 160 KB of LDS hold no third stage of this tile.
  // MI355X_GEMM_WIDE=0 never, =2 whenever the shape allows.
  const int wideMode = getenv("MI355X_GEMM_WIDE") ? atoi(getenv("MI355X_GEMM_WIDE")) : 1;   // read at every call: tests switch it
  bool wide = false;
  if (!force && wideMode != 0 && d->M >= 256 && d->N >= 256)
    wide = wideMode == 2 || (tiles(256, 256) >= 192 && d->K >= 2048);
  if (wide) { bm = 256; bn = 256; }
  g.tilesM = (int)((d->M + bm - 1) / bm);
  g.tilesN = (int)((d->N + bn - 1) / bn);
  g.total = (long long)g.tilesM * g.tilesN * nb;
  if (g.total > 0x7FFFFFFFll) return -1;
  if (wide) return pb.rowsOfK ? launch<256, 256, 2, true, 4>(g, st) : launch<256, 256, 2, false, 4>(g, st);
  // two ring stages keep three workgroups of 128x64 resident per compute unit; deeper rings (MI355X_GEMM_STAGES=3|4, a tuning aid)
  // leave room for fewer and measured slower on the benchmark shapes: twelve resident wavefronts hide more than a third stage
  static const int stagesEnv = getenv("MI355X_GEMM_STAGES") ? atoi(getenv("MI355X_GEMM_STAGES")) : 0;
  if (pb.rowsOfK && stagesEnv) {
    if (bm == 128 && bn == 128) {
      if (stagesEnv == 3) return launch<128, 128, 3, true>(g, st);
      if (stagesEnv == 4) return launch<128, 128, 4, true>(g, st);
    } else if (bm == 128) {
      if (stagesEnv == 3) return launch<128, 64, 3, true>(g, st);
      if (stagesEnv == 4) return launch<128, 64, 4, true>(g, st);
    } else if (bm == 64) {
      if (stagesEnv == 3) return launch<64, 64, 3, true>(g, st);
      if (stagesEnv == 4) return launch<64, 64, 4, true>(g, st);
    }
  }
  if (pb.rowsOfK) {
    if (bm == 256) return launch<256, 128, 3, true>(g, st);
    if (bm == 128 && bn == 128) return launch<128, 128, 2, true>(g, st);
    if (bm == 128) return launch<128, 64, 2, true>(g, st);
    return launch<64, 64, 2, true>(g, st);
  }
  if (bm == 256) return launch<256, 128, 3, false>(g, st);
  if (bm == 128 && bn == 128) return launch<128, 128, 2, false>(g, st);
  if (bm == 128) return launch<128, 64, 2, false>(g, st);
  return launch<64, 64, 2, false>(g, st);
}
