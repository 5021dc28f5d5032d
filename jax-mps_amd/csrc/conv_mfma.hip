// Implicit-GEMM convolution on the fp32 matrix cores of gfx950.
//
//   out[b, o0, o1, f] = sum over (k0, k1, c) of lhs[b, pos0, pos1, c] * rhs[k0, k1, c, f]
//
// seen as C[M, N] = A[M, K] x B[K, N] with M = batch x output positions, N = output
// features, K = window taps x input features.  Every tensor is addressed through the
// element strides of its logical dims, so forward convolutions (NHWC x HWIO), input
// gradients (lhs dilation, reversed kernel with i/o swapped) and filter gradients
// (batch and feature swapped, rhs dilation) are the same kernel with different loaders:
//
//   A loader  K-vector: features contiguous in lhs      (forward, input gradient)
//             M-vector: conv-batch dim contiguous in lhs (filter gradient)
//             scalar  : anything else (3-channel stem, odd strides)
//   B loader  N-vector: output features contiguous in rhs (forward, filter gradient)
//             K-vector: input features contiguous in rhs  (input gradient)
//             scalar  : anything else
//
// A workgroup of four wavefronts owns a BM x BN tile (2 x 2 wavefronts, each WM x WN built
// from 32x32 accumulators of v_mfma_f32_32x32x2_f32).  Tiles of A and B go through two LDS
// stages and two register sets, so that a tile is being fetched two k-steps ahead of the
// one being multiplied.  Problems with few output tiles (filter gradients, late stages)
// split K across workgroups into partial sums that a second kernel folds in a fixed order,
// which keeps results reproducible.
//
// Two kernels share this scheme: conv_igemm_lean for the vector loaders (every large
// convolution; its k-loop carries next to no vector arithmetic, see the comment above it)
// and conv_igemm_f32 for the scalar loaders (a 3-channel stem, odd layouts), which computes
// every element's address and validity as it goes.  The lean kernel can also deliver the
// column sums and sums of squares of its output (batch-norm statistics), run several
// unsplit problems in one launch (the residue classes of an input-dilated convolution) and
// number the workgroups of a split launch by XCD.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstdint>
#include <vector>
#include <cstdlib>
#include <type_traits>

#include "hip_abi.h"

typedef float float16v __attribute__((ext_vector_type(16)));

namespace {

constexpr int BK = 16;

struct ConvP {
  const float* lhs;
  const float* rhs;
  float* out;       // final output, or partial sums [split][M][N] when splitK > 1
  int M, N, K;
  int Nb, C;
  int in0, in1, k0n, k1n, o0n, o1n;
  int kb0, ks0, kc0, kb1, ks1, kc1;   // window taps visited: kb + ks * t, t < kc (all of them unless a dilation class narrows it)
  int s0, s1, p0, p1, ld0, ld1, rd0, rd1, rev0, rev1;
  int lhsB, lhsF, lhsS0, lhsS1, rhsI, rhsO, rhsS0, rhsS1, outB, outF, outS0, outS1;
  int bFast;            // 1: m = (o0, o1, b) with b fastest; 0: m = (b, o0, o1)
  long long outRow;     // > 0: output row m starts at m * outRow (the usual dense layouts): no index decode when storing
  int outVec;           // columns are contiguous and every row of the destination (output or partial sums) starts 16-byte aligned: float4 stores
  int cTiles;           // k-tiles per window tap (tap-chunk tiling)
  int kTiles;           // total k-tiles
  int splitK, tilesPerSplit;
  unsigned lhsBytes, rhsBytes;   // sizes for the buffer descriptors of the vector-loader kernel (both below 2 GiB)
  int taps;                      // window taps this launch visits (kc0 * kc1)
  int tilesM, tilesXY;           // split launches of the vector-loader kernel: tile rows and tiles per K range (tilesXY 0: a 3-d grid)
  // Column statistics of the output taken from the accumulators (batch-norm's sum and sum of squares over all rows):
  // workgroup (tile row i, tile column) writes the sums over its rows to statSum[n * tile rows + i] / statSq[n * tile rows + i];
  // a later pass folds the tile rows in order.  Null when not wanted.
  float* statSum;
  float* statSq;
};

struct Row {
  int base;   // element offset of (b) in lhs; -1 when the row is outside M
  int i0, i1; // window origin in the dilated, padded input
};

__device__ __forceinline__ Row makeRow(const ConvP& p, int m) {
  Row r;
  if (m >= p.M) { r.base = -1; r.i0 = 0; r.i1 = 0; return r; }
  int b, o0, o1;
  if (p.bFast) { b = m % p.Nb; int t = m / p.Nb; o1 = t % p.o1n; o0 = t / p.o1n; }
  else { o1 = m % p.o1n; int t = m / p.o1n; o0 = t % p.o0n; b = t / p.o0n; }
  r.base = b * p.lhsB;
  r.i0 = o0 * p.s0 - p.p0;
  r.i1 = o1 * p.s1 - p.p1;
  return r;
}

// offset of the input element that window tap (k0, k1) touches for this row, or -1 (padding / dilation hole)
__device__ __forceinline__ int tapOffset(const ConvP& p, const Row& r, int k0, int k1) {
  if (r.base < 0) return -1;
  int q0 = r.i0 + k0 * p.rd0, q1 = r.i1 + k1 * p.rd1;
  if (q0 < 0 || q1 < 0) return -1;
  if (p.ld0 != 1) { if (q0 % p.ld0) return -1; q0 /= p.ld0; }
  if (p.ld1 != 1) { if (q1 % p.ld1) return -1; q1 /= p.ld1; }
  if (q0 >= p.in0 || q1 >= p.in1) return -1;
  return r.base + q0 * p.lhsS0 + q1 * p.lhsS1;
}

__device__ __forceinline__ int rhsTapOffset(const ConvP& p, int k0, int k1) {
  int a = p.rev0 ? p.k0n - 1 - k0 : k0, b = p.rev1 ? p.k1n - 1 - k1 : k1;
  return a * p.rhsS0 + b * p.rhsS1;
}

// Writes a workgroup's accumulators.  The products were issued with their operands swapped, so a lane holds the
// transposed tile: one output row (lane & 31) and, per group of four accumulator registers, four consecutive output
// columns.  A lane decodes one row per 32-row block instead of sixteen, and stores 16 bytes at a time where the
// layout allows.
template <int TM, int TN, int WM, int WN>
__device__ __forceinline__ void storeAccumulators(const ConvP& p, float16v (&acc)[TM][TN], int m0, int n0, int wm, int wn, int lane, int split) {
  const bool partial = p.splitK > 1;
  const bool vec = p.outVec != 0;
#pragma unroll
  for (int a = 0; a < TM; ++a) {
    const int m = m0 + wm * WM + a * 32 + (lane & 31);
    if (m >= p.M) continue;
    long long rowOff;
    if (partial) {
      rowOff = ((long long)split * p.M + m) * p.N;
    } else if (p.outRow > 0) {
      rowOff = (long long)m * p.outRow;
    } else {
      int b, o0, o1;
      if (p.bFast) { b = m % p.Nb; int t = m / p.Nb; o1 = t % p.o1n; o0 = t / p.o1n; }
      else { o1 = m % p.o1n; int t = m / p.o1n; o0 = t % p.o0n; b = t / p.o0n; }
      rowOff = (long long)b * p.outB + (long long)o0 * p.outS0 + (long long)o1 * p.outS1;
    }
    const long long colStride = partial ? 1 : p.outF;
#pragma unroll
    for (int b = 0; b < TN; ++b) {
#pragma unroll
      for (int g4 = 0; g4 < 4; ++g4) {
        const int n = n0 + wn * WN + b * 32 + g4 * 8 + (lane >> 5) * 4;
        if (n >= p.N) continue;
        if (vec) {
          *(float4*)(p.out + rowOff + n) = make_float4(acc[a][b][4 * g4], acc[a][b][4 * g4 + 1], acc[a][b][4 * g4 + 2], acc[a][b][4 * g4 + 3]);
        } else {
#pragma unroll
          for (int r = 0; r < 4; ++r)
            if (n + r < p.N) p.out[rowOff + (n + r) * colStride] = acc[a][b][4 * g4 + r];
        }
      }
    }
  }
}

// wavefronts per SIMD the register budget is held to: four workgroups per CU for the vector loaders of the narrower tiles
constexpr int wavesPerSimd(int bm, int bn, int amode, int bmode) { return bm * bn == 128 * 128 ? 2 : (amode == 0 || bmode == 0 ? 3 : 4); }

template <int BM, int BN, int AMODE, int BMODE, bool KFLAT>
__global__ void __launch_bounds__(256, wavesPerSimd(BM, BN, AMODE, BMODE)) conv_igemm_f32(ConvP p) {
  constexpr int WM = BM / 2, WN = BN / 2, TM = WM / 32, TN = WN / 32;
  constexpr int NA4 = BM / 64, NB4 = BN / 64;            // float4 per thread per tile (vector loaders)
  constexpr int NAS = BM * BK / 256, NBS = BN * BK / 256; // floats per thread per tile (scalar loaders)
  // k-major tiles, two stages.  Row padding: 2 floats make the transposing (K-vector) stores
  // conflict-free, 4 floats keep the float4 stores of the M/N-vector loaders 16-byte aligned.
  constexpr int PA = AMODE == 1 ? 2 : 4, PB = BMODE == 2 ? 2 : 4;
  __shared__ __attribute__((aligned(16))) float As[2][BK][BM + PA];
  __shared__ __attribute__((aligned(16))) float Bs[2][BK][BN + PB];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  // Workgroups go to the eight XCDs round-robin by linear id; tiles that are neighbours along M share window rows,
  // so each XCD (one L2) takes a contiguous band of M tiles when the grid allows it.
  int bx = blockIdx.x;
  if ((gridDim.x & 7) == 0) bx = (bx & 7) * (gridDim.x >> 3) + (bx >> 3);
  const int m0 = bx * BM, n0 = blockIdx.y * BN;
  const int ktBegin = blockIdx.z * p.tilesPerSplit;
  const int ktEnd = min(p.kTiles, ktBegin + p.tilesPerSplit);

  // ---- per-thread rows of the A tile (fixed for the whole K loop)
  Row rowsA[AMODE == 0 ? NAS : NA4];
  if (AMODE == 1) {
#pragma unroll
    for (int i = 0; i < NA4; ++i) rowsA[i] = makeRow(p, m0 + (tid >> 2) + 64 * i);
  } else if (AMODE == 2) {
    rowsA[0] = makeRow(p, m0 + 4 * (tid % (BM / 4)));     // 4 consecutive m share (o0, o1); b .. b+3 are contiguous
#pragma unroll
    for (int i = 1; i < NA4; ++i) rowsA[i] = rowsA[0];
  } else {
#pragma unroll
    for (int i = 0; i < NAS; ++i) rowsA[i] = makeRow(p, m0 + (tid + 256 * i) / BK);
  }

  // two register sets: the tile after next is already on its way while the next one is written to LDS
  float4 ra[2][NA4 > 0 ? NA4 : 1];
  float4 rb[2][NB4 > 0 ? NB4 : 1];
  float ras[2][NAS], rbs[2][NBS];

  // Position of the next k-tile to fetch, advanced incrementally (no divisions in the loop):
  // window tap (nk0, nk1) and first input feature nc.  Row offsets and validity only change
  // when the tap changes, so they are cached per tap.
  int nk0 = 0, nk1 = 0, nc = 0;
  if (!KFLAT) {
    int tap = ktBegin / p.cTiles;
    nc = (ktBegin - tap * p.cTiles) * BK;
    nk0 = tap / p.kc1;
    nk1 = tap - nk0 * p.kc1;
  }
  constexpr int NROW = AMODE == 0 ? NAS : (AMODE == 1 ? NA4 : 1);
  int offA[NROW];
  int toffB = 0;
  auto newTap = [&]() {
    if (KFLAT) return;
#pragma unroll
    for (int i = 0; i < NROW; ++i) offA[i] = tapOffset(p, rowsA[i], p.kb0 + p.ks0 * nk0, p.kb1 + p.ks1 * nk1);
    toffB = rhsTapOffset(p, p.kb0 + p.ks0 * nk0, p.kb1 + p.ks1 * nk1);
  };
  newTap();
  // per-thread constants of the loaders
  const int aKq = (tid & 3) * 4;
  const int aKr = tid / (BM / 4);
  const int bNq = 4 * (tid % (BN / 4));
  const int bKr = tid / (BN / 4);
  const bool bNok = n0 + bNq < p.N;

  // Loads are unconditional: an element outside the input, the filter or K is read from offset 0 of its tensor and
  // replaced by zero when the tile is written to LDS (a load under a branch would make the compiler drain every
  // outstanding load before issuing the next ones, which defeats fetching two tiles ahead).
  unsigned okA[2] = {0, 0}, okB[2] = {0, 0};
  auto loadTile = [&](int kt, auto setTag) {
    constexpr int S = decltype(setTag)::value;
    okA[S] = 0; okB[S] = 0;
    // ---------------- A
    if (AMODE == 1) {
#pragma unroll
      for (int i = 0; i < NA4; ++i)
        { const bool ok = offA[i] >= 0; ra[S][i] = *(const float4*)(p.lhs + (unsigned)((ok ? offA[i] : 0) + nc + aKq)); okA[S] |= (unsigned)ok << i; }
    } else if (AMODE == 2) {
#pragma unroll
      for (int i = 0; i < NA4; ++i) {
        int kr = aKr + (1024 / BM) * i;
        const bool ok = offA[0] >= 0;
        ra[S][i] = *(const float4*)(p.lhs + (unsigned)((ok ? offA[0] : 0) + (nc + kr) * p.lhsF));
        okA[S] |= (unsigned)ok << i;
      }
    } else {
#pragma unroll
      for (int i = 0; i < NAS; ++i) {
        int k = (tid + 256 * i) % BK;
        int off, c = nc + k;
        if (KFLAT) {
          int kf = kt * BK + k;
          int t = kf / p.C;
          c = kf - t * p.C;
          int kk0 = t / p.k1n;
          off = kf < p.K ? tapOffset(p, rowsA[i], kk0, t - kk0 * p.k1n) : -1;
        } else {
          off = offA[i];
        }
        ras[S][i] = p.lhs[off >= 0 ? off + c * p.lhsF : 0];
        okA[S] |= (unsigned)(off >= 0) << i;
      }
    }
    // ---------------- B
    if (BMODE == 1) {
#pragma unroll
      for (int i = 0; i < NB4; ++i) {
        int kr = bKr + (1024 / BN) * i;
        rb[S][i] = *(const float4*)(p.rhs + (unsigned)(toffB + (nc + kr) * p.rhsI + (bNok ? n0 + bNq : 0)));
        okB[S] |= (unsigned)bNok << i;
      }
    } else if (BMODE == 2) {
#pragma unroll
      for (int i = 0; i < NB4; ++i) {
        int n = n0 + (tid >> 2) + 64 * i;
        rb[S][i] = *(const float4*)(p.rhs + (unsigned)(toffB + (n < p.N ? n : 0) * p.rhsO + nc + aKq));
        okB[S] |= (unsigned)(n < p.N) << i;
      }
    } else {
#pragma unroll
      for (int i = 0; i < NBS; ++i) {
        int e = tid + 256 * i;
        int n = n0 + e % BN, k = e / BN;
        int c = nc + k, toff = toffB;
        bool ok = n < p.N;
        if (KFLAT) {
          int kf = kt * BK + k;
          ok = ok && kf < p.K;
          int t = kf / p.C;
          c = kf - t * p.C;
          int kk0 = t / p.k1n;
          toff = rhsTapOffset(p, kk0, t - kk0 * p.k1n);
        }
        rbs[S][i] = p.rhs[ok ? toff + c * p.rhsI + n * p.rhsO : 0];
        okB[S] |= (unsigned)ok << i;
      }
    }
    // ---------------- advance to the following tile
    if (!KFLAT) {
      nc += BK;
      if (nc >= p.C) {
        nc = 0;
        if (++nk1 == p.kc1) { nk1 = 0; ++nk0; }
        newTap();
      }
    }
  };

  auto storeTile = [&](auto stageTag, auto setTag) {
    constexpr int st = decltype(stageTag)::value;   // compile-time stage: every LDS address is a per-thread base plus an immediate
    constexpr int S = decltype(setTag)::value;
    if (AMODE == 1) {
      const int kq = (tid & 3) * 4;
#pragma unroll
      for (int i = 0; i < NA4; ++i) {
        int m = (tid >> 2) + 64 * i;
        if (!((okA[S] >> i) & 1)) ra[S][i] = make_float4(0.f, 0.f, 0.f, 0.f);
        As[st][kq + 0][m] = ra[S][i].x; As[st][kq + 1][m] = ra[S][i].y; As[st][kq + 2][m] = ra[S][i].z; As[st][kq + 3][m] = ra[S][i].w;
      }
    } else if (AMODE == 2) {
#pragma unroll
      for (int i = 0; i < NA4; ++i) {
        int kr = tid / (BM / 4) + (1024 / BM) * i;
        *(float4*)&As[st][kr][4 * (tid % (BM / 4))] = ((okA[S] >> i) & 1) ? ra[S][i] : make_float4(0.f, 0.f, 0.f, 0.f);
      }
    } else {
#pragma unroll
      for (int i = 0; i < NAS; ++i) { int e = tid + 256 * i; As[st][e % BK][e / BK] = ((okA[S] >> i) & 1) ? ras[S][i] : 0.f; }
    }
    if (BMODE == 1) {
#pragma unroll
      for (int i = 0; i < NB4; ++i) {
        int kr = tid / (BN / 4) + (1024 / BN) * i;
        *(float4*)&Bs[st][kr][4 * (tid % (BN / 4))] = ((okB[S] >> i) & 1) ? rb[S][i] : make_float4(0.f, 0.f, 0.f, 0.f);
      }
    } else if (BMODE == 2) {
      const int kq = (tid & 3) * 4;
#pragma unroll
      for (int i = 0; i < NB4; ++i) {
        int n = (tid >> 2) + 64 * i;
        if (!((okB[S] >> i) & 1)) rb[S][i] = make_float4(0.f, 0.f, 0.f, 0.f);
        Bs[st][kq + 0][n] = rb[S][i].x; Bs[st][kq + 1][n] = rb[S][i].y; Bs[st][kq + 2][n] = rb[S][i].z; Bs[st][kq + 3][n] = rb[S][i].w;
      }
    } else {
#pragma unroll
      for (int i = 0; i < NBS; ++i) { int e = tid + 256 * i; Bs[st][e / BN][e % BN] = ((okB[S] >> i) & 1) ? rbs[S][i] : 0.f; }
    }
  };

  float16v acc[TM][TN];
#pragma unroll
  for (int a = 0; a < TM; ++a)
#pragma unroll
    for (int b = 0; b < TN; ++b) acc[a][b] = (float16v){0};

  if (ktBegin < ktEnd) {
    std::integral_constant<int, 0> s0;
    std::integral_constant<int, 1> s1;
    const int kh = lane >> 5, col = lane & 31;
    auto multiply = [&](auto stageTag) {
      constexpr int cur = decltype(stageTag)::value;
      __builtin_amdgcn_s_setprio(2);       // a wavefront that has its operands wins the matrix pipe over ones still fetching
#pragma unroll
      for (int kk = 0; kk < BK; kk += 2) {
        float av[TM], bv[TN];
#pragma unroll
        for (int a = 0; a < TM; ++a) av[a] = As[cur][kk + kh][wm * WM + a * 32 + col];
#pragma unroll
        for (int b = 0; b < TN; ++b) bv[b] = Bs[cur][kk + kh][wn * WN + b * 32 + col];
#pragma unroll
        for (int a = 0; a < TM; ++a)
#pragma unroll
          for (int b = 0; b < TN; ++b) acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x2f32(bv[b], av[a], acc[a][b], 0, 0, 0);   // operands swapped: the transposed tile
      }
      __builtin_amdgcn_s_setprio(0);
    };
    // Tile kt is multiplied from LDS while tile kt + 1 waits in one register set and tile kt + 2 is being fetched
    // into the other: a global load has two multiply phases to arrive before anyone waits for it.
    loadTile(ktBegin, s0);
    storeTile(s0, s0);
    if (ktBegin + 1 < ktEnd) loadTile(ktBegin + 1, s0);
    __syncthreads();
    int kt = ktBegin;
    // Steady state: every fetch is unconditional, so that the wait before an LDS write covers only the older register
    // set (a fetch under a condition would make the compiler wait for the newer loads as well).  Each half works on
    // a fixed LDS stage: tile kt in stage 0, tile kt + 1 in stage 1.
    for (; kt + 3 < ktEnd; kt += 2) {
      loadTile(kt + 2, s1);
      multiply(s0);
      storeTile(s1, s0);                    // the other stage: nobody reads it during this half
      __syncthreads();
      loadTile(kt + 3, s0);
      multiply(s1);
      storeTile(s0, s1);
      __syncthreads();
    }
    for (; kt < ktEnd; kt += 2) {           // the last one to three tiles
      if (kt + 2 < ktEnd) loadTile(kt + 2, s1);
      multiply(s0);
      if (kt + 1 < ktEnd) storeTile(s1, s0);
      __syncthreads();
      if (kt + 1 >= ktEnd) break;
      multiply(s1);
      if (kt + 2 < ktEnd) storeTile(s0, s1);
      __syncthreads();
    }
  }

  storeAccumulators<TM, TN, WM, WN>(p, acc, m0, n0, wm, wn, lane, (int)blockIdx.z);
}

// ---------------------------------------------------------------------------------------------------------------
// The kernel for the vector loaders (every large convolution of a training step).  An fp32 MFMA occupies the SIMD
// for 64 cycles and every other vector instruction costs about four of them, so the k-loop is stripped of vector
// arithmetic: tiles are fetched with buffer loads whose per-lane offset changes only when the window tap changes
// (the advance along the features is a scalar offset), an element outside the input, the filter or N is given an
// offset beyond the buffer and comes back as zero from the hardware range check (no selects, no masks), per-tap row
// offsets come from a table in LDS filled once per workgroup when the window is small enough, and both LDS stages
// are compile-time so every LDS address is a per-lane base plus an immediate.
typedef unsigned int uint4v __attribute__((ext_vector_type(4)));
constexpr unsigned kOutside = 0x80000000u;     // an offset no tensor reaches (tensors stay below 2 GiB here)
constexpr int kTapTableBytes = 16384;          // largest per-workgroup tap table

template <int BM, int BN, int AMODE, int BMODE, bool TABLE>
__device__ __forceinline__ void leanBody(const ConvP& p, int split) {
  constexpr int WM = BM / 2, WN = BN / 2, TM = WM / 32, TN = WN / 32;
  constexpr int NA4 = BM / 64, NB4 = BN / 64;
  // A tile fetched with K-vectors stays row-major in LDS ([row or column][k], rows 20 floats apart): a fetched vector
  // is one 16-byte LDS write, and a lane reads its operands for four MFMA steps with one 16-byte read.  The order of k
  // inside a tile is free as long as both operands agree, so lane half h takes k = 8q + 4h + j for step (q, j).  Tiles
  // fetched with M- or N-vectors are k-major ([k][row or column]) and follow the same order of k.
  constexpr bool AROW = AMODE == 1, BROW = BMODE == 2, PERM = AROW || BROW;
  constexpr int RS = BK + 4;
  constexpr int LDA = BM + 4, LDB = BN + 4;
  constexpr int ASTAGE = AROW ? BM * RS : BK * LDA, BSTAGE = BROW ? BN * RS : BK * LDB;
  __shared__ __attribute__((aligned(16))) float As[2 * ASTAGE];
  __shared__ __attribute__((aligned(16))) float Bs[2 * BSTAGE];
  extern __shared__ unsigned tapTab[];        // [tap][row of the tile]: byte offset of (row, tap, feature 0) or kOutside

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  int bx = blockIdx.x, by = blockIdx.y;
  if (p.tilesXY > 0) {
    // A launch that splits K is one-dimensional: workgroups go to the eight XCDs round-robin by their number, and the
    // numbering here puts all output tiles of one K range on the same XCD, next to each other, so that the tiles of
    // an operand they share (every tile row reads the same rhs tiles, neighbouring taps the same lhs rows) meet in one L2.
    const int xcd = bx & 7, slot = bx >> 3;
    const int group = slot / p.tilesXY, t = slot - group * p.tilesXY;
    split = xcd + 8 * group;
    if (split >= p.splitK) return;
    by = t / p.tilesM;
    bx = t - by * p.tilesM;
  } else if ((gridDim.x & 7) == 0) {
    bx = (bx & 7) * (gridDim.x >> 3) + (bx >> 3);
  }
  const int m0 = bx * BM, n0 = by * BN;
  if (m0 >= p.M) return;                      // (a launch shared by several problems is as wide as the widest)
  const int ktBegin = split * p.tilesPerSplit;
  const int ktEnd = min(p.kTiles, ktBegin + p.tilesPerSplit);

  const __amdgpu_buffer_rsrc_t rsA = __builtin_amdgcn_make_buffer_rsrc((void*)p.lhs, 0, (int)p.lhsBytes, 0x00020000);
  const __amdgpu_buffer_rsrc_t rsB = __builtin_amdgcn_make_buffer_rsrc((void*)p.rhs, 0, (int)p.rhsBytes, 0x00020000);

  // rows of the A tile this lane fetches: NA4 rows 64 apart (K-vector), or one group of four consecutive rows (M-vector)
  constexpr int NROW = AMODE == 1 ? NA4 : 1;
  int rowInTile[NROW];
#pragma unroll
  for (int i = 0; i < NROW; ++i) rowInTile[i] = AMODE == 1 ? (tid >> 2) + 64 * i : 4 * (tid % (BM / 4));
  Row rowsA[TABLE ? 1 : NROW];
  if (!TABLE) {
#pragma unroll
    for (int i = 0; i < NROW; ++i) rowsA[i] = makeRow(p, m0 + rowInTile[i]);
  } else {
    const Row r = makeRow(p, m0 + tid % BM);
    for (int t = tid / BM; t < p.taps; t += 256 / BM) {
      const int t0 = t / p.kc1, t1 = t - t0 * p.kc1;
      const int off = tapOffset(p, r, p.kb0 + p.ks0 * t0, p.kb1 + p.ks1 * t1);
      tapTab[t * BM + tid % BM] = off >= 0 ? (unsigned)off * 4u : kOutside;
    }
    __syncthreads();
  }

  // position of the next k-tile to fetch: window tap (nk0, nk1) and first feature nc, all uniform
  // (integer division runs on the vector unit; the results are the same in every lane and are moved to scalar registers)
  int tap = __builtin_amdgcn_readfirstlane(ktBegin / p.cTiles);
  int nc = (ktBegin - tap * p.cTiles) * BK;
  int nk0 = __builtin_amdgcn_readfirstlane(tap / p.kc1), nk1 = tap - nk0 * p.kc1;
  const int aKq = (tid & 3) * 4;
  unsigned aFix[NA4];          // the part of a lane's A offset that never changes
#pragma unroll
  for (int i = 0; i < NA4; ++i) aFix[i] = AMODE == 1 ? (unsigned)aKq * 4u : (unsigned)((tid / (BM / 4) + (1024 / BM) * i) * p.lhsF) * 4u;
  unsigned aV[NA4], bV[NB4];
#pragma unroll
  for (int i = 0; i < NB4; ++i) {
    if (BMODE == 1) {
      const int nq = 4 * (tid % (BN / 4)), kr = tid / (BN / 4) + (1024 / BN) * i;
      bV[i] = n0 + nq < p.N ? (unsigned)(kr * p.rhsI + n0 + nq) * 4u : kOutside;
    } else {
      const int n = n0 + (tid >> 2) + 64 * i;
      bV[i] = n < p.N ? (unsigned)(n * p.rhsO + aKq) * 4u : kOutside;
    }
  }
  int toffB = 0;
  auto newTap = [&]() {
    const int k0 = p.kb0 + p.ks0 * nk0, k1 = p.kb1 + p.ks1 * nk1;
#pragma unroll
    for (int i = 0; i < NROW; ++i) {
      unsigned o;
      if (TABLE) {
        o = tapTab[tap * BM + rowInTile[i]];
      } else {
        const int off = tapOffset(p, rowsA[i], k0, k1);
        o = off >= 0 ? (unsigned)off * 4u : kOutside;
      }
      if (AMODE == 1) {
        aV[i] = o + aFix[i];
      } else {
#pragma unroll
        for (int j = 0; j < NA4; ++j) aV[j] = o + aFix[j];
      }
    }
    toffB = __builtin_amdgcn_readfirstlane(rhsTapOffset(p, k0, k1));
  };
  newTap();

  float4 ra[2][NA4], rb[2][NB4];   // two register sets: the tile after next is on its way while the next one goes to LDS
  auto loadTile = [&](auto setTag) {
    constexpr int S = decltype(setTag)::value;
    const unsigned sA = (unsigned)(AMODE == 1 ? nc : nc * p.lhsF) * 4u;
    const unsigned sB = (unsigned)(BMODE == 1 ? toffB + nc * p.rhsI : toffB + nc) * 4u;
#pragma unroll
    for (int i = 0; i < NA4; ++i) ra[S][i] = __builtin_bit_cast(float4, __builtin_amdgcn_raw_buffer_load_b128(rsA, (int)aV[i], (int)sA, 0));
#pragma unroll
    for (int i = 0; i < NB4; ++i) rb[S][i] = __builtin_bit_cast(float4, __builtin_amdgcn_raw_buffer_load_b128(rsB, (int)bV[i], (int)sB, 0));
    nc += BK;
    if (nc >= p.C) {
      nc = 0;
      ++tap;
      if (++nk1 == p.kc1) { nk1 = 0; ++nk0; }
      if (tap < p.taps) newTap();
    }
  };

  // LDS write positions (per lane, stage 0)
  float* const aWr = AROW ? As + (tid >> 2) * RS + aKq : As + (tid / (BM / 4)) * LDA + 4 * (tid % (BM / 4));
  float* const bWr = BROW ? Bs + (tid >> 2) * RS + aKq : Bs + (tid / (BN / 4)) * LDB + 4 * (tid % (BN / 4));
  auto storeTile = [&](auto stageTag, auto setTag) {
    constexpr int ST = decltype(stageTag)::value, S = decltype(setTag)::value;
#pragma unroll
    for (int i = 0; i < NA4; ++i) {
      if (AROW) *(float4*)(aWr + ST * ASTAGE + 64 * i * RS) = ra[S][i];
      else *(float4*)(aWr + ST * ASTAGE + (1024 / BM) * i * LDA) = ra[S][i];
    }
#pragma unroll
    for (int i = 0; i < NB4; ++i) {
      if (BROW) *(float4*)(bWr + ST * BSTAGE + 64 * i * RS) = rb[S][i];
      else *(float4*)(bWr + ST * BSTAGE + (1024 / BN) * i * LDB) = rb[S][i];
    }
  };

  float16v acc[TM][TN];
#pragma unroll
  for (int a = 0; a < TM; ++a)
#pragma unroll
    for (int b = 0; b < TN; ++b) acc[a][b] = (float16v){0};

  if (ktBegin < ktEnd) {
    std::integral_constant<int, 0> s0;
    std::integral_constant<int, 1> s1;
    const int kh = lane >> 5, col = lane & 31;
    const float* const aRd = AROW ? As + (wm * WM + col) * RS + 4 * kh : As + (PERM ? 4 * kh : kh) * LDA + wm * WM + col;
    const float* const bRd = BROW ? Bs + (wn * WN + col) * RS + 4 * kh : Bs + (PERM ? 4 * kh : kh) * LDB + wn * WN + col;
    auto multiply = [&](auto stageTag) {
      constexpr int ST = decltype(stageTag)::value;
      __builtin_amdgcn_s_setprio(2);       // a wavefront that has its operands wins the matrix pipe over ones still fetching
      if (PERM) {
#pragma unroll
        for (int q = 0; q < BK / 8; ++q) {
          float av[TM][4], bv[TN][4];
#pragma unroll
          for (int a = 0; a < TM; ++a) {
            if (AROW) {
              const float4 v = *(const float4*)(aRd + ST * ASTAGE + a * 32 * RS + 8 * q);
              av[a][0] = v.x; av[a][1] = v.y; av[a][2] = v.z; av[a][3] = v.w;
            } else {
#pragma unroll
              for (int j = 0; j < 4; ++j) av[a][j] = aRd[ST * ASTAGE + (8 * q + j) * LDA + a * 32];
            }
          }
#pragma unroll
          for (int b = 0; b < TN; ++b) {
            if (BROW) {
              const float4 v = *(const float4*)(bRd + ST * BSTAGE + b * 32 * RS + 8 * q);
              bv[b][0] = v.x; bv[b][1] = v.y; bv[b][2] = v.z; bv[b][3] = v.w;
            } else {
#pragma unroll
              for (int j = 0; j < 4; ++j) bv[b][j] = bRd[ST * BSTAGE + (8 * q + j) * LDB + b * 32];
            }
          }
#pragma unroll
          for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int a = 0; a < TM; ++a)
#pragma unroll
              for (int b = 0; b < TN; ++b) acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x2f32(bv[b][j], av[a][j], acc[a][b], 0, 0, 0);   // operands swapped: the transposed tile
        }
      } else {
#pragma unroll
        for (int kk = 0; kk < BK; kk += 2) {
          float av[TM], bv[TN];
#pragma unroll
          for (int a = 0; a < TM; ++a) av[a] = aRd[ST * ASTAGE + kk * LDA + a * 32];
#pragma unroll
          for (int b = 0; b < TN; ++b) bv[b] = bRd[ST * BSTAGE + kk * LDB + b * 32];
#pragma unroll
          for (int a = 0; a < TM; ++a)
#pragma unroll
            for (int b = 0; b < TN; ++b) acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x2f32(bv[b], av[a], acc[a][b], 0, 0, 0);
        }
      }
      __builtin_amdgcn_s_setprio(0);
    };
    // Tile kt is multiplied from LDS stage 0 while tile kt + 1 waits in one register set and tile kt + 2 is being
    // fetched into the other: a load has two multiply phases to arrive before anyone waits for it.  Fetches in the
    // steady state are unconditional, so the wait before an LDS write covers only the older register set.
    loadTile(s0);
    storeTile(s0, s0);
    if (ktBegin + 1 < ktEnd) loadTile(s0);
    __syncthreads();
    int kt = ktBegin;
    for (; kt + 3 < ktEnd; kt += 2) {
      loadTile(s1);
      multiply(s0);
      storeTile(s1, s0);                    // the other stage: nobody reads it during this half
      __syncthreads();
      loadTile(s0);
      multiply(s1);
      storeTile(s0, s1);
      __syncthreads();
    }
    for (; kt < ktEnd; kt += 2) {           // the last one to three tiles
      if (kt + 2 < ktEnd) loadTile(s1);
      multiply(s0);
      if (kt + 1 < ktEnd) storeTile(s1, s0);
      __syncthreads();
      if (kt + 1 >= ktEnd) break;
      multiply(s1);
      if (kt + 2 < ktEnd) storeTile(s0, s1);
      __syncthreads();
    }
  }

  storeAccumulators<TM, TN, WM, WN>(p, acc, m0, n0, wm, wn, lane, split);

  if (p.statSum != nullptr) {
    // Per-column sums over the workgroup's rows (rows past M hold zeros).  Each wavefront lays its 32 x 32 block
    // (summed over its row blocks) into LDS, lane l < 32 then adds column l and lane 32 + l the squares of column l,
    // in row order; the two wavefront rows are combined through LDS and one of them writes.  The tiles of the K
    // loop are dead by now, so their LDS is reused: 32 x 33 floats per wavefront.
    __syncthreads();
    constexpr int LDT = 33;
    static_assert(2 * 32 * LDT <= 2 * ASTAGE && 2 * 32 * LDT <= 2 * BSTAGE, "statistics scratch does not fit the tile buffers");
    float* const scratch = (wave < 2 ? As : Bs) + (wave & 1) * 32 * LDT;
    __shared__ float colPart[2][2][2][TN * 32];   // [wave row][wave column][sum / squares][column]
    const int row = lane & 31, half = lane >> 5;
#pragma unroll
    for (int b = 0; b < TN; ++b) {
      // squares need the rows apart, so each 32-row block goes through the scratch on its own
      float s = 0.f;
#pragma unroll
      for (int a = 0; a < TM; ++a) {
#pragma unroll
        for (int g4 = 0; g4 < 4; ++g4)
#pragma unroll
          for (int r = 0; r < 4; ++r) scratch[row * LDT + g4 * 8 + half * 4 + r] = acc[a][b][4 * g4 + r];
        __syncthreads();
#pragma unroll 8
        for (int i = 0; i < 32; ++i) {
          const float v = scratch[i * LDT + row];
          s += half ? v * v : v;
        }
        __syncthreads();
      }
      colPart[wm][wn][half][b * 32 + row] = s;
    }
    __syncthreads();
    if (wm == 0) {
#pragma unroll
      for (int b = 0; b < TN; ++b) {
        const int n = n0 + wn * WN + b * 32 + row;
        if (n < p.N) {
          const float v = colPart[0][wn][half][b * 32 + row] + colPart[1][wn][half][b * 32 + row];
          (half ? p.statSq : p.statSum)[(size_t)n * gridDim.x + bx] = v;
        }
      }
    }
  }
}

template <int BM, int BN, int AMODE, int BMODE, bool TABLE>
__global__ void __launch_bounds__(256, wavesPerSimd(BM, BN, AMODE, BMODE)) conv_igemm_lean(ConvP p) {
  leanBody<BM, BN, AMODE, BMODE, TABLE>(p, (int)blockIdx.z);
}

// Several unsplit problems of one convolution (the residue classes of an input-dilated one) as one launch:
// blockIdx.z picks the problem.  Each class alone is a short K loop over few workgroups; together they fill the device.
constexpr int kMaxPack = 4;
struct ConvPack { ConvP c[kMaxPack]; };

template <int BM, int BN, int AMODE, int BMODE, bool TABLE>
__global__ void __launch_bounds__(256, wavesPerSimd(BM, BN, AMODE, BMODE)) conv_igemm_lean_pack(ConvPack ps) {
  leanBody<BM, BN, AMODE, BMODE, TABLE>(ps.c[blockIdx.z], 0);
}

// out(m, n) = sum over splits of partial[s][m][n].  32 consecutive outputs per workgroup, the
// splits dealt round-robin to 8 groups of lanes whose sums are then added in group order, so
// the result depends only on the split count, never on timing.
__global__ void __launch_bounds__(256) conv_fold_partials(const float* __restrict__ part, float* __restrict__ out, ConvP p) {
  __shared__ float sm[8][33];
  const int lane = threadIdx.x & 31, grp = threadIdx.x >> 5;
  const long long total = (long long)p.M * p.N;
  const long long i = (long long)blockIdx.x * 32 + lane;
  float s = 0.f;
  if (i < total) {
#pragma unroll 4
    for (int z = grp; z < p.splitK; z += 8) s += part[(long long)z * total + i];
  }
  sm[grp][lane] = s;
  __syncthreads();
  if (grp != 0 || i >= total) return;
#pragma unroll
  for (int g = 1; g < 8; ++g) s += sm[g][lane];
  int m = (int)(i / p.N), n = (int)(i - (long long)m * p.N);
  int b, o0, o1;
  if (p.bFast) { b = m % p.Nb; int t = m / p.Nb; o1 = t % p.o1n; o0 = t / p.o1n; }
  else { o1 = m % p.o1n; int t = m / p.o1n; o0 = t % p.o0n; b = t / p.o0n; }
  out[(long long)b * p.outB + (long long)o0 * p.outS0 + (long long)o1 * p.outS1 + (long long)n * p.outF] = s;
}

// Few splits: one lane per four consecutive outputs (16-byte reads of every partial), splits added in order.
__global__ void __launch_bounds__(256) conv_fold_few(const float* __restrict__ part, float* __restrict__ out, ConvP p) {
  const long long total = (long long)p.M * p.N;   // p.N % 4 == 0 (checked by the launcher)
  const long long i = ((long long)blockIdx.x * 256 + threadIdx.x) * 4;
  if (i >= total) return;
  float4 s = *(const float4*)(part + i);
  for (int z = 1; z < p.splitK; ++z) {
    float4 v = *(const float4*)(part + (long long)z * total + i);
    s.x += v.x; s.y += v.y; s.z += v.z; s.w += v.w;
  }
  const int m = (int)(i / p.N), n = (int)(i - (long long)m * p.N);
  int b, o0, o1;
  if (p.bFast) { b = m % p.Nb; int t = m / p.Nb; o1 = t % p.o1n; o0 = t / p.o1n; }
  else { o1 = m % p.o1n; int t = m / p.o1n; o0 = t % p.o0n; b = t / p.o0n; }
  float* o = out + (long long)b * p.outB + (long long)o0 * p.outS0 + (long long)o1 * p.outS1 + (long long)n * p.outF;
  if (p.outF == 1 && (((uintptr_t)o) & 15) == 0) *(float4*)o = s;
  else { o[0] = s.x; o[p.outF] = s.y; o[2 * (long long)p.outF] = s.z; o[3 * (long long)p.outF] = s.w; }
}

// Filter laid out with the contracted feature contiguous (data gradients): rewritten once per call
// as [tap][contracted feature][output feature] so that the B tile loads are 16-byte rows along n.
__global__ void __launch_bounds__(256) conv_repack_filter(const float* __restrict__ src, float* __restrict__ dst, ConvP p, int taps) {
  __shared__ float tile[32][33];
  const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;   // 32 x 8
  const int tap = blockIdx.z;
  const int t0 = tap / p.k1n, t1 = tap % p.k1n;
  const float* s = src + (long long)t0 * p.rhsS0 + (long long)t1 * p.rhsS1;
  float* d = dst + (long long)tap * p.C * p.N;
  const int c0 = blockIdx.x * 32, n0 = blockIdx.y * 32;
  (void)taps;
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int n = n0 + ty + 8 * r, c = c0 + tx;   // source: c contiguous (rhsI == 1)
    tile[ty + 8 * r][tx] = (n < p.N && c < p.C) ? s[(long long)c * p.rhsI + (long long)n * p.rhsO] : 0.f;
  }
  __syncthreads();
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int c = c0 + ty + 8 * r, n = n0 + tx;
    if (c < p.C && n < p.N) d[(long long)c * p.N + n] = tile[tx][ty + 8 * r];
  }
}

struct ConvChoice {
  bool fast = false;
  int amode = 0, bmode = 0, bm = 128, bn = 128, splitK = 1, tilesPerSplit = 0, kTiles = 0, cTiles = 0, bFast = 0;
  bool kflat = false;
};

bool fitsInt(const mi355_conv_desc* d) {
  long long lhs = d->N * d->batchGroups * d->C, rhs = d->C * d->O, out = d->N * d->O;
  for (int k = 0; k < d->nsp; ++k) { lhs *= d->in[k]; rhs *= d->k[k]; out *= d->out[k]; }
  return lhs < (1ll << 29) && rhs < (1ll << 29) && out < (1ll << 31);   // inputs below 2 GiB: buffer descriptors and byte offsets are 32-bit
}

ConvChoice choose(const mi355_conv_desc* d, long long tapsVisited = -1, int sharedLaunch = 1) {
  ConvChoice c;
  if (d->dtype != 0 || d->nsp > 2 || d->featureGroups != 1 || d->batchGroups != 1 || !fitsInt(d)) return c;
  c.fast = true;
  long long M = d->N, K = d->C;
  for (int k = 0; k < d->nsp; ++k) { M *= d->out[k]; K *= d->k[k]; }
  long long N = d->O;
  bool chunk = d->C % BK == 0;
  auto mult4 = [](long long x) { return x % 4 == 0; };
  long long s0 = d->nsp > 0 ? d->lhsS[0] : 0, s1 = d->nsp > 1 ? d->lhsS[1] : 0;
  long long r0 = d->nsp > 0 ? d->rhsS[0] : 0, r1 = d->nsp > 1 ? d->rhsS[1] : 0;
  if (chunk && d->lhsF == 1 && mult4(d->lhsB) && mult4(s0) && mult4(s1)) c.amode = 1;
  else if (chunk && d->lhsB == 1 && d->N % 4 == 0 && mult4(d->lhsF) && mult4(s0) && mult4(s1)) { c.amode = 2; c.bFast = 1; }
  if (chunk && d->rhsO == 1 && N % 4 == 0 && mult4(d->rhsI) && mult4(r0) && mult4(r1)) c.bmode = 1;
  else if (chunk && d->rhsI == 1 && mult4(d->rhsO) && mult4(r0) && mult4(r1)) c.bmode = 2;
  c.kflat = !chunk;
  long long taps = 1;
  for (int k = 0; k < d->nsp; ++k) taps *= d->k[k];
  if (tapsVisited >= 0 && chunk) taps = tapsVisited;
  c.cTiles = chunk ? (int)(d->C / BK) : 1;
  c.kTiles = chunk ? (int)(taps * c.cTiles) : (int)((K + BK - 1) / BK);
  // largest tile that still leaves minTiles output tiles (split-K then multiplies the workgroups); tuned on the ResNet18 step
  auto tilesOf = [&](int bm, int bn) { return ((M + bm - 1) / bm) * ((N + bn - 1) / bn); };
  static const int forced = getenv("MI355X_CONV_TILE") ? atoi(getenv("MI355X_CONV_TILE")) : 0;
  // (measured on the ResNet18 step: forward and data-gradient shapes prefer 64x64 tiles with little or no split of K over
  // wider tiles split further, whose partial sums cost a fold pass; the filter gradients, with their long K, prefer wide tiles)
  static const int minTilesEnv = getenv("MI355X_CONV_MIN_TILES") ? atoi(getenv("MI355X_CONV_MIN_TILES")) : 0;
  static const int minTilesLongK = getenv("MI355X_CONV_MIN_TILES_LONGK") ? atoi(getenv("MI355X_CONV_MIN_TILES_LONGK")) : 128;
  const int minTiles = minTilesEnv ? minTilesEnv : (c.amode == 2 ? minTilesLongK : 1024);
  if (forced == 128 || (!forced && N >= 128 && tilesOf(128, 128) >= minTiles)) { c.bm = 128; c.bn = 128; }
  else if (forced == 12864 || (!forced && tilesOf(128, 64) >= minTiles)) { c.bm = 128; c.bn = 64; }
  else { c.bm = 64; c.bn = 64; }
  // At most 256 tiles of 128x128 would be split four ways or more to fill the chip; 128x64 tiles need half the split,
  // which halves the partial sums written and folded (measured: 0.7 % of a ResNet step; 64x64 tiles with no split lose).
  // The long-K filter gradients keep the wide tile: their output is small and their K loop is all that matters.
  if (!forced && c.bm == 128 && c.bn == 128 && tilesOf(128, 128) <= 256 && c.kTiles < 2048) c.bn = 64;
  long long tiles = ((M + c.bm - 1) / c.bm) * ((N + c.bn - 1) / c.bn) * sharedLaunch;   // problems launched together fill the device together
  // Split K until there are about `target` workgroups: four per CU, which is what stays resident, so that a
  // tile count that is not a multiple of the CU count costs little, without exceeding it (a fifth
  // workgroup per CU waits for a whole workgroup time: 1280 measured a tenth slower than 1024).
  static const int target = getenv("MI355X_CONV_BLOCKS") ? atoi(getenv("MI355X_CONV_BLOCKS")) : 1024;
  int split = 1;
  static const int minSplitTiles = getenv("MI355X_CONV_MIN_SPLIT_KTILES") ? atoi(getenv("MI355X_CONV_MIN_SPLIT_KTILES")) : 1;
  // (measured: splitting pays even for a short K, the shorter dependent chain per workgroup outweighs the fold launch)
  static const int splitFactor = getenv("MI355X_CONV_SPLIT_FACTOR") ? atoi(getenv("MI355X_CONV_SPLIT_FACTOR")) : 3;
  if (tiles * (c.amode == 2 ? 2 : splitFactor) <= target && c.kTiles >= minSplitTiles) split = (int)std::min<long long>(target / tiles, std::max(1, c.kTiles / (tiles < 64 ? 4 : 8)));
  split = std::max(1, std::min(split, 256));
  static const bool xcdSplit = getenv("MI355X_CONV_XCD_SPLIT") && getenv("MI355X_CONV_XCD_SPLIT")[0] == '1';
  if (xcdSplit && split >= 16) split = split / 8 * 8;   // whole groups of K ranges per XCD, so that no XCD runs a workgroup more than the others
  c.tilesPerSplit = (c.kTiles + split - 1) / split;
  c.splitK = (c.kTiles + c.tilesPerSplit - 1) / c.tilesPerSplit;
  return c;
}

template <int BM, int BN>
void launchIgemm(const ConvChoice& c, const ConvP& p, dim3 grid, hipStream_t st) {
#define CASE(A, B, F) conv_igemm_f32<BM, BN, A, B, F><<<grid, 256, 0, st>>>(p)
#define LEAN(A, B) do { if (table) conv_igemm_lean<BM, BN, A, B, true><<<grid, 256, table, st>>>(p); else conv_igemm_lean<BM, BN, A, B, false><<<grid, 256, 0, st>>>(p); } while (0)
  if (c.kflat) { CASE(0, 0, true); return; }
  const size_t tableBytes = (size_t)p.taps * BM * sizeof(unsigned);
  const unsigned table = tableBytes <= (size_t)kTapTableBytes ? (unsigned)tableBytes : 0u;
  switch (c.amode * 3 + c.bmode) {
    case 0: CASE(0, 0, false); break;
    case 1: CASE(0, 1, false); break;
    case 2: CASE(0, 2, false); break;
    case 3: CASE(1, 0, false); break;
    case 4: LEAN(1, 1); break;
    case 5: LEAN(1, 2); break;
    case 6: CASE(2, 0, false); break;
    case 7: LEAN(2, 1); break;
    case 8: LEAN(2, 2); break;
  }
#undef LEAN
#undef CASE
}

template <int BM, int BN>
void launchPack(const ConvChoice& c, const ConvPack& ps, int count, hipStream_t st) {
  int maxM = 0, maxTaps = 0;
  for (int i = 0; i < count; ++i) { maxM = std::max(maxM, ps.c[i].M); maxTaps = std::max(maxTaps, ps.c[i].taps); }
  dim3 grid((unsigned)((maxM + BM - 1) / BM), (unsigned)((ps.c[0].N + BN - 1) / BN), (unsigned)count);
  const size_t tableBytes = (size_t)maxTaps * BM * sizeof(unsigned);
  const unsigned table = tableBytes <= (size_t)kTapTableBytes ? (unsigned)tableBytes : 0u;
#define PACK(A, B) do { if (table) conv_igemm_lean_pack<BM, BN, A, B, true><<<grid, 256, table, st>>>(ps); else conv_igemm_lean_pack<BM, BN, A, B, false><<<grid, 256, 0, st>>>(ps); } while (0)
  switch (c.amode * 3 + c.bmode) {
    case 4: PACK(1, 1); break;
    case 5: PACK(1, 2); break;
    case 7: PACK(2, 1); break;
    case 8: PACK(2, 2); break;
  }
#undef PACK
}

// One launch of the implicit-GEMM kernel: the whole convolution, or one residue class of an
// input-dilated one.  With lhs dilation L (the data gradient of a stride-L convolution) an
// output position o only meets real input where (o - pad + tap) is a multiple of L, so the
// outputs with o = c (mod L) all use the same subset of the taps (tap = (pad - c) mod L,
// step L).  Run per class, no product with an inserted zero is ever formed: a 3x3 filter
// with L = 2 does 9 tap-products per 4 outputs instead of 36.
struct ConvPart {
  mi355_conv_desc d;
  int kb[2] = {0, 0}, ks[2] = {1, 1}, kc[2] = {1, 1};
  long long outOffset = 0;
  long long taps() const { return (long long)kc[0] * kc[1]; }
};

std::vector<ConvPart> partsOf(const mi355_conv_desc* d) {
  std::vector<ConvPart> parts;
  ConvPart whole;
  whole.d = *d;
  for (int k = 0; k < 2; ++k) whole.kc[k] = k < d->nsp ? (int)d->k[k] : 1;
  bool dilated = false, eligible = d->nsp == 2 && d->C % BK == 0 && d->dtype == 0 && d->featureGroups == 1 && d->batchGroups == 1;
  for (int k = 0; k < d->nsp && k < 2; ++k) {
    if (d->ldil[k] > 1) dilated = true;
    if (d->stride[k] != 1 || d->rdil[k] != 1 || d->k[k] < d->ldil[k] || d->out[k] < d->ldil[k]) eligible = false;
  }
  static const bool off = getenv("MI355X_CONV_CLASSES") && getenv("MI355X_CONV_CLASSES")[0] == '0';
  if (!dilated || !eligible || off) { parts.push_back(whole); return parts; }
  const int L0 = (int)d->ldil[0], L1 = (int)d->ldil[1];
  for (int c0 = 0; c0 < L0; ++c0) {
    for (int c1 = 0; c1 < L1; ++c1) {
      ConvPart p = whole;
      const int cls[2] = {c0, c1};
      for (int k = 0; k < 2; ++k) {
        const int L = (int)d->ldil[k];
        p.d.out[k] = (d->out[k] - cls[k] + L - 1) / L;          // outputs o = cls + L * j
        p.d.stride[k] = L;                                      // input coordinate of j: j * L + cls - pad
        p.d.padLo[k] = d->padLo[k] - cls[k];
        p.d.outS[k] = d->outS[k] * L;
        p.outOffset += (long long)cls[k] * d->outS[k];
        p.kb[k] = (int)((((d->padLo[k] - cls[k]) % L) + L) % L);
        p.ks[k] = L;
        p.kc[k] = (int)((d->k[k] - p.kb[k] + L - 1) / L);
      }
      parts.push_back(p);
    }
  }
  return parts;
}

// A filter whose contracted feature is the contiguous one (the layout data gradients see) is
// worth rewriting when the GEMM has many rows: returns the bytes of the rewritten copy and
// the descriptor that addresses it, or 0.
size_t repackedFilter(const mi355_conv_desc* d, mi355_conv_desc* out) {
  if (d->dtype != 0 || d->nsp > 2 || d->featureGroups != 1 || d->batchGroups != 1 || !fitsInt(d)) return 0;
  // (measured: with the row-major B tile of the vector-loader kernel the rewritten copy no longer pays; kept as an option)
  static const bool on = getenv("MI355X_CONV_REPACK") && getenv("MI355X_CONV_REPACK")[0] == '1';
  if (!on) return 0;
  if (d->rhsI != 1 || d->rhsO == 1 || d->C % BK != 0 || d->O % 4 != 0) return 0;
  long long M = d->N, taps = 1;
  for (int k = 0; k < d->nsp; ++k) { M *= d->out[k]; taps *= d->k[k]; }
  if (M < 2048) return 0;
  *out = *d;
  out->rhsO = 1;
  out->rhsI = d->O;
  if (d->nsp > 1) out->rhsS[1] = d->C * d->O;
  if (d->nsp > 0) out->rhsS[0] = (d->nsp > 1 ? d->k[1] : 1) * d->C * d->O;
  size_t bytes = (size_t)taps * (size_t)d->C * (size_t)d->O * sizeof(float);
  return (bytes + 255) / 256 * 256;
}

}  // namespace

extern "C" {

size_t mi355_conv_workspace_bytes(const mi355_conv_desc* d) {
  mi355_conv_desc d2;
  size_t repack = repackedFilter(d, &d2);
  if (repack) d = &d2;
  size_t most = 0;
  for (const ConvPart& part : partsOf(d)) {
    ConvChoice c = choose(&part.d, part.taps());
    if (!c.fast || c.splitK <= 1) continue;
    long long M = part.d.N;
    for (int k = 0; k < part.d.nsp; ++k) M *= part.d.out[k];
    most = std::max(most, (size_t)c.splitK * (size_t)M * (size_t)d->O * sizeof(float));
  }
  return repack + most;
}

int mi355_conv_direct(const mi355_conv_desc* d, const void* lhs, const void* rhs, void* out, mi355_stream_t s);

// Launches one part; with `prepared` set it only fills the kernel parameters of an unsplit part (returns -1 when the part cannot be prepared that way).
static int launchPart(const ConvPart& part, const void* lhs, const void* rhs, void* out, void* workspace, size_t workspace_bytes, hipStream_t st,
                      int sharedLaunch = 1, ConvChoice* preparedChoice = nullptr, ConvP* prepared = nullptr, float* statSum = nullptr, float* statSq = nullptr) {
  const mi355_conv_desc* d = &part.d;
  ConvChoice c = choose(d, part.taps(), sharedLaunch);
  ConvP p;
  p.lhs = (const float*)lhs;
  p.rhs = (const float*)rhs;
  p.statSum = statSum;
  p.statSq = statSq;
  p.tilesM = 0;
  p.tilesXY = 0;
  long long M = d->N, K = d->C;
  for (int k = 0; k < d->nsp; ++k) { M *= d->out[k]; K *= d->k[k]; }
  if (M <= 0 || d->O <= 0) return prepared ? -1 : 0;
  p.M = (int)M; p.N = (int)d->O; p.K = (int)K;
  p.Nb = (int)d->N; p.C = (int)d->C;
  auto dim = [&](const int64_t* a, int k, int64_t dflt) { return k < d->nsp ? (int)a[k] : (int)dflt; };
  p.in0 = dim(d->in, 0, 1); p.in1 = dim(d->in, 1, 1);
  p.k0n = dim(d->k, 0, 1); p.k1n = dim(d->k, 1, 1);
  p.kb0 = part.kb[0]; p.ks0 = part.ks[0]; p.kc0 = part.kc[0];
  p.kb1 = part.kb[1]; p.ks1 = part.ks[1]; p.kc1 = part.kc[1];
  p.o0n = dim(d->out, 0, 1); p.o1n = dim(d->out, 1, 1);
  p.s0 = dim(d->stride, 0, 1); p.s1 = dim(d->stride, 1, 1);
  p.p0 = dim(d->padLo, 0, 0); p.p1 = dim(d->padLo, 1, 0);
  p.ld0 = dim(d->ldil, 0, 1); p.ld1 = dim(d->ldil, 1, 1);
  p.rd0 = dim(d->rdil, 0, 1); p.rd1 = dim(d->rdil, 1, 1);
  p.rev0 = dim(d->rev, 0, 0); p.rev1 = dim(d->rev, 1, 0);
  p.lhsB = (int)d->lhsB; p.lhsF = (int)d->lhsF; p.lhsS0 = dim(d->lhsS, 0, 0); p.lhsS1 = dim(d->lhsS, 1, 0);
  p.rhsI = (int)d->rhsI; p.rhsO = (int)d->rhsO; p.rhsS0 = dim(d->rhsS, 0, 0); p.rhsS1 = dim(d->rhsS, 1, 0);
  p.outB = (int)d->outB; p.outF = (int)d->outF; p.outS0 = dim(d->outS, 0, 0); p.outS1 = dim(d->outS, 1, 0);
  p.bFast = c.bFast;
  {
    // Is the offset of output row m linear in m?  It is a mixed-radix function of m, so agreement at the carries decides.
    auto rowOff = [&](long long m) {
      long long b, o0, o1;
      if (p.bFast) { b = m % p.Nb; long long t = m / p.Nb; o1 = t % p.o1n; o0 = t / p.o1n; }
      else { o1 = m % p.o1n; long long t = m / p.o1n; o0 = t % p.o0n; b = t / p.o0n; }
      return b * (long long)p.outB + o0 * (long long)p.outS0 + o1 * (long long)p.outS1;
    };
    const long long unit = M > 1 ? rowOff(1) : 1;
    const long long inner = p.bFast ? p.Nb : p.o1n, mid = inner * (p.bFast ? p.o1n : p.o0n);
    bool linear = unit > 0;
    for (long long m : {inner - 1, inner, mid - 1, mid, mid + inner, M - 1})
      if (m > 0 && m < M && rowOff(m) != m * unit) linear = false;
    p.outRow = linear ? unit : 0;
  }
  p.cTiles = c.cTiles; p.kTiles = c.kTiles; p.splitK = c.splitK; p.tilesPerSplit = c.tilesPerSplit;
  p.taps = part.kc[0] * part.kc[1];
  {
    long long lhsN = d->N * d->batchGroups * d->C, rhsN = d->C * d->O;
    for (int k = 0; k < d->nsp; ++k) { lhsN *= d->in[k]; rhsN *= d->k[k]; }
    p.lhsBytes = (unsigned)(lhsN * 4); p.rhsBytes = (unsigned)(rhsN * 4);   // below 2 GiB each (fitsInt)
  }
  float* dst = (float*)out + part.outOffset;
  if (c.splitK > 1) {
    size_t need = (size_t)c.splitK * (size_t)M * (size_t)d->O * sizeof(float);
    if (!workspace || workspace_bytes < need) return 3;   // caller sized the workspace wrong
    p.out = (float*)workspace;
    p.outVec = (p.N & 3) == 0 && ((uintptr_t)workspace & 15) == 0;
  } else {
    p.out = dst;
    auto mult4 = [](long long x) { return (x & 3) == 0; };
    p.outVec = p.outF == 1 && mult4(p.N) && mult4(p.outB) && mult4(p.outS0) && mult4(p.outS1) && ((uintptr_t)dst & 15) == 0;
  }
  if (prepared) {
    if (c.splitK > 1 || c.kflat || c.amode == 0 || c.bmode == 0) return -1;
    *prepared = p;
    *preparedChoice = c;
    return 0;
  }
  dim3 grid((unsigned)((p.M + c.bm - 1) / c.bm), (unsigned)((p.N + c.bn - 1) / c.bn), (unsigned)c.splitK);
  if (grid.y > 65535) return 4;
  static const bool xcdSplitOn = getenv("MI355X_CONV_XCD_SPLIT") && getenv("MI355X_CONV_XCD_SPLIT")[0] == '1';
  if (c.splitK >= 16 && !c.kflat && c.amode != 0 && c.bmode != 0 && xcdSplitOn) {   // (with fewer K ranges than a few per XCD the XCDs would not be loaded evenly)
    p.tilesM = (int)grid.x;
    p.tilesXY = (int)(grid.x * grid.y);
    grid = dim3((unsigned)(8 * p.tilesXY * ((c.splitK + 7) / 8)), 1, 1);
  }
  if (c.bm == 128 && c.bn == 128) launchIgemm<128, 128>(c, p, grid, st);
  else if (c.bm == 128) launchIgemm<128, 64>(c, p, grid, st);
  else launchIgemm<64, 64>(c, p, grid, st);
  if (c.splitK > 1) {
    long long total = M * d->O;
    if (c.splitK <= 8 && p.N % 4 == 0 && ((uintptr_t)workspace & 15) == 0)
      conv_fold_few<<<(unsigned)((total / 4 + 255) / 256), 256, 0, st>>>((const float*)workspace, dst, p);
    else
      conv_fold_partials<<<(unsigned)((total + 31) / 32), 256, 0, st>>>((const float*)workspace, dst, p);
  }
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? 0 : (int)e;
}

// Rows of per-tile column sums the convolution can deliver next to its output (one per tile row of the implicit GEMM),
// or 0 when it cannot: the vector-loader kernel, unsplit, one launch, output rows dense and in GEMM row order.
int mi355_conv_stats_rows(const mi355_conv_desc* d) {
  static const bool off = getenv("MI355X_CONV_STATS") && getenv("MI355X_CONV_STATS")[0] == '0';
  mi355_conv_desc d2;
  if (off || repackedFilter(d, &d2)) return 0;
  ConvChoice c = choose(d);
  if (!c.fast || c.kflat || c.amode == 0 || c.bmode == 0 || c.splitK != 1 || c.bFast) return 0;
  if (partsOf(d).size() != 1) return 0;
  long long M = d->N;
  for (int k = 0; k < d->nsp; ++k) M *= d->out[k];
  if (M <= 0 || d->outF != 1) return 0;
  // dense output in GEMM row order: row (b, o0, o1) starts at ((b * out0 + o0) * out1 + o1) * O
  long long expect = d->O;
  for (int k = d->nsp - 1; k >= 0; --k) { if (d->outS[k] != expect) return 0; expect *= d->out[k]; }
  if (d->outB != expect) return 0;
  return (int)((M + c.bm - 1) / c.bm);
}

int mi355_conv_stats(const mi355_conv_desc* d, const void* lhs, const void* rhs, void* out, void* workspace, size_t workspace_bytes,
                     float* stat_sum, float* stat_sq, mi355_stream_t s);

int mi355_conv(const mi355_conv_desc* d, const void* lhs, const void* rhs, void* out, void* workspace, size_t workspace_bytes,
               mi355_stream_t s) {
  return mi355_conv_stats(d, lhs, rhs, out, workspace, workspace_bytes, nullptr, nullptr, s);
}

int mi355_conv_stats(const mi355_conv_desc* d, const void* lhs, const void* rhs, void* out, void* workspace, size_t workspace_bytes,
                     float* stat_sum, float* stat_sq, mi355_stream_t s) {
  hipStream_t st = (hipStream_t)s;
  if (stat_sum && mi355_conv_stats_rows(d) == 0) return 5;   // the planner asked for statistics this convolution cannot deliver
  mi355_conv_desc d2;
  size_t repack = repackedFilter(d, &d2);
  if (repack) {
    if (!workspace || workspace_bytes < repack) return 3;   // caller sized the workspace wrong
    ConvP q;
    q.C = (int)d->C; q.N = (int)d->O;
    q.k1n = d->nsp > 1 ? (int)d->k[1] : 1;
    q.rhsI = (int)d->rhsI; q.rhsO = (int)d->rhsO;
    q.rhsS0 = d->nsp > 0 ? (int)d->rhsS[0] : 0; q.rhsS1 = d->nsp > 1 ? (int)d->rhsS[1] : 0;
    int taps = 1;
    for (int k = 0; k < d->nsp; ++k) taps *= (int)d->k[k];
    dim3 grid((unsigned)((d->C + 31) / 32), (unsigned)((d->O + 31) / 32), (unsigned)taps);
    conv_repack_filter<<<grid, 256, 0, st>>>((const float*)rhs, (float*)workspace, q, taps);
    rhs = workspace;
    workspace = (char*)workspace + repack;
    workspace_bytes -= repack;
    d = &d2;
  }
  if (!choose(d).fast) return mi355_conv_direct(d, lhs, rhs, out, s);
  const std::vector<ConvPart> parts = partsOf(d);
  static const bool packOff = getenv("MI355X_CONV_PACK") && getenv("MI355X_CONV_PACK")[0] == '0';
  if (parts.size() > 1 && parts.size() <= (size_t)kMaxPack && !packOff) {
    // residue classes that need no split of K when counted together share one launch
    ConvPack ps;
    ConvChoice cs[kMaxPack];
    bool ok = true;
    for (size_t i = 0; i < parts.size() && ok; ++i) {
      ok = launchPart(parts[i], lhs, rhs, out, workspace, workspace_bytes, st, (int)parts.size(), &cs[i], &ps.c[i]) == 0;
      if (ok && i > 0) ok = cs[i].amode == cs[0].amode && cs[i].bmode == cs[0].bmode && cs[i].bm == cs[0].bm && cs[i].bn == cs[0].bn && ps.c[i].N == ps.c[0].N;
    }
    if (ok) {
      if (cs[0].bm == 128 && cs[0].bn == 128) launchPack<128, 128>(cs[0], ps, (int)parts.size(), st);
      else if (cs[0].bm == 128) launchPack<128, 64>(cs[0], ps, (int)parts.size(), st);
      else launchPack<64, 64>(cs[0], ps, (int)parts.size(), st);
      hipError_t e = hipGetLastError();
      return e == hipSuccess ? 0 : (int)e;
    }
  }
  for (const ConvPart& part : parts) {
    // parts run back to back on the stream, so they can share the split-K scratch
    if (int r = launchPart(part, lhs, rhs, out, workspace, workspace_bytes, st, 1, nullptr, nullptr, stat_sum, stat_sq)) return r;
  }
  return 0;
}

}  // extern "C"
