// Ahead-of-time HIP kernels for gfx950 (CDNA4): strided batched GEMM on MFMA
// (fp32 and bf16 inputs, fp32 accumulation), direct convolution for arbitrary
// StableHLO dimension numbers, deterministic row scatter (stable radix sort +
// in-order segment fold) and a vector copy.
//
// Reference call sites these replace: dot_general -> mlx einsum/matmul
// (src/pjrt_plugin/ops/linalg.cc:89-250), convolution -> mlx conv_general
// (linalg.cc:253-550), scatter -> mlx scatter_add with float atomics
// (ops/gather_scatter.cc:55-77; order-dependent there, ordered here).
#include <hip/hip_runtime.h>

#include <cstdint>

#include "hip_abi.h"

typedef unsigned short u16;
typedef unsigned int u32;
typedef float float16v __attribute__((ext_vector_type(16)));
typedef float float4v __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

__device__ __forceinline__ float bf2f(u16 b) { return __uint_as_float(((u32)b) << 16); }
__device__ __forceinline__ u16 f2bf(float f) {
  u32 u = __float_as_uint(f);
  if ((u & 0x7FFFFFFFu) > 0x7F800000u) return (u16)((u >> 16) | 0x40);
  u += 0x7FFFu + ((u >> 16) & 1u);
  return (u16)(u >> 16);
}

// ------------------------------------------------------------------- copy
__global__ void __launch_bounds__(256) copy_vec16(const uint4* __restrict__ src, uint4* __restrict__ dst, size_t n16) {
  size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i < n16) dst[i] = src[i];
}
__global__ void __launch_bounds__(256) copy_bytes(const unsigned char* __restrict__ src, unsigned char* __restrict__ dst, size_t n) {
  size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i < n) dst[i] = src[i];
}

struct MultiCopyArgs {
  const unsigned char* src[16];
  unsigned char* dst[16];
  unsigned long long bytes[16];
  // optional condition, read on the device: mode 1 copies when *flag != 0 (a loop still running); mode 2 copies when the
  // branch index at `flag` (indexBytes wide; 0 = one-byte predicate), clamped to the last branch when out of range, is `want`
  const void* flag;
  int mode, indexBytes;
  long long want, count;
};
__device__ __forceinline__ bool copyEnabled(const MultiCopyArgs& a) {
  if (a.mode == 0) return true;
  if (a.mode == 1) return *(const int*)a.flag != 0;
  long long idx;
  switch (a.indexBytes) {
    case 0: idx = *(const unsigned char*)a.flag ? 1 : 0; break;
    case 1: idx = *(const signed char*)a.flag; break;
    case 2: idx = *(const short*)a.flag; break;
    case 4: idx = *(const int*)a.flag; break;
    default: idx = *(const long long*)a.flag; break;
  }
  if (idx < 0 || idx >= a.count) idx = a.count - 1;
  return idx == a.want;
}
// flag[0] = parent ? *parent : 1, flag[1] = 0  (pred == null), or  flag[0] = flag[0] && *pred, flag[1] += flag[0]
// (flag[1] counts the iterations that ran while the loop was alive)
__global__ void flag_update(int* flag, const int* parent, const unsigned char* pred) {
  if (threadIdx.x != 0 || blockIdx.x != 0) return;
  if (pred) {
    const int alive = (flag[0] != 0 && *pred != 0) ? 1 : 0;
    flag[0] = alive;
    flag[1] += alive;
  } else {
    flag[0] = parent ? (*parent != 0 ? 1 : 0) : 1;
    flag[1] = 0;
  }
}
__global__ void __launch_bounds__(256) copy_multi(MultiCopyArgs a) {
  if (!copyEnabled(a)) return;
  const int j = blockIdx.y;
  const unsigned char* src = a.src[j];
  unsigned char* dst = a.dst[j];
  const size_t bytes = a.bytes[j];
  const size_t stride = (size_t)gridDim.x * 256;
  if ((((uintptr_t)src | (uintptr_t)dst | bytes) & 15) == 0) {
    const size_t n16 = bytes / 16;
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n16; i += stride) ((uint4*)dst)[i] = ((const uint4*)src)[i];
  } else {
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < bytes; i += stride) dst[i] = src[i];
  }
}

// ------------------------------------------------------------------- GEMM
// Workgroup tile 64x64, four wavefronts in a 2x2 arrangement, each owning a 32x32
// accumulator held by one MFMA 32x32 instruction.  A and B tiles are staged in LDS
// k-major (fp32) or k-minor in groups of 8 (bf16) so that every MFMA operand read is a
// conflict-free row.  Operands are addressed through element strides, so transposed and
// batched layouts of dot_general need no copies.
struct GemmArgs {
  const void* a;
  const void* b;
  void* c;
  long long M, N, K;
  long long aB0, aB1, aRow, aCol, bB0, bB1, bRow, bCol;
  int batch1;
  int outBf16;
  const void* bias;   // N values of the output type, or null
};

// c[r][n] += bias[n], then the activation, for kernels without an epilogue of their own (c is already rounded to its type)
struct ActArgs { int act; float a, b, c; };
__device__ __forceinline__ float geluTanh(float x, const ActArgs& k) {
  const float u = k.c * (x + k.b * (x * x * x));
  const float e = __expf(2.f * fminf(u, 20.f));          // 1 + tanh(u) = 2 e^(2u) / (1 + e^(2u)): no cancellation for negative u
  return k.a * x * (2.f * e * __builtin_amdgcn_rcpf(1.f + e));
}
template <typename T>
__global__ void __launch_bounds__(256) gemm_add_bias(T* c, const T* bias, long long total, long long N, ActArgs act) {
  const long long i = (long long)blockIdx.x * 256 + threadIdx.x;
  if (i >= total) return;
  if constexpr (sizeof(T) == 2) {
    u16 r = c[i];
    if (bias) r = f2bf(bf2f(r) + bf2f(bias[i % N]));
    if (act.act == 1) r = f2bf(geluTanh(bf2f(r), act));
    c[i] = r;
  } else {
    if (bias) c[i] = c[i] + bias[i % N];
  }
}

__global__ void __launch_bounds__(256) gemm_f32_mfma(GemmArgs g) {
  constexpr int BM = 64, BN = 64, BK = 16;
  __shared__ float As[BK][BM + 4];
  __shared__ float Bs[BK][BN + 4];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const long long b0 = blockIdx.z / g.batch1, b1 = blockIdx.z % g.batch1;
  const float* A = (const float*)g.a + b0 * g.aB0 + b1 * g.aB1;
  const float* B = (const float*)g.b + b0 * g.bB0 + b1 * g.bB1;
  const long long m0 = (long long)blockIdx.y * BM, n0 = (long long)blockIdx.x * BN;
  float16v acc = {0};
  const bool aKfast = g.aCol == 1 || g.aRow != 1;   // walk k fastest when k is the contiguous axis
  const bool bNfast = g.bCol == 1 || g.bRow != 1;
  for (long long k0 = 0; k0 < g.K; k0 += BK) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      int e = tid + 256 * i;
      int m, k;
      if (aKfast) { m = e / BK; k = e % BK; } else { k = e / BM; m = e % BM; }
      long long gm = m0 + m, gk = k0 + k;
      As[k][m] = (gm < g.M && gk < g.K) ? A[gm * g.aRow + gk * g.aCol] : 0.f;
      int n, kb;
      if (bNfast) { kb = e / BN; n = e % BN; } else { n = e / BK; kb = e % BK; }
      long long gn = n0 + n, gkb = k0 + kb;
      Bs[kb][n] = (gn < g.N && gkb < g.K) ? B[gkb * g.bRow + gn * g.bCol] : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < BK; kk += 2) {
      float av = As[kk + (lane >> 5)][wm * 32 + (lane & 31)];
      float bv = Bs[kk + (lane >> 5)][wn * 32 + (lane & 31)];
      acc = __builtin_amdgcn_mfma_f32_32x32x2f32(av, bv, acc, 0, 0, 0);
    }
    __syncthreads();
  }
  const long long cBase = (long long)blockIdx.z * g.M * g.N;
  const long long col = n0 + wn * 32 + (lane & 31);
  if (col >= g.N) return;
#pragma unroll
  for (int j = 0; j < 16; ++j) {
    long long row = m0 + wm * 32 + (j >> 2) * 8 + (lane >> 5) * 4 + (j & 3);
    if (row < g.M) {
      if (g.outBf16) ((u16*)g.c)[cBase + row * g.N + col] = f2bf(acc[j]);
      else ((float*)g.c)[cBase + row * g.N + col] = acc[j];
    }
  }
}

// fp32 GEMMs with few output elements (recurrent cells, classifier heads, per-step projections):
// one workgroup per TxT output tile, the four waves split K between them and fold their partial
// tiles through LDS, so the whole product is one short launch with no split-K workspace.  Operands
// are read straight from memory in the MFMA operand layout (one element per lane per step).
// Up to two products of the same shape are summed into one result (x*Wi + h*Wh of a recurrent cell).
struct SmallPair {
  const float* a;
  const float* b;
  long long K, aB0, aB1, aRow, aCol, bB0, bB1, bRow, bCol;
  int aVec, bVec;   // k is the contiguous, 16-byte aligned axis of the operand: four k values per load
};
struct SmallArgs {
  SmallPair p[2];
  int pairs;
  float* c;
  const float* bias;   // N values or null
  const float* addend; // a tensor laid out like C that is added to the product (an accumulator carried by a loop), or null
  long long M, N;
  int batch1;
  int relu;            // the stored value is maximum(sum + bias, 0)
};

// The MFMA contraction does not care which k a lane's operand slot stands for as long as A and B agree, so a
// lane takes four consecutive k per "super-step" (one 16-byte load where k is contiguous, four strided loads
// otherwise) and feeds them to four products: lane kl of a row covers k = 4 * KS * s + 4 * kl + j in product j.
template <int T, bool AVEC, bool BVEC, typename ACC>
__device__ __forceinline__ void smallGemmPair(const SmallPair& pr, ACC& acc, long long b0, long long b1, long long rowA, long long rowB, int kl,
                                              int w) {
  constexpr int KS = T == 16 ? 4 : 2;         // k values per MFMA
  constexpr int KSS = 4 * KS;                 // k values per super-step
  // rowA / rowB are clamped to the operand's last row: a row of A only reaches its own row of the result and a
  // column of B its own column, and results outside M x N are never stored, so whatever the clamped lanes load
  // is harmless and every load of a whole super-step is unconditional (a predicated load is a branch around the
  // load: a batch of twenty of them took 1 700 cycles to issue).  Only the one ragged super-step at the end of
  // K selects zeros, for the k beyond K.
  const float* ap = pr.a + b0 * pr.aB0 + b1 * pr.aB1 + rowA * pr.aRow;
  const float* bp = pr.b + b0 * pr.bB0 + b1 * pr.bB1 + rowB * pr.bCol;
  const int K = (int)pr.K;
  const long long aCol = pr.aCol, bRow = pr.bRow;
  const int fullSteps = K / KSS, steps = (K + KSS - 1) / KSS, per = (steps + 3) / 4;
  const int s0 = w * per, s1 = s0 + per < steps ? s0 + per : steps;
  const int sFull = s1 < fullSteps ? s1 : fullSteps;
  auto fetch = [&](int kb, float (&xa)[4], float (&xb)[4]) {
    if constexpr (AVEC) {
      const float4 t = *(const float4*)(ap + kb);
      xa[0] = t.x; xa[1] = t.y; xa[2] = t.z; xa[3] = t.w;
    } else {
#pragma unroll
      for (int j = 0; j < 4; ++j) xa[j] = ap[(kb + j) * aCol];
    }
    if constexpr (BVEC) {
      const float4 t = *(const float4*)(bp + kb);
      xb[0] = t.x; xb[1] = t.y; xb[2] = t.z; xb[3] = t.w;
    } else {
#pragma unroll
      for (int j = 0; j < 4; ++j) xb[j] = bp[(kb + j) * bRow];
    }
  };
  auto fetchRagged = [&](int kb, float (&xa)[4], float (&xb)[4]) {   // never the vector layouts: those need K % 16 == 0
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const bool in = kb + j < K;
      const int k = in ? kb + j : K - 1;
      const float va = ap[k * aCol], vb = bp[k * bRow];
      xa[j] = in ? va : 0.f;
      xb[j] = in ? vb : 0.f;
    }
  };
  auto products = [&](const float (&av)[4], const float (&bv)[4]) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      if constexpr (T == 16) acc = __builtin_amdgcn_mfma_f32_16x16x4f32(av[j], bv[j], acc, 0, 0, 0);
      else acc = __builtin_amdgcn_mfma_f32_32x32x2f32(av[j], bv[j], acc, 0, 0, 0);
    }
  };
  // Batches of four super-steps in two register sets: the loads of one batch are in flight while the other is multiplied,
  // so a long K costs one round trip and then the products, not a round trip per batch (a K of 1024 on four wavefronts took
  // 8.2 us with batches of eight loaded and multiplied in turn, against 4.4 us for a K of 256).  The order of the products,
  // and with it every bit of the result, is that of the plain loop.
  int s = s0;
  const int batches = (sFull - s0) / 4;
  if (batches > 0) {
    float a0[4][4], b0[4][4], a1[4][4], b1[4][4];
    auto load4 = [&](int first, float (&av)[4][4], float (&bv)[4][4]) {
#pragma unroll
      for (int u = 0; u < 4; ++u) fetch((first + u) * KSS + 4 * kl, av[u], bv[u]);
    };
    auto products4 = [&](const float (&av)[4][4], const float (&bv)[4][4]) {
#pragma unroll
      for (int u = 0; u < 4; ++u) products(av[u], bv[u]);
    };
    load4(s0, a0, b0);
    if (batches > 1) load4(s0 + 4, a1, b1);
    for (int b = 0; b < batches; b += 2) {
      products4(a0, b0);
      if (b + 2 < batches) load4(s0 + 4 * (b + 2), a0, b0);
      if (b + 1 < batches) {
        products4(a1, b1);
        if (b + 3 < batches) load4(s0 + 4 * (b + 3), a1, b1);
      }
    }
    s = s0 + 4 * batches;
  }
  for (; s < sFull; ++s) {
    float av[4], bv[4];
    fetch(s * KSS + 4 * kl, av, bv);
    products(av, bv);
  }
  for (; s < s1; ++s) {
    float av[4], bv[4];
    fetchRagged(s * KSS + 4 * kl, av, bv);
    products(av, bv);
  }
}

template <int T>
__device__ __forceinline__ void smallGemmTileBody(const SmallArgs& g, unsigned bx, unsigned by, unsigned bz) {
  constexpr int NACC = T == 16 ? 4 : 16;
  typedef float accv __attribute__((ext_vector_type(NACC)));
  __shared__ float red[4][T * T];
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  const long long b0 = bz / g.batch1, b1 = bz % g.batch1;
  const long long m0 = (long long)by * T, n0 = (long long)bx * T;
  const int r = lane % T, kl = lane / T;
  const bool mOk = m0 + r < g.M, nOk = n0 + r < g.N;
  const long long rowA = mOk ? m0 + r : g.M - 1, rowB = nOk ? n0 + r : g.N - 1;
  accv acc = {0};
  for (int q = 0; q < g.pairs; ++q) {
    const SmallPair& pr = g.p[q];
    switch (pr.aVec * 2 + pr.bVec) {   // uniform; the loaders are compile-time so that their loads batch
      case 0: smallGemmPair<T, false, false>(pr, acc, b0, b1, rowA, rowB, kl, w); break;
      case 1: smallGemmPair<T, false, true>(pr, acc, b0, b1, rowA, rowB, kl, w); break;
      case 2: smallGemmPair<T, true, false>(pr, acc, b0, b1, rowA, rowB, kl, w); break;
      default: smallGemmPair<T, true, true>(pr, acc, b0, b1, rowA, rowB, kl, w); break;
    }
  }
#pragma unroll
  for (int i = 0; i < NACC; ++i) {
    const int row = T == 16 ? kl * 4 + i : (i >> 2) * 8 + kl * 4 + (i & 3);
    red[w][row * T + r] = acc[i];
  }
  __syncthreads();
  float* C = g.c + (long long)bz * g.M * g.N;
  const float* D = g.addend ? g.addend + (long long)bz * g.M * g.N : nullptr;
  for (int e = threadIdx.x; e < T * T; e += 256) {
    const long long row = m0 + e / T, col = n0 + e % T;
    if (row < g.M && col < g.N) {
      float sum = (red[0][e] + red[1][e]) + (red[2][e] + red[3][e]);
      if (D) sum += D[row * g.N + col];
      const float v = g.bias ? sum + g.bias[col] : sum;
      C[row * g.N + col] = g.relu ? ((v > 0.f || v != v) ? v : 0.f) : v;   // maximum(v, 0): NaN stays NaN, -0 becomes +0
    }
  }
}

template <int T>
__global__ void __launch_bounds__(256) gemm_f32_small(SmallArgs g) {
  smallGemmTileBody<T>(g, blockIdx.x, blockIdx.y, blockIdx.z);
}

// several independent small products in one launch: workgroup b belongs to the problem whose tile range holds b
constexpr int kMaxSmallGroup = 4;
struct SmallGroupArgs {
  SmallArgs prob[kMaxSmallGroup];
  unsigned first[kMaxSmallGroup + 1];   // first workgroup of each problem
  unsigned tilesN[kMaxSmallGroup], tilesM[kMaxSmallGroup];
  int n;
};

template <int T>
__global__ void __launch_bounds__(256) gemm_f32_small_group(SmallGroupArgs g) {
  const unsigned b = blockIdx.x;
  int p = 0;
  while (p + 1 < g.n && b >= g.first[p + 1]) ++p;
  const unsigned local = b - g.first[p];
  const unsigned tx = local % g.tilesN[p], rest = local / g.tilesN[p];
  smallGemmTileBody<T>(g.prob[p], tx, rest % g.tilesM[p], rest / g.tilesM[p]);
}

__global__ void __launch_bounds__(256) gemm_bf16_mfma(GemmArgs g) {
  constexpr int BM = 64, BN = 64, BK = 32;
  __shared__ __attribute__((aligned(16))) u16 As[BM][BK + 8];
  __shared__ __attribute__((aligned(16))) u16 Bs[BN][BK + 8];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const long long b0 = blockIdx.z / g.batch1, b1 = blockIdx.z % g.batch1;
  const u16* A = (const u16*)g.a + b0 * g.aB0 + b1 * g.aB1;
  const u16* B = (const u16*)g.b + b0 * g.bB0 + b1 * g.bB1;
  const long long m0 = (long long)blockIdx.y * BM, n0 = (long long)blockIdx.x * BN;
  float16v acc = {0};
  const bool aKfast = g.aCol == 1 || g.aRow != 1;
  const bool bNfast = g.bCol == 1 || g.bRow != 1;
  for (long long k0 = 0; k0 < g.K; k0 += BK) {
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      int e = tid + 256 * i;
      int m, k;
      if (aKfast) { m = e / BK; k = e % BK; } else { k = e / BM; m = e % BM; }
      long long gm = m0 + m, gk = k0 + k;
      As[m][k] = (gm < g.M && gk < g.K) ? A[gm * g.aRow + gk * g.aCol] : (u16)0;
      int n, kb;
      if (bNfast) { kb = e / BN; n = e % BN; } else { n = e / BK; kb = e % BK; }
      long long gn = n0 + n, gkb = k0 + kb;
      Bs[n][kb] = (gn < g.N && gkb < g.K) ? B[gkb * g.bRow + gn * g.bCol] : (u16)0;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < BK; kk += 16) {
      bf16x8 av = *(const bf16x8*)&As[wm * 32 + (lane & 31)][kk + (lane >> 5) * 8];
      bf16x8 bv = *(const bf16x8*)&Bs[wn * 32 + (lane & 31)][kk + (lane >> 5) * 8];
      acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(av, bv, acc, 0, 0, 0);
    }
    __syncthreads();
  }
  const long long cBase = (long long)blockIdx.z * g.M * g.N;
  const long long col = n0 + wn * 32 + (lane & 31);
  if (col >= g.N) return;
#pragma unroll
  for (int j = 0; j < 16; ++j) {
    long long row = m0 + wm * 32 + (j >> 2) * 8 + (lane >> 5) * 4 + (j & 3);
    if (row < g.M) {
      if (g.outBf16) ((u16*)g.c)[cBase + row * g.N + col] = f2bf(acc[j]);
      else ((float*)g.c)[cBase + row * g.N + col] = acc[j];
    }
  }
}

// ------------------------------------------------------------ convolution
// Direct form: one thread per output element, fp32 accumulation.  Handles every
// combination the StableHLO op allows (dimension numbers through strides, window
// strides, negative padding, lhs/rhs dilation, window reversal, feature and batch groups).
struct ConvArgs {
  mi355_conv_desc d;
  const void* lhs;
  const void* rhs;
  void* out;
  long long total;
};

template <typename T>
__device__ __forceinline__ float ldf(const T* p);
template <>
__device__ __forceinline__ float ldf<float>(const float* p) { return *p; }
template <>
__device__ __forceinline__ float ldf<u16>(const u16* p) { return bf2f(*p); }

template <typename T>
__global__ void __launch_bounds__(256) conv_direct(ConvArgs a) {
  const mi355_conv_desc& d = a.d;
  long long i = (long long)blockIdx.x * 256 + threadIdx.x;
  if (i >= a.total) return;
  // decompose i -> (b, o0, o1, o2, f) with f fastest when outF == 1 (feature-minor outputs), generic otherwise
  long long r = i;
  long long f = r % d.O; r /= d.O;
  long long os[3] = {0, 0, 0};
  for (int s = d.nsp - 1; s >= 0; --s) { os[s] = r % d.out[s]; r /= d.out[s]; }
  long long b = r;
  const long long groups = d.featureGroups > 1 ? d.featureGroups : d.batchGroups;
  const long long opg = d.O / (groups > 0 ? groups : 1);   // output features per group
  long long cPerGroup = d.C / d.featureGroups;
  long long cBase = 0, bBase = b;
  if (d.featureGroups > 1) cBase = (f / opg) * cPerGroup;
  if (d.batchGroups > 1) bBase = (f / opg) * d.N + b;
  const T* L = (const T*)a.lhs;
  const T* R = (const T*)a.rhs;
  float acc = 0.f;
  const long long k0n = d.k[0], k1n = d.nsp > 1 ? d.k[1] : 1, k2n = d.nsp > 2 ? d.k[2] : 1;
  for (long long k0 = 0; k0 < k0n; ++k0) {
    long long p0 = os[0] * d.stride[0] - d.padLo[0] + k0 * d.rdil[0];
    if (p0 < 0 || p0 % d.ldil[0] != 0) continue;
    p0 /= d.ldil[0];
    if (p0 >= d.in[0]) continue;
    long long kk0 = d.rev[0] ? d.k[0] - 1 - k0 : k0;
    for (long long k1 = 0; k1 < k1n; ++k1) {
      long long p1 = 0, kk1 = 0;
      if (d.nsp > 1) {
        p1 = os[1] * d.stride[1] - d.padLo[1] + k1 * d.rdil[1];
        if (p1 < 0 || p1 % d.ldil[1] != 0) continue;
        p1 /= d.ldil[1];
        if (p1 >= d.in[1]) continue;
        kk1 = d.rev[1] ? d.k[1] - 1 - k1 : k1;
      }
      for (long long k2 = 0; k2 < k2n; ++k2) {
        long long p2 = 0, kk2 = 0;
        if (d.nsp > 2) {
          p2 = os[2] * d.stride[2] - d.padLo[2] + k2 * d.rdil[2];
          if (p2 < 0 || p2 % d.ldil[2] != 0) continue;
          p2 /= d.ldil[2];
          if (p2 >= d.in[2]) continue;
          kk2 = d.rev[2] ? d.k[2] - 1 - k2 : k2;
        }
        const T* lp = L + bBase * d.lhsB + cBase * d.lhsF + p0 * d.lhsS[0] + p1 * d.lhsS[1] + p2 * d.lhsS[2];
        const T* rp = R + f * d.rhsO + kk0 * d.rhsS[0] + kk1 * d.rhsS[1] + kk2 * d.rhsS[2];
        for (long long c = 0; c < cPerGroup; ++c) acc += ldf<T>(lp + c * d.lhsF) * ldf<T>(rp + c * d.rhsI);
      }
    }
  }
  long long off = b * d.outB + f * d.outF + os[0] * d.outS[0] + os[1] * d.outS[1] + os[2] * d.outS[2];
  if (sizeof(T) == 2) ((u16*)a.out)[off] = f2bf(acc);
  else ((float*)a.out)[off] = acc;
}

// ---------------------------------------------------------- row scatter
// keys[i] = destination row of update i (`rows` if outside the operand: dropped),
// vals[i] = i.  A stable LSD radix sort by key keeps updates of one row in their
// original order; every row segment is then folded front to back.
__global__ void __launch_bounds__(256) scatter_init_keys(const void* idx, int idxBytes, long long n, long long rows, u32* keys, u32* vals) {
  long long i = (long long)blockIdx.x * 256 + threadIdx.x;
  if (i >= n) return;
  long long r = idxBytes == 8 ? ((const long long*)idx)[i] : (long long)((const int*)idx)[i];
  keys[i] = (r < 0 || r >= rows) ? (u32)rows : (u32)r;   // rows = "dropped", sorts last
  vals[i] = (u32)i;
}

constexpr int kSortBlocks = 64;

__global__ void __launch_bounds__(256) radix_hist(const u32* __restrict__ keys, long long n, int shift, u32* __restrict__ counts) {
  __shared__ u32 h[256];
  h[threadIdx.x] = 0;
  __syncthreads();
  long long chunk = (n + gridDim.x - 1) / gridDim.x;
  long long lo = (long long)blockIdx.x * chunk, hi = lo + chunk < n ? lo + chunk : n;
  for (long long i = lo + threadIdx.x; i < hi; i += 256) atomicAdd(&h[(keys[i] >> shift) & 255u], 1u);
  __syncthreads();
  counts[threadIdx.x * gridDim.x + blockIdx.x] = h[threadIdx.x];   // digit-major
}

__global__ void __launch_bounds__(256) radix_scan(u32* counts, int nblocks) {
  // exclusive scan over 256*nblocks counters, digit-major; one workgroup
  __shared__ u32 tot[256];
  u32 sum = 0;
  for (int b = 0; b < nblocks; ++b) sum += counts[threadIdx.x * nblocks + b];
  tot[threadIdx.x] = sum;
  __syncthreads();
  if (threadIdx.x == 0) {
    u32 run = 0;
    for (int d = 0; d < 256; ++d) { u32 t = tot[d]; tot[d] = run; run += t; }
  }
  __syncthreads();
  u32 run = tot[threadIdx.x];
  for (int b = 0; b < nblocks; ++b) {
    u32 c = counts[threadIdx.x * nblocks + b];
    counts[threadIdx.x * nblocks + b] = run;
    run += c;
  }
}

__global__ void __launch_bounds__(256) radix_scatter(const u32* __restrict__ keysIn, const u32* __restrict__ valsIn, long long n, int shift,
                                                     const u32* __restrict__ offsets, u32* __restrict__ keysOut, u32* __restrict__ valsOut) {
  __shared__ u32 base[256];          // running output position per digit for this block
  __shared__ u32 waveCount[4][256];  // per-wave digit counts of the current tile
  base[threadIdx.x] = offsets[threadIdx.x * gridDim.x + blockIdx.x];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  long long chunk = (n + gridDim.x - 1) / gridDim.x;
  long long lo = (long long)blockIdx.x * chunk, hi = lo + chunk < n ? lo + chunk : n;
  for (long long t0 = lo; t0 < hi; t0 += 256) {
    for (int w = 0; w < 4; ++w) waveCount[w][threadIdx.x] = 0;
    __syncthreads();
    long long i = t0 + threadIdx.x;
    bool valid = i < hi;
    u32 key = valid ? keysIn[i] : 0u, val = valid ? valsIn[i] : 0u;
    u32 digit = (key >> shift) & 255u;
    // lanes of this wavefront holding the same digit
    unsigned long long peers = __ballot(valid);
#pragma unroll
    for (int b = 0; b < 8; ++b) {
      unsigned long long m = __ballot((digit >> b) & 1u);
      peers &= ((digit >> b) & 1u) ? m : ~m;
    }
    unsigned long long lower = peers & ((1ull << lane) - 1ull);
    u32 rankInWave = (u32)__popcll(lower);
    if (valid && lower == 0) waveCount[wave][digit] = (u32)__popcll(peers);
    __syncthreads();
    if (valid) {
      u32 pos = base[digit] + rankInWave;
      for (int w = 0; w < wave; ++w) pos += waveCount[w][digit];
      keysOut[pos] = key;
      valsOut[pos] = val;
    }
    __syncthreads();
    base[threadIdx.x] += waveCount[0][threadIdx.x] + waveCount[1][threadIdx.x] + waveCount[2][threadIdx.x] + waveCount[3][threadIdx.x];
    __syncthreads();
  }
}

// Up to 8192 updates (the benchmark's embedding batch) are sorted by one workgroup in LDS: the seven launches of
// the general path cost more in launch latency than the sort itself.  1024 lanes hold eight (key, update number)
// pairs each, pair (w, k, lane) at index w * 512 + k * 64 + lane.  One pass per 8-bit digit: a wavefront ranks its
// 64 pairs of a round among themselves with ballots and keeps a running count per digit in its own column of
// cnt[digit][wave]; an exclusive scan of cnt in (digit, wave) order gives every (digit, wave) its first output
// position; pairs are written to LDS at their position and read back in index order.  Equal digits keep their
// index order in every pass, so the sort is stable.  Slots past n hold key 0xFFFFFFFF: their digits are 255 in
// every pass and they start behind every real pair, so they end behind every real pair.
constexpr int kSmallSort = 8192;

// Splat fill of the scatter result for workgroups 1 .. gridDim.x - 1 (workgroup 0 sorts meanwhile, or does nothing
// in the launch of the general sort path): 16-byte stores, the last bytes of an odd size in 16-bit units.
__device__ __forceinline__ void fillSplat(unsigned char* dst, unsigned long long bytes, u32 bits32) {
  const unsigned long long n16 = bytes / 16, lanes = (unsigned long long)(gridDim.x - 1) * blockDim.x;
  const uint4 v = make_uint4(bits32, bits32, bits32, bits32);
  for (unsigned long long i = (unsigned long long)(blockIdx.x - 1) * blockDim.x + threadIdx.x; i < n16; i += lanes) ((uint4*)dst)[i] = v;
  if (blockIdx.x == 1 && threadIdx.x < (bytes % 16) / 2) ((u16*)(dst + n16 * 16))[threadIdx.x] = (u16)(threadIdx.x & 1 ? bits32 >> 16 : bits32);
}

__global__ void __launch_bounds__(1024) scatter_fill(unsigned char* fillDst, unsigned long long fillBytes, u32 fillBits) {
  if (blockIdx.x > 0) fillSplat(fillDst, fillBytes, fillBits);
}

__global__ void __launch_bounds__(1024) scatter_sort_small(const void* idx, int idxBytes, int n, long long rows, int bits,
                                                           u32* __restrict__ keysOut, u32* __restrict__ valsOut,
                                                           unsigned char* fillDst, unsigned long long fillBytes, u32 fillBits) {
  if (blockIdx.x > 0) {
    fillSplat(fillDst, fillBytes, fillBits);
    return;
  }
  __shared__ u32 keysL[kSmallSort];
  __shared__ u16 valsL[kSmallSort];
  __shared__ u16 cnt[256][16];
  __shared__ u32 waveTotal[16];
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  u32 key[8], val[8];
#pragma unroll
  for (int k = 0; k < 8; ++k) {
    const int i = w * 512 + k * 64 + lane;
    val[k] = (u32)i;
    key[k] = 0xFFFFFFFFu;
    if (i < n) {
      long long r = idxBytes == 8 ? ((const long long*)idx)[i] : (long long)((const int*)idx)[i];
      key[k] = (r < 0 || r >= rows) ? (u32)rows : (u32)r;   // rows = "dropped", sorts behind every row
    }
  }
  for (int shift = 0; shift < bits; shift += 8) {
    ((u32*)&cnt[0][0])[threadIdx.x] = 0;
    ((u32*)&cnt[0][0])[threadIdx.x + 1024] = 0;
    __syncthreads();
    u32 local[8];
#pragma unroll
    for (int k = 0; k < 8; ++k) {
      const u32 digit = (key[k] >> shift) & 255u;
      unsigned long long peers = ~0ull;
#pragma unroll
      for (int b = 0; b < 8; ++b) {
        const unsigned long long m = __ballot((digit >> b) & 1u);
        peers &= ((digit >> b) & 1u) ? m : ~m;
      }
      const unsigned long long lower = peers & ((1ull << lane) - 1ull);
      const u32 before = cnt[digit][w];                     // pairs of this digit in this wavefront's earlier rounds
      local[k] = before + (u32)__popcll(lower);
      __builtin_amdgcn_wave_barrier();                      // every lane has read the count before its leader moves it on
      if (lower == 0) cnt[digit][w] = (u16)(before + (u32)__popcll(peers));
      __builtin_amdgcn_wave_barrier();
    }
    __syncthreads();
    // exclusive scan of the 4096 counts in (digit, wave) order: four per lane, wavefront scan, wavefront totals
    u16* flat = &cnt[0][0];
    const u32 c0 = flat[4 * threadIdx.x], c1 = flat[4 * threadIdx.x + 1], c2 = flat[4 * threadIdx.x + 2], c3 = flat[4 * threadIdx.x + 3];
    const u32 mine = c0 + c1 + c2 + c3;
    u32 incl = mine;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
      const u32 up = __shfl_up(incl, d);
      if (lane >= d) incl += up;
    }
    if (lane == 63) waveTotal[w] = incl;
    __syncthreads();
    u32 base = incl - mine;
    for (int q = 0; q < w; ++q) base += waveTotal[q];
    flat[4 * threadIdx.x] = (u16)base;
    flat[4 * threadIdx.x + 1] = (u16)(base + c0);
    flat[4 * threadIdx.x + 2] = (u16)(base + c0 + c1);
    flat[4 * threadIdx.x + 3] = (u16)(base + c0 + c1 + c2);
    __syncthreads();
#pragma unroll
    for (int k = 0; k < 8; ++k) {
      const u32 pos = cnt[(key[k] >> shift) & 255u][w] + local[k];
      keysL[pos] = key[k];
      valsL[pos] = (u16)val[k];
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < 8; ++k) {
      const int i = w * 512 + k * 64 + lane;
      key[k] = keysL[i];
      val[k] = valsL[i];
    }
    __syncthreads();
  }
#pragma unroll
  for (int k = 0; k < 8; ++k) {
    const int i = w * 512 + k * 64 + lane;
    if (i < n) {
      keysOut[i] = key[k];
      valsOut[i] = val[k];
    }
  }
}

template <typename T>
struct ScatterOps;
template <>
struct ScatterOps<float> {
  static __device__ __forceinline__ float apply(int kind, float a, float u) {
    switch (kind) {
      case 0: return a + u;
      case 1: return u;
      case 2: return a * u;
      case 3: return (a < u || a != a) ? a : u;
      default: return (a > u || a != a) ? a : u;
    }
  }
};
template <>
struct ScatterOps<int> {
  static __device__ __forceinline__ int apply(int kind, int a, int u) {
    switch (kind) {   // (sums and products wrap: computed on the unsigned type)
      case 0: return (int)((u32)a + (u32)u);
      case 1: return u;
      case 2: return (int)((u32)a * (u32)u);
      case 3: return a < u ? a : u;
      default: return a > u ? a : u;
    }
  }
};
template <>
struct ScatterOps<u32> {
  static __device__ __forceinline__ u32 apply(int kind, u32 a, u32 u) {
    switch (kind) {
      case 0: return a + u;
      case 1: return u;
      case 2: return a * u;
      case 3: return a < u ? a : u;
      default: return a > u ? a : u;
    }
  }
};

// Segment fold.  After the stable sort, the updates of one destination row are a run of equal
// keys whose values (update numbers) ascend; applying them in that order to the row is exactly
// what a sequential scatter does, bit for bit, and rows are independent of each other.
//
// Storage / accumulator policies (bf16 rounds after every application, like a bf16 loop would).
template <typename T>
struct Plain {
  typedef T S;
  typedef T A;
  static __device__ __forceinline__ A load(S s) { return s; }
  static __device__ __forceinline__ S store(A a) { return a; }
  static __device__ __forceinline__ A apply(int kind, A a, S u) { return ScatterOps<T>::apply(kind, a, u); }
};
struct Bf16 {
  typedef u16 S;
  typedef float A;
  static __device__ __forceinline__ A load(S s) { return bf2f(s); }
  static __device__ __forceinline__ S store(A a) { return f2bf(a); }
  static __device__ __forceinline__ A apply(int kind, A a, S u) { return bf2f(f2bf(ScatterOps<float>::apply(kind, a, bf2f(u)))); }
};

// Ends of the run of `key` around a position known to hold it, in sorted keys.  Every lane of a wavefront probes
// one position per step (64-way search: three dependent loads for 8192 keys where a bisection needs thirteen);
// all lanes return the same value.
__device__ __forceinline__ long long runHead(const u32* __restrict__ keys, long long p, u32 key, int lane) {
  long long lo = 0, hi = p;                 // the first position holding `key` lies in [lo, hi]; keys[hi] == key
  while (lo < hi) {
    const long long step = (hi - lo + 62) / 63;                // 63 steps reach hi: the last lane always answers
    const long long pos = lo + lane * step;
    const bool here = pos >= hi || keys[pos] == key;           // sorted: positions holding `key` form a suffix of [lo, hi]
    const int f = __ffsll((long long)__ballot(here)) - 1;      // lane 63 has pos >= hi, so f >= 0
    const long long top = lo + f * step;
    lo = f > 0 ? top - step + 1 : lo;
    hi = top < hi ? top : hi;
  }
  return lo;
}
__device__ __forceinline__ long long runLast(const u32* __restrict__ keys, long long p, long long n, u32 key, int lane) {
  long long lo = p, hi = n - 1;             // the last position holding `key` lies in [lo, hi]; keys[lo] == key
  while (lo < hi) {
    const long long step = (hi - lo + 62) / 63;
    const long long pos = hi - lane * step;
    const bool here = pos <= lo || keys[pos] == key;           // positions holding `key` form a prefix of [lo, hi]
    const int f = __ffsll((long long)__ballot(here)) - 1;
    const long long bottom = hi - f * step;
    hi = f > 0 ? bottom + step - 1 : hi;
    lo = bottom > lo ? bottom : lo;
  }
  return lo;
}

constexpr int kLongSegment = 16;   // runs at least this long go to the column-parallel kernels
constexpr int kHugeSegment = 256;  // runs at least this long go to the narrow-column kernel with deep prefetch

template <typename P, int C>
__device__ __forceinline__ void foldShortRun(typename P::A& acc, const u32* __restrict__ vals, int cnt, const typename P::S* __restrict__ updates,
                                             long long rowElems, long long col, int kind) {
  u32 src[C];
#pragma unroll
  for (int q = 0; q < C; ++q) src[q] = vals[q < cnt ? q : cnt - 1];
  typename P::S u[C];
#pragma unroll
  for (int q = 0; q < C; ++q) u[q] = updates[(long long)src[q] * rowElems + col];
#pragma unroll
  for (int q = 0; q < C; ++q)
    if (q < cnt) acc = P::apply(kind, acc, u[q]);
}

// Short runs (fewer than kLongSegment updates, the common case): one workgroup per run head and chunk of 256
// columns; every lane fetches all updates of its column at once, then applies them in order.
template <typename P>
__device__ __forceinline__ void foldShortRuns(long long i, unsigned colChunk, const u32* __restrict__ keys, const u32* __restrict__ vals, long long n,
                                              long long rowElems, int kind, typename P::S* __restrict__ result,
                                              const typename P::S* __restrict__ updates, u32 rows) {
  const u32 key = keys[i];
  if (key >= rows) return;
  if (i > 0 && keys[i - 1] == key) return;
  if (i + kLongSegment - 1 < n && keys[i + kLongSegment - 1] == key) return;   // long run: other kernel
  const long long col = (long long)colChunk * 256 + threadIdx.x;
  if (col >= rowElems) return;
  int cnt = 1;
  while (cnt < kLongSegment && i + cnt < n && keys[i + cnt] == key) ++cnt;
  typename P::A acc = P::load(result[(long long)key * rowElems + col]);
  // The run length is the same for the whole workgroup; by length class, all loads of the class are issued
  // unconditionally (positions past the run repeat its last update and are not applied), so they are in flight
  // together instead of one branch and one round trip per update.
  if (cnt <= 1) foldShortRun<P, 1>(acc, vals + i, cnt, updates, rowElems, col, kind);
  else if (cnt <= 2) foldShortRun<P, 2>(acc, vals + i, cnt, updates, rowElems, col, kind);
  else if (cnt <= 4) foldShortRun<P, 4>(acc, vals + i, cnt, updates, rowElems, col, kind);
  else if (cnt <= 8) foldShortRun<P, 8>(acc, vals + i, cnt, updates, rowElems, col, kind);
  else foldShortRun<P, kLongSegment - 1>(acc, vals + i, cnt, updates, rowElems, col, kind);
  result[(long long)key * rowElems + col] = P::store(acc);
}

template <typename P>
__global__ void __launch_bounds__(256) scatter_fold_short(const u32* __restrict__ keys, const u32* __restrict__ vals, long long n, long long rowElems,
                                                          int kind, typename P::S* __restrict__ result, const typename P::S* __restrict__ updates, u32 rows) {
  foldShortRuns<P>(blockIdx.x, blockIdx.y, keys, vals, n, rowElems, kind, result, updates, rows);
}

// Long runs (hot rows of a skewed index distribution) are bound by the latency of fetching their updates and by
// the sequential fold (about 5 ns per update and column: one LDS read and one dependent operation), so the row is
// cut into column chunks, one workgroup each, and many fetches are in flight: four wavefronts stage a round of
// updates in LDS (32 independent loads per lane), then the first wavefront applies the staged values of its column
// in order.  Runs of kLongSegment .. kHugeSegment - 1 updates use chunks of 64 columns and rounds of 128 updates
// (scatter_fold_long); longer ones (the head of a Zipf distribution: a tenth of all updates go to one row) chunks of
// 8 columns and rounds of 1024, a wavefront load covering eight updates, with the fetches of the next round issued
// before the staged one is folded and the update numbers of round r + 1 fetched during round r - 1
// (scatter_fold_huge).  A run of length >= L contains a multiple of L, so only those positions get a workgroup, and
// the first of them inside the run does the work.
//
// Workgroup number = position * chunks + column chunk.  The column chunk is the fast index because workgroups with
// neighbouring numbers go to different XCDs and shader engines: with the position as the fast index, the few
// workgroups that find work (one run's chunks) all landed on the eight CUs of one shader engine and ran in turns.
template <typename P, int KIND, int STRIDE>
__device__ __forceinline__ void foldStaged(typename P::A& acc, const typename P::S* column, int m) {
  int r = 0;
  for (; r + 16 <= m; r += 16) {
    typename P::S v[16];
#pragma unroll
    for (int q = 0; q < 16; ++q) v[q] = column[(r + q) * STRIDE];
#pragma unroll
    for (int q = 0; q < 16; ++q) acc = P::apply(KIND, acc, v[q]);
  }
  for (; r < m; ++r) acc = P::apply(KIND, acc, column[r * STRIDE]);
}

template <typename P, int kCols, int kPerLane>
__device__ __forceinline__ void foldLongRun(typename P::S* stage, const u32* __restrict__ vals, long long rowElems, int kind,
                                            typename P::S* __restrict__ result, const typename P::S* __restrict__ updates,
                                            u32 key, long long head, long long total, u32 chunk, int lane, int w) {
  typedef typename P::S S;
  constexpr int kSubs = 64 / kCols;                 // updates per wavefront load
  constexpr int kStep = 4 * kSubs;                  // updates per load of the whole workgroup
  constexpr int kRound = kStep * kPerLane;
  const int sub = lane / kCols, c = lane % kCols;
  const long long col = (long long)chunk * kCols + c;
  const bool active = col < rowElems;
  const long long colc = active ? col : rowElems - 1;
  const bool folder = w == 0 && sub == 0 && active;
  typename P::A acc = typename P::A();
  if (folder) acc = P::load(result[(long long)key * rowElems + col]);
  // Every load is unconditional (a predicated load is a branch around it): positions past the run repeat its last
  // update, columns past the row the last column; neither is folded or stored.
  auto fetchNumbers = [&](long long round, u32* vi) {
#pragma unroll
    for (int q = 0; q < kPerLane; ++q) {
      const long long t = round * kRound + q * kStep + w * kSubs + sub;
      vi[q] = vals[head + (t < total ? t : total - 1)];
    }
  };
  const long long rounds = (total + kRound - 1) / kRound;
  u32 vi[kPerLane], vnext[kPerLane];
  S u[kPerLane];
  // The scheduling fences keep each group of loads together: interleaved with the loads that depend on them,
  // every pair waits for its own round trip and the latencies add up.
  fetchNumbers(0, vi);
  __builtin_amdgcn_sched_barrier(0);
  fetchNumbers(rounds > 1 ? 1 : 0, vnext);
  __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int q = 0; q < kPerLane; ++q) u[q] = updates[(long long)vi[q] * rowElems + colc];
  __builtin_amdgcn_sched_barrier(0);
  for (long long r = 0; r < rounds; ++r) {
#pragma unroll
    for (int q = 0; q < kPerLane; ++q) stage[(q * kStep + w * kSubs + sub) * kCols + c] = u[q];
    __builtin_amdgcn_sched_barrier(0);
    if (r + 1 < rounds) {
#pragma unroll
      for (int q = 0; q < kPerLane; ++q) u[q] = updates[(long long)vnext[q] * rowElems + colc];
      __builtin_amdgcn_sched_barrier(0);
      fetchNumbers(r + 2 < rounds ? r + 2 : r + 1, vnext);
      __builtin_amdgcn_sched_barrier(0);
    }
    __syncthreads();
    if (folder) {
      const long long left = total - r * kRound;
      const int m = left < kRound ? (int)left : kRound;
      // the combiner is fixed outside the loop so that the LDS reads of a column pipeline
      switch (kind) {
        case 0: foldStaged<P, 0, kCols>(acc, stage + c, m); break;
        case 1: foldStaged<P, 1, kCols>(acc, stage + c, m); break;
        case 2: foldStaged<P, 2, kCols>(acc, stage + c, m); break;
        case 3: foldStaged<P, 3, kCols>(acc, stage + c, m); break;
        default: foldStaged<P, 4, kCols>(acc, stage + c, m); break;
      }
    }
    __syncthreads();
  }
  if (folder) result[(long long)key * rowElems + col] = P::store(acc);
}

constexpr int kHugeCols = 8, kHugePerLane = 32;

// Very long runs: chunks of 8 columns and rounds of 1024 updates (see above).
template <typename P>
__global__ void __launch_bounds__(256) scatter_fold_huge(const u32* __restrict__ keys, const u32* __restrict__ vals, long long n, long long rowElems,
                                                          int kind, typename P::S* __restrict__ result, const typename P::S* __restrict__ updates, u32 rows, u32 chunks) {
  typedef typename P::S S;
  __shared__ S stage[4 * (64 / kHugeCols) * kHugePerLane * kHugeCols];
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  const u32 chunk = blockIdx.x % chunks;                       // workgroup number = position * chunks + column chunk
  const long long p = (long long)(blockIdx.x / chunks) * kHugeSegment;
  if (p >= n) return;
  const u32 key = keys[p];
  if (key >= rows) return;
  if (p >= kHugeSegment && keys[p - kHugeSegment] == key) return;                    // an earlier workgroup owns this run
  const long long head = runHead(keys, p, key, lane);
  if (head + kHugeSegment - 1 >= n || keys[head + kHugeSegment - 1] != key) return;   // shorter run: other kernels
  const long long total = runLast(keys, head + kHugeSegment - 1, n, key, lane) - head + 1;
  foldLongRun<P, kHugeCols, kHugePerLane>(stage, vals, rowElems, kind, result, updates, key, head, total, chunk, lane, w);
}

// Long runs below kHugeSegment: chunks of 64 columns, rounds of 128 updates whose numbers are staged through LDS.
template <typename P>
__device__ __forceinline__ void foldLongRuns(unsigned block, const u32* __restrict__ keys, const u32* __restrict__ vals, long long n, long long rowElems,
                                             int kind, typename P::S* __restrict__ result, const typename P::S* __restrict__ updates, u32 rows, u32 chunks) {
  typedef typename P::S S;
  constexpr int kWaves = 4, kPerLane = 32, kRound = kWaves * kPerLane;   // 128 updates x 64 columns staged per round
  __shared__ u32 sval[256];
  __shared__ S stage[kRound][64];
  const u32 chunk = block % chunks;                            // workgroup number = position * chunks + column chunk
  const long long p = (long long)(block / chunks) * kLongSegment;
  if (p >= n) return;
  const u32 key = keys[p];
  if (key >= rows) return;
  if (p >= kLongSegment && keys[p - kLongSegment] == key) return;                    // an earlier workgroup owns this run
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  const long long head = runHead(keys, p, key, lane);
  if (head + kLongSegment - 1 >= n || keys[head + kLongSegment - 1] != key) return;   // short run
  if (head + kHugeSegment - 1 < n && keys[head + kHugeSegment - 1] == key) return;    // very long run: scatter_fold_huge
  const long long col = (long long)chunk * 64 + lane;
  const bool active = col < rowElems;
  const long long colc = active ? col : rowElems - 1;
  typename P::A acc = typename P::A();
  if (w == 0 && active) acc = P::load(result[(long long)key * rowElems + col]);
  for (long long base = head;; base += 256) {
    const long long j = base + threadIdx.x;
    const bool mine = j < n && keys[j] == key;
    __syncthreads();
    sval[threadIdx.x] = mine ? vals[j] : 0u;
    const int cnt = __syncthreads_count(mine);   // sorted: the matches are a prefix of the tile
    for (int t0 = 0; t0 < cnt; t0 += kRound) {
      const int m = cnt - t0 < kRound ? cnt - t0 : kRound;
      // All 32 loads of a lane are unconditional (a predicated load is a branch around it, and 32 branches issue
      // far slower than 32 loads): positions past the run read update row sval[..] = 0 and columns past the row
      // read the last column; neither is ever folded or stored.
      S u[kPerLane];
#pragma unroll
      for (int q = 0; q < kPerLane; ++q) u[q] = updates[(long long)sval[t0 + w + kWaves * q] * rowElems + colc];
#pragma unroll
      for (int q = 0; q < kPerLane; ++q) stage[w + kWaves * q][lane] = u[q];
      __syncthreads();
      if (w == 0 && active) {
        // the combiner is fixed outside the loop so that the LDS reads of a column pipeline
        switch (kind) {
          case 0: foldStaged<P, 0, 64>(acc, &stage[0][lane], m); break;
          case 1: foldStaged<P, 1, 64>(acc, &stage[0][lane], m); break;
          case 2: foldStaged<P, 2, 64>(acc, &stage[0][lane], m); break;
          case 3: foldStaged<P, 3, 64>(acc, &stage[0][lane], m); break;
          default: foldStaged<P, 4, 64>(acc, &stage[0][lane], m); break;
        }
      }
      __syncthreads();
    }
    if (cnt < 256) break;
  }
  if (w == 0 && active) result[(long long)key * rowElems + col] = P::store(acc);
}

template <typename P>
__global__ void __launch_bounds__(256) scatter_fold_long(const u32* __restrict__ keys, const u32* __restrict__ vals, long long n, long long rowElems,
                                                         int kind, typename P::S* __restrict__ result, const typename P::S* __restrict__ updates, u32 rows, u32 chunks) {
  foldLongRuns<P>(blockIdx.x, keys, vals, n, rowElems, kind, result, updates, rows, chunks);
}

// Runs below kHugeSegment, short and long, in one launch: workgroups [0, blocksLong) take the long runs, the rest the
// short ones (run head = rest / chunksShort, 256-column chunk = rest % chunksShort).  The two classes touch different
// rows and each is a short chain of dependent fetches, so side by side they take the time of one.
template <typename P>
__global__ void __launch_bounds__(256) scatter_fold_runs(const u32* __restrict__ keys, const u32* __restrict__ vals, long long n, long long rowElems,
                                                         int kind, typename P::S* __restrict__ result, const typename P::S* __restrict__ updates, u32 rows,
                                                         u32 chunksLong, u32 blocksLong, u32 chunksShort) {
  if (blockIdx.x < blocksLong) {
    foldLongRuns<P>(blockIdx.x, keys, vals, n, rowElems, kind, result, updates, rows, chunksLong);
    return;
  }
  const u32 rest = blockIdx.x - blocksLong;
  foldShortRuns<P>(rest / chunksShort, rest % chunksShort, keys, vals, n, rowElems, kind, result, updates, rows);
}

namespace {
thread_local const char* g_kerr = "";
int check(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) { g_kerr = what; return (int)e; }
  return 0;
}
}  // namespace

extern "C" {

int mi355_copy(void* dst, const void* src, size_t bytes, mi355_stream_t s) {
  if (bytes == 0 || dst == src) return 0;
  hipStream_t st = (hipStream_t)s;
  if (((uintptr_t)dst | (uintptr_t)src | bytes) % 16 == 0) {
    size_t n16 = bytes / 16;
    copy_vec16<<<(unsigned)((n16 + 255) / 256), 256, 0, st>>>((const uint4*)src, (uint4*)dst, n16);
  } else {
    copy_bytes<<<(unsigned)((bytes + 255) / 256), 256, 0, st>>>((const unsigned char*)src, (unsigned char*)dst, bytes);
  }
  return check("copy");
}

int mi355_flag_init(void* flag, const void* parent, mi355_stream_t s) {
  flag_update<<<1, 64, 0, (hipStream_t)s>>>((int*)flag, (const int*)parent, nullptr);
  return check("flag_init");
}
int mi355_flag_and(void* flag, const void* pred, mi355_stream_t s) {
  flag_update<<<1, 64, 0, (hipStream_t)s>>>((int*)flag, nullptr, (const unsigned char*)pred);
  return check("flag_and");
}

int mi355_copy_multi(int n, void* const* dst, const void* const* src, const size_t* bytes, mi355_stream_t s) {
  return mi355_copy_multi_if(n, dst, src, bytes, nullptr, s);
}

int mi355_copy_multi_if(int n, void* const* dst, const void* const* src, const size_t* bytes, const mi355_copy_cond* cond, mi355_stream_t s) {
  if (n <= 0) return 0;
  if (n > 16) return 1;
  MultiCopyArgs a;
  a.flag = cond ? cond->flag : nullptr;
  a.mode = cond ? cond->mode : 0;
  a.indexBytes = cond ? cond->index_bytes : 0;
  a.want = cond ? cond->want : 0;
  a.count = cond ? cond->count : 0;
  if (a.mode != 0 && !a.flag) return 1;
  size_t most = 0;
  for (int i = 0; i < n; ++i) {
    a.src[i] = (const unsigned char*)src[i];
    a.dst[i] = (unsigned char*)dst[i];
    a.bytes[i] = bytes[i];
    size_t units = ((((uintptr_t)src[i] | (uintptr_t)dst[i] | bytes[i]) & 15) == 0) ? bytes[i] / 16 : bytes[i];
    most = units > most ? units : most;
  }
  if (most == 0) return 0;
  unsigned gx = (unsigned)((most + 255) / 256);
  if (gx > 2048) gx = 2048;
  copy_multi<<<dim3(gx, (unsigned)n), 256, 0, (hipStream_t)s>>>(a);
  return check("copy_multi");
}

// An unbatched fp32 GEMM is a convolution without spatial dims (rows = batch, k = input
// features, columns = output features): it then runs on the implicit-GEMM kernel with its
// vector tile loaders, register prefetch and split-K for shapes with few output tiles.
static bool gemmAsPointwiseConv(const mi355_gemm_desc* d, mi355_conv_desc* c) {
  if (d->in_dtype != 0 || d->out_dtype != 0 || d->batch0 * d->batch1 != 1 || d->K <= 0) return false;
  *c = mi355_conv_desc{};
  c->nsp = 0;
  c->N = d->M; c->C = d->K; c->O = d->N;
  c->featureGroups = 1; c->batchGroups = 1;
  c->lhsB = d->aRow; c->lhsF = d->aCol;
  c->rhsI = d->bRow; c->rhsO = d->bCol;
  c->outB = d->N; c->outF = 1;
  c->dtype = 0;
  return true;
}

// Tile edge of the small-product kernel for this GEMM, 0 when the product is big enough to want
// the tiled kernels (enough output tiles to fill the chip, or a long K per tile).
static int smallGemmTile(const mi355_gemm_desc* d) {
  if (d->in_dtype != 0 || d->out_dtype != 0 || d->K <= 0) return 0;
  static const int off = getenv("MI355X_SMALL_GEMM") ? atoi(getenv("MI355X_SMALL_GEMM")) == 0 : 0;
  if (off) return 0;
  const long long nb = d->batch0 * d->batch1;
  if (nb > 65535) return 0;
  const double flops = 2.0 * (double)nb * (double)d->M * (double)d->N * (double)d->K;
  if (flops > 3.0e8) return 0;
  const long long t16 = ((d->M + 15) / 16) * ((d->N + 15) / 16) * nb;
  const long long t32 = ((d->M + 31) / 32) * ((d->N + 31) / 32) * nb;
  if (t16 <= 1024) return 16;
  if (t32 <= 2048) return 32;
  return 0;
}

size_t mi355_gemm_workspace_bytes(const mi355_gemm_desc* d) {
  if (d->in_dtype == 1) return mi355_gemm_bf16_async_workspace_bytes(d);
  if (smallGemmTile(d)) return 0;
  mi355_conv_desc cd;
  if (gemmAsPointwiseConv(d, &cd)) return mi355_conv_workspace_bytes(&cd);
  return 0;
}

static SmallPair smallPair(const mi355_gemm_desc* d, const void* a, const void* b) {
  SmallPair p;
  p.a = (const float*)a; p.b = (const float*)b;
  p.K = d->K;
  p.aB0 = d->aB0; p.aB1 = d->aB1; p.aRow = d->aRow; p.aCol = d->aCol;
  p.bB0 = d->bB0; p.bB1 = d->bB1; p.bRow = d->bRow; p.bCol = d->bCol;
  // 16-byte loads along k: k contiguous, every row / batch offset a multiple of 4 floats, no ragged last super-step
  const bool whole = d->K % 16 == 0;
  auto mult4 = [](long long x) { return x % 4 == 0; };
  p.aVec = whole && d->aCol == 1 && mult4(d->aRow) && mult4(d->aB0) && mult4(d->aB1) && ((uintptr_t)a & 15) == 0;
  p.bVec = whole && d->bRow == 1 && mult4(d->bCol) && mult4(d->bB0) && mult4(d->bB1) && ((uintptr_t)b & 15) == 0;
  return p;
}

int mi355_gemm_is_small(const mi355_gemm_desc* d) { return smallGemmTile(d); }

static bool fillSmall(SmallArgs& g, const void* addend, const mi355_gemm_desc* d1, const void* a1, const void* b1, const mi355_gemm_desc* d2, const void* a2,
                      const void* b2, void* c, const void* bias) {
  if (!smallGemmTile(d1)) return false;
  if (d2 && (!smallGemmTile(d2) || d2->M != d1->M || d2->N != d1->N || d2->batch0 != d1->batch0 || d2->batch1 != d1->batch1)) return false;
  g.p[0] = smallPair(d1, a1, b1);
  g.p[1] = d2 ? smallPair(d2, a2, b2) : g.p[0];
  g.pairs = d2 ? 2 : 1;
  g.c = (float*)c;
  g.bias = (const float*)bias;
  g.addend = (const float*)addend;
  g.M = d1->M; g.N = d1->N;
  g.batch1 = (int)d1->batch1;
  g.relu = d1->act == 2;
  return true;
}

// n <= 4 independent problems of one tile class (mi355_gemm_is_small gives it), each C = A1 x B1 (+ A2 x B2) (+ addend)
// (+ bias); d2[i] and addend[i] may be NULL.
int mi355_gemm_small_group(int n, const mi355_gemm_desc* const* d1, const void* const* a1, const void* const* b1,
                           const mi355_gemm_desc* const* d2, const void* const* a2, const void* const* b2, void* const* c,
                           const void* const* bias, const void* const* addend, mi355_stream_t s) {
  if (n <= 0) return 0;
  if (n > kMaxSmallGroup) return -1;
  SmallGroupArgs g;
  const int t = smallGemmTile(d1[0]);
  unsigned total = 0;
  int k = 0;
  for (int i = 0; i < n; ++i) {
    if (smallGemmTile(d1[i]) != t || !fillSmall(g.prob[k], addend[i], d1[i], a1[i], b1[i], d2[i], a2[i], b2[i], c[i], bias[i])) return -1;
    const long long nb = d1[i]->batch0 * d1[i]->batch1;
    if (d1[i]->M <= 0 || d1[i]->N <= 0 || nb <= 0) continue;
    g.first[k] = total;
    g.tilesN[k] = (unsigned)((d1[i]->N + t - 1) / t);
    g.tilesM[k] = (unsigned)((d1[i]->M + t - 1) / t);
    total += g.tilesN[k] * g.tilesM[k] * (unsigned)nb;
    ++k;
  }
  if (k == 0) return 0;
  g.first[k] = total;
  g.n = k;
  if (t == 16) gemm_f32_small_group<16><<<total, 256, 0, (hipStream_t)s>>>(g);
  else gemm_f32_small_group<32><<<total, 256, 0, (hipStream_t)s>>>(g);
  return check("gemm group");
}

// C = A1 x B1 (+ A2 x B2 when d2 is given: same M, N and batch dims) (+ addend, laid out like C) (+ bias), both products
// small fp32 ones.
int mi355_gemm_small_sum(const mi355_gemm_desc* d1, const void* a1, const void* b1, const mi355_gemm_desc* d2, const void* a2,
                         const void* b2, void* c, const void* bias, const void* addend, mi355_stream_t s) {
  const int t = smallGemmTile(d1);
  if (!t) return -1;
  if (d2 && (!smallGemmTile(d2) || d2->M != d1->M || d2->N != d1->N || d2->batch0 != d1->batch0 || d2->batch1 != d1->batch1)) return -1;
  if (d1->M <= 0 || d1->N <= 0 || d1->batch0 * d1->batch1 <= 0) return 0;
  SmallArgs g;
  g.p[0] = smallPair(d1, a1, b1);
  g.p[1] = d2 ? smallPair(d2, a2, b2) : g.p[0];
  g.pairs = d2 ? 2 : 1;
  g.c = (float*)c;
  g.bias = (const float*)bias;
  g.addend = (const float*)addend;
  g.M = d1->M; g.N = d1->N;
  g.batch1 = (int)d1->batch1;
  g.relu = d1->act == 2;
  dim3 grid((unsigned)((d1->N + t - 1) / t), (unsigned)((d1->M + t - 1) / t), (unsigned)(d1->batch0 * d1->batch1));
  if (t == 16) gemm_f32_small<16><<<grid, 256, 0, (hipStream_t)s>>>(g);
  else gemm_f32_small<32><<<grid, 256, 0, (hipStream_t)s>>>(g);
  return check("gemm");
}

static int addBias(const mi355_gemm_desc* d, void* c, const void* bias, mi355_stream_t s) {
  if (d->act && d->out_dtype != 1) return 2;   // the activation epilogue exists for bf16 results only
  if (!bias && !d->act) return 0;
  const ActArgs act{d->act, d->act_a, d->act_b, d->act_c};
  const long long total = d->batch0 * d->batch1 * d->M * d->N;
  const unsigned grid = (unsigned)((total + 255) / 256);
  if (d->out_dtype == 1) gemm_add_bias<u16><<<grid, 256, 0, (hipStream_t)s>>>((u16*)c, (const u16*)bias, total, d->N, act);
  else gemm_add_bias<float><<<grid, 256, 0, (hipStream_t)s>>>((float*)c, (const float*)bias, total, d->N, act);
  return check("gemm bias");
}

int mi355_gemm(const mi355_gemm_desc* d, const void* a, const void* b, void* c, const void* bias, void* workspace,
               size_t workspace_bytes, mi355_stream_t s) {
  if (d->M <= 0 || d->N <= 0 || d->batch0 * d->batch1 <= 0) return 0;
  GemmArgs g;
  g.a = a; g.b = b; g.c = c;
  g.M = d->M; g.N = d->N; g.K = d->K;
  g.aB0 = d->aB0; g.aB1 = d->aB1; g.aRow = d->aRow; g.aCol = d->aCol;
  g.bB0 = d->bB0; g.bB1 = d->bB1; g.bRow = d->bRow; g.bCol = d->bCol;
  g.batch1 = (int)d->batch1;
  g.outBf16 = d->out_dtype == 1;
  g.bias = bias;
  long long nb = d->batch0 * d->batch1;
  if (d->in_dtype == 1) {
    int r = mi355_gemm_bf16_async(d, a, b, c, bias, workspace, workspace_bytes, s);
    if (r >= 0) return r;
    r = mi355_gemm_bf16_tiled(d, a, b, c, s);
    if (r >= 0) return r ? r : addBias(d, c, bias, s);
  }
  if (d->act == 2 ? !smallGemmTile(d) : (d->act && d->out_dtype != 1)) return 2;   // epilogues: GELU for bf16 results, maximum(x, 0) for small fp32 products
  if (smallGemmTile(d)) return mi355_gemm_small_sum(d, a, b, nullptr, nullptr, nullptr, c, bias, nullptr, s);
  mi355_conv_desc cd;
  // strided views may start anywhere; the implicit-GEMM loaders issue 16-byte loads
  if (gemmAsPointwiseConv(d, &cd) && (((uintptr_t)a | (uintptr_t)b) & 15) == 0) {
    int r = mi355_conv(&cd, a, b, c, workspace, workspace_bytes, s);
    return r ? r : addBias(d, c, bias, s);
  }
  if (nb > 65535) return 1;   // grid.z limit; callers fold larger batches
  dim3 grid((unsigned)((d->N + 63) / 64), (unsigned)((d->M + 63) / 64), (unsigned)nb);
  if (d->in_dtype == 0) gemm_f32_mfma<<<grid, 256, 0, (hipStream_t)s>>>(g);
  else if (d->in_dtype == 1) gemm_bf16_mfma<<<grid, 256, 0, (hipStream_t)s>>>(g);
  else return 2;
  if (int r = check("gemm")) return r;
  return addBias(d, c, bias, s);
}

// Direct convolution: the general fallback behind mi355_conv (groups, 3-d windows, bf16).
int mi355_conv_direct(const mi355_conv_desc* d, const void* lhs, const void* rhs, void* out, mi355_stream_t s) {
  ConvArgs a;
  a.d = *d;
  a.lhs = lhs; a.rhs = rhs; a.out = out;
  long long total = d->N * d->O;
  for (int k = 0; k < d->nsp; ++k) total *= d->out[k];
  a.total = total;
  if (total <= 0) return 0;
  unsigned grid = (unsigned)((total + 255) / 256);
  if (d->dtype == 0) conv_direct<float><<<grid, 256, 0, (hipStream_t)s>>>(a);
  else if (d->dtype == 1) conv_direct<u16><<<grid, 256, 0, (hipStream_t)s>>>(a);
  else return 2;
  return check("conv");
}

size_t mi355_scatter_workspace_bytes(int64_t n) {
  // keys[2][n], vals[2][n], counts[256*kSortBlocks]
  return (size_t)(4 * n * 4 + 256 * kSortBlocks * 4 + 1024);
}

int mi355_scatter_rows(const mi355_scatter_desc* d, void* result, const void* indices, const void* updates, void* workspace,
                       mi355_stream_t s) {
  return mi355_scatter_rows_fill(d, result, indices, updates, workspace, 0, 0, s);
}

int mi355_scatter_rows_fill(const mi355_scatter_desc* d, void* result, const void* indices, const void* updates, void* workspace,
                            int fill, uint32_t fillBits, mi355_stream_t s) {
  long long n = d->numUpdates;
  hipStream_t st = (hipStream_t)s;
  const int elemBytes = d->dtype == 1 ? 2 : 4;
  if (d->dtype < 0 || d->dtype > 3) return 2;
  // grids of the fold launches, checked before anything is enqueued
  const long long chunksHuge = (d->rowElems + kHugeCols - 1) / kHugeCols, chunksLong = (d->rowElems + 63) / 64;
  const long long blocksHuge = chunksHuge * ((n + kHugeSegment - 1) / kHugeSegment), blocksLong = chunksLong * ((n + kLongSegment - 1) / kLongSegment);
  if (blocksHuge > 0x7FFFFFFFll || blocksLong > 0x7FFFFFFFll || n > 0x7FFFFFFFll || (d->rowElems + 255) / 256 > 65535)
    return MI355_SCATTER_GRID_TOO_LARGE;
  const unsigned long long fillBytes = fill ? (unsigned long long)d->operandRows * d->rowElems * elemBytes : 0;
  if (elemBytes == 2) fillBits = (fillBits & 0xFFFFu) | (fillBits << 16);
  // enough workgroups of 1024 lanes to keep every CU writing, each lane storing a few times
  unsigned fillBlocks = (unsigned)((fillBytes / 16 + 8191) / 8192);
  fillBlocks = fillBytes == 0 ? 0 : (fillBlocks < 1 ? 1 : (fillBlocks > 2048 ? 2048 : fillBlocks));
  if (n <= 0 || d->rowElems <= 0) {
    if (fillBlocks) scatter_fill<<<1 + fillBlocks, 1024, 0, st>>>((unsigned char*)result, fillBytes, fillBits);
    return check("scatter_rows");
  }
  u32* keys0 = (u32*)workspace;
  u32* keys1 = keys0 + n;
  u32* vals0 = keys1 + n;
  u32* vals1 = vals0 + n;
  u32* counts = vals1 + n;
  // keys lie in [0, rows]: sort only the bits that can be set
  int bits = 1;
  while (bits < 32 && (1ll << bits) <= d->operandRows) ++bits;
  u32 *kin = keys0, *kout = keys1, *vin = vals0, *vout = vals1;
  static const bool smallSort = !(getenv("MI355X_SCATTER_SMALL_SORT") && getenv("MI355X_SCATTER_SMALL_SORT")[0] == '0');
  const bool small = smallSort && n <= kSmallSort;
  if (small) {
    scatter_sort_small<<<1 + fillBlocks, 1024, 0, st>>>(indices, d->index_bytes, (int)n, d->operandRows, bits, kin, vin,
                                                         (unsigned char*)result, fillBytes, fillBits);
    bits = 0;   // sorted
  } else {
    if (fillBlocks) scatter_fill<<<1 + fillBlocks, 1024, 0, st>>>((unsigned char*)result, fillBytes, fillBits);
    unsigned gb = (unsigned)((n + 255) / 256);
    scatter_init_keys<<<gb, 256, 0, st>>>(indices, d->index_bytes, n, d->operandRows, keys0, vals0);
  }
  // few keys: few sorting workgroups, so that the single-workgroup scan over their histograms stays short
  int sortBlocks = (int)((n + 2047) / 2048);
  sortBlocks = sortBlocks < 1 ? 1 : (sortBlocks > kSortBlocks ? kSortBlocks : sortBlocks);
  for (int shift = 0; shift < bits; shift += 8) {
    radix_hist<<<sortBlocks, 256, 0, st>>>(kin, n, shift, counts);
    radix_scan<<<1, 256, 0, st>>>(counts, sortBlocks);
    radix_scatter<<<sortBlocks, 256, 0, st>>>(kin, vin, n, shift, counts, kout, vout);
    u32* t = kin; kin = kout; kout = t;
    t = vin; vin = vout; vout = t;
  }
  dim3 gridShort((unsigned)n, (unsigned)((d->rowElems + 255) / 256));
  const long long chunksShort = (d->rowElems + 255) / 256, blocksRuns = blocksLong + n * chunksShort;
  // (measured on 8192 Zipf-distributed updates of 768 columns: 26 us together against 11.7 + 11.6 us apart, so one launch is
  // kept for callers that ask for it)
  static const bool oneLaunch = getenv("MI355X_SCATTER_ONE_FOLD") && getenv("MI355X_SCATTER_ONE_FOLD")[0] == '1';
  const bool together = oneLaunch && n >= kLongSegment && blocksRuns <= 0x7FFFFFFFll;
#define FOLD(P) do { \
    if (n >= kHugeSegment) scatter_fold_huge<P><<<(unsigned)blocksHuge, 256, 0, st>>>(kin, vin, n, d->rowElems, d->kind, (typename P::S*)result, (const typename P::S*)updates, (u32)d->operandRows, (u32)chunksHuge); \
    if (together) { \
      scatter_fold_runs<P><<<(unsigned)blocksRuns, 256, 0, st>>>(kin, vin, n, d->rowElems, d->kind, (typename P::S*)result, (const typename P::S*)updates, (u32)d->operandRows, (u32)chunksLong, (u32)blocksLong, (u32)chunksShort); \
    } else { \
      if (n >= kLongSegment) scatter_fold_long<P><<<(unsigned)blocksLong, 256, 0, st>>>(kin, vin, n, d->rowElems, d->kind, (typename P::S*)result, (const typename P::S*)updates, (u32)d->operandRows, (u32)chunksLong); \
      scatter_fold_short<P><<<gridShort, 256, 0, st>>>(kin, vin, n, d->rowElems, d->kind, (typename P::S*)result, (const typename P::S*)updates, (u32)d->operandRows); \
    } \
  } while (0)
  if (d->dtype == 0) FOLD(Plain<float>);
  else if (d->dtype == 2) FOLD(Plain<int>);
  else if (d->dtype == 3) FOLD(Plain<u32>);
  else FOLD(Bf16);
#undef FOLD
  return check("scatter_rows");
}

}  // extern "C"

// ---- ordered row scatter for callers that cannot allocate (include/mi355x_noalloc.h) --------------------
// The sort workspace is a device array of the library instead of a caller / arena buffer.  Host code may not
// pass the array's name to a kernel (on the host it is a stand-in, not a device address): the address is taken
// once per device with hipGetSymbolAddress and only that pointer is used afterwards.
#include <mutex>

#include "../../include/mi355x_noalloc.h"

static_assert(sizeof(mi355x_scatter_desc) == sizeof(mi355_scatter_desc), "public and internal scatter descriptors must agree");
static_assert(offsetof(mi355x_scatter_desc, index_bytes) == offsetof(mi355_scatter_desc, index_bytes), "descriptor layout");

namespace {
constexpr size_t kNoAllocScratchBytes = (size_t)4 * MI355X_NOALLOC_MAX_UPDATES * 4 + 256 * kSortBlocks * 4 + 1024;
constexpr int kMaxDevices = 64;
std::mutex g_scratchMutex;
void* g_scratchPtr[kMaxDevices] = {};
}  // namespace

static __device__ __align__(256) unsigned char scratch[kNoAllocScratchBytes];

// Device address of `scratch` on the current device (each GPU holds its own copy at its own address).
static int noallocScratch(void** out, char* error, size_t error_len) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e == hipSuccess && (dev < 0 || dev >= kMaxDevices)) e = hipErrorInvalidDevice;
  if (e == hipSuccess) {
    std::lock_guard<std::mutex> lock(g_scratchMutex);
    if (!g_scratchPtr[dev]) {
      void* p = nullptr;
      e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
      if (e == hipSuccess && !p) e = hipErrorInvalidSymbol;
      if (e == hipSuccess) g_scratchPtr[dev] = p;
    }
    if (e == hipSuccess) *out = g_scratchPtr[dev];
  }
  if (e != hipSuccess) {
    if (error && error_len) snprintf(error, error_len, "mi355x_scatter_rows_noalloc: cannot resolve the workspace on device %d: %s", dev, hipGetErrorString(e));
    return 1000 + (int)e;
  }
  return 0;
}

extern "C" {

// called when a PJRT client takes a device, so that the first scatter call finds the address resolved
int mi355_noalloc_setup(void) {
  void* p = nullptr;
  return noallocScratch(&p, nullptr, 0);
}

__attribute__((visibility("default")))
int mi355x_scatter_rows_noalloc(const mi355x_scatter_desc* desc, void* result, const void* indices, const void* updates,
                                void* hip_stream, char* error, size_t error_len) {
  auto fail = [&](int code, const char* msg) {
    if (error && error_len) snprintf(error, error_len, "mi355x_scatter_rows_noalloc: %s", msg);
    return code;
  };
  if (!desc) return fail(1, "desc is NULL");
  if (desc->num_updates < 0 || desc->row_elems < 0 || desc->operand_rows < 0) return fail(1, "negative size in desc");
  if (desc->num_updates > MI355X_NOALLOC_MAX_UPDATES) {
    if (error && error_len)
      snprintf(error, error_len, "mi355x_scatter_rows_noalloc: num_updates %lld exceeds the fixed workspace (MI355X_NOALLOC_MAX_UPDATES = %d)",
               (long long)desc->num_updates, MI355X_NOALLOC_MAX_UPDATES);
    return 2;
  }
  if (desc->kind < 0 || desc->kind > 4) return fail(1, "kind must be 0 (add), 1 (set), 2 (multiply), 3 (minimum) or 4 (maximum)");
  if (desc->dtype < 0 || desc->dtype > 3) return fail(1, "dtype must be 0 (f32), 1 (bf16), 2 (s32) or 3 (u32)");
  if (desc->index_bytes != 4 && desc->index_bytes != 8) return fail(1, "index_bytes must be 4 or 8");
  if (desc->operand_rows > 0xFFFFFFFEll) return fail(1, "operand_rows must fit 32 bits");
  if (desc->num_updates == 0 || desc->row_elems == 0 || desc->operand_rows == 0) return 0;
  if (!result || !indices || !updates) return fail(1, "result, indices and updates must be device pointers");
  void* ws = nullptr;
  if (int rc = noallocScratch(&ws, error, error_len)) return rc;
  mi355_scatter_desc d;
  d.numUpdates = desc->num_updates;
  d.rowElems = desc->row_elems;
  d.operandRows = desc->operand_rows;
  d.kind = desc->kind;
  d.dtype = desc->dtype;
  d.index_bytes = desc->index_bytes;
  int rc = mi355_scatter_rows(&d, result, indices, updates, ws, (mi355_stream_t)hip_stream);
  if (rc == MI355_SCATTER_GRID_TOO_LARGE)      // found before any launch
    return fail(3, "row_elems x num_updates needs more workgroups than one launch holds (row_elems above 16 776 960, or a fold grid above 2^31 - 1)");
  if (rc != 0 && error && error_len) snprintf(error, error_len, "mi355x_scatter_rows_noalloc: kernel launch failed: %s", hipGetErrorString((hipError_t)rc));
  return rc == 0 ? 0 : 1000 + rc;
}

}  // extern "C"
