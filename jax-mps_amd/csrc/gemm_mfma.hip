// Tiled bf16 GEMM on the gfx950 matrix cores (v_mfma_f32_32x32x16_bf16, fp32 accumulation).
//
// Replaces the reference's dot_general lowering to mlx einsum/matmul
// (src/pjrt_plugin/ops/linalg.cc:89-250) for 16-bit operands whose layouts allow 16-byte
// global loads; every other layout stays on the strided kernel in kernels.hip.
//
// Workgroup = 4 wavefronts (2x2) over a BMxBN tile of C, K walked in slabs of 64.  Both
// operands sit in LDS k-minor ([row][k], padded), which is the order the MFMA wants: lane
// l supplies row l%32 and the eight consecutive k starting at 8*(l/32), one ds_read_b128.
// An operand that is k-contiguous in HBM goes to LDS with plain 16-byte copies; one that
// is contiguous along m (or n) is read as 4(k) x 8(row) register blocks, transposed in
// registers and written as 8-byte pieces.  The next slab is fetched into registers while
// the current one is multiplied.  Workgroup ids are remapped so that the eight XCDs (which
// receive consecutive ids round-robin) each work on a contiguous band of tiles and share
// operand rows through their own L2.
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

struct TiledArgs {
  const u16* a;
  const u16* b;
  void* c;
  long long M, N, K;
  long long aB0, aB1, aLd, bB0, bB1, bLd;   // batch strides and leading dimension (elements)
  int batch1;
  int outBf16;
  int tilesM, tilesN;
  long long total;   // workgroups
};

constexpr int BK = 64;
constexpr int LDK = BK + 8;   // LDS row pitch in elements (144 B keeps 16-byte alignment, spreads banks)

__device__ __forceinline__ u16 to_bf16(float f) { return __builtin_bit_cast(u16, (__bf16)f); }

// One operand tile (ROWS x BK) on its way from HBM to LDS.
template <int ROWS, bool TRANS>
struct TileLoader {
  // direct: ROWS*8 vectors of 8 k; transposed: (BK/4)*(ROWS/8) blocks of 4 k x 8 rows
  static constexpr int kUnits = TRANS ? (BK / 4) * (ROWS / 8) : ROWS * 8;
  static constexpr int kPerThread = (kUnits + 255) / 256;
  static constexpr int kRegs = TRANS ? kPerThread * 4 : kPerThread;
  uint4 r[kRegs];

  __device__ __forceinline__ void fetch(const u16* __restrict__ base, long long ld, long long row0, long long rows, long long k0, long long K, int tid) {
#pragma unroll
    for (int i = 0; i < kPerThread; ++i) {
      const int u = tid + 256 * i;
      if (!TRANS) {
        const int row = u >> 3, kv = u & 7;
        const long long gr = row0 + row, gk = k0 + kv * 8;
        r[i] = (gr < rows && gk < K) ? *(const uint4*)(base + gr * ld + gk) : make_uint4(0, 0, 0, 0);
      } else {
        const int kb = u / (ROWS / 8), rb = u % (ROWS / 8);
        const long long gr = row0 + rb * 8;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const long long gk = k0 + kb * 4 + q;
          r[i * 4 + q] = (u < kUnits && gr < rows && gk < K) ? *(const uint4*)(base + gk * ld + gr) : make_uint4(0, 0, 0, 0);
        }
      }
    }
  }

  __device__ __forceinline__ void stash(u16* __restrict__ lds, int tid) const {
#pragma unroll
    for (int i = 0; i < kPerThread; ++i) {
      const int u = tid + 256 * i;
      if (!TRANS) {
        const int row = u >> 3, kv = u & 7;
        *(uint4*)(lds + row * LDK + kv * 8) = r[i];
      } else {
        if (u >= kUnits) continue;
        const int kb = u / (ROWS / 8), rb = u % (ROWS / 8);
        const u32* q0 = (const u32*)&r[i * 4 + 0];
        const u32* q1 = (const u32*)&r[i * 4 + 1];
        const u32* q2 = (const u32*)&r[i * 4 + 2];
        const u32* q3 = (const u32*)&r[i * 4 + 3];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          // dword j of each k-row holds rows 2j (low half) and 2j+1 (high half)
          uint2 lo, hi;
          lo.x = (q0[j] & 0xFFFFu) | (q1[j] << 16);
          lo.y = (q2[j] & 0xFFFFu) | (q3[j] << 16);
          hi.x = (q0[j] >> 16) | (q1[j] & 0xFFFF0000u);
          hi.y = (q2[j] >> 16) | (q3[j] & 0xFFFF0000u);
          *(uint2*)(lds + (rb * 8 + 2 * j) * LDK + kb * 4) = lo;
          *(uint2*)(lds + (rb * 8 + 2 * j + 1) * LDK + kb * 4) = hi;
        }
      }
    }
  }
};

template <int BM, int BN, bool AT, bool BT>
__global__ void __launch_bounds__(256) gemm_bf16_tiled(TiledArgs g) {
  constexpr int TM = BM / 64, TN = BN / 64;   // 32x32 MFMA tiles per wavefront in each direction
  __shared__ __attribute__((aligned(16))) u16 As[BM * LDK];
  __shared__ __attribute__((aligned(16))) u16 Bs[BN * LDK];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;

  // XCD-aware id: consecutive hardware ids go to different XCDs; give each XCD a contiguous band
  long long id = blockIdx.x;
  if ((g.total & 7) == 0) id = (id & 7) * (g.total >> 3) + (id >> 3);
  const long long perBatch = (long long)g.tilesM * g.tilesN;
  const long long bz = id / perBatch;
  const int t = (int)(id % perBatch);
  const int tm = t / g.tilesN, tn = t % g.tilesN;
  const long long b0 = bz / g.batch1, b1 = bz % g.batch1;
  const u16* A = g.a + b0 * g.aB0 + b1 * g.aB1;
  const u16* B = g.b + b0 * g.bB0 + b1 * g.bB1;
  const long long m0 = (long long)tm * BM, n0 = (long long)tn * BN;

  float16v acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

  TileLoader<BM, AT> la;
  TileLoader<BN, BT> lb;
  la.fetch(A, g.aLd, m0, g.M, 0, g.K, tid);
  lb.fetch(B, g.bLd, n0, g.N, 0, g.K, tid);
  la.stash(As, tid);
  lb.stash(Bs, tid);
  __syncthreads();

  const u16* aFrag = As + (wm * (BM / 2) + (lane & 31)) * LDK + (lane >> 5) * 8;
  const u16* bFrag = Bs + (wn * (BN / 2) + (lane & 31)) * LDK + (lane >> 5) * 8;
  for (long long k0 = 0; k0 < g.K; k0 += BK) {
    const bool more = k0 + BK < g.K;
    if (more) {
      la.fetch(A, g.aLd, m0, g.M, k0 + BK, g.K, tid);
      lb.fetch(B, g.bLd, n0, g.N, k0 + BK, g.K, tid);
    }
#pragma unroll
    for (int kk = 0; kk < BK; kk += 16) {
      bf16x8 av[TM], bv[TN];
#pragma unroll
      for (int i = 0; i < TM; ++i) av[i] = *(const bf16x8*)(aFrag + i * 32 * LDK + kk);
#pragma unroll
      for (int j = 0; j < TN; ++j) bv[j] = *(const bf16x8*)(bFrag + j * 32 * LDK + kk);
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(av[i], bv[j], acc[i][j], 0, 0, 0);
    }
    __syncthreads();
    if (more) {
      la.stash(As, tid);
      lb.stash(Bs, tid);
      __syncthreads();
    }
  }

  // accumulator element e of lane l: row 8*(e/4) + 4*(l/32) + e%4, column l%32
  const long long cBase = bz * g.M * g.N;
#pragma unroll
  for (int i = 0; i < TM; ++i) {
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const long long col = n0 + wn * (BN / 2) + j * 32 + (lane & 31);
      if (col >= g.N) continue;
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const long long row = m0 + wm * (BM / 2) + i * 32 + (e >> 2) * 8 + (lane >> 5) * 4 + (e & 3);
        if (row >= g.M) continue;
        if (g.outBf16) ((u16*)g.c)[cBase + row * g.N + col] = to_bf16(acc[i][j][e]);
        else ((float*)g.c)[cBase + row * g.N + col] = acc[i][j][e];
      }
    }
  }
}

template <int BM, int BN>
void launchLayout(bool at, bool bt, const TiledArgs& g, hipStream_t st) {
  dim3 grid((unsigned)g.total);
  if (!at && !bt) gemm_bf16_tiled<BM, BN, false, false><<<grid, 256, 0, st>>>(g);
  else if (!at && bt) gemm_bf16_tiled<BM, BN, false, true><<<grid, 256, 0, st>>>(g);
  else if (at && !bt) gemm_bf16_tiled<BM, BN, true, false><<<grid, 256, 0, st>>>(g);
  else gemm_bf16_tiled<BM, BN, true, true><<<grid, 256, 0, st>>>(g);
}

bool aligned16(const void* p) { return ((uintptr_t)p & 15) == 0; }

}  // namespace

// Returns 0 when the tiled kernel took the job, -1 when the layout does not qualify (the
// caller then uses the strided kernel), another value on a launch error.
extern "C" int mi355_gemm_bf16_tiled(const mi355_gemm_desc* d, const void* a, const void* b, void* c, mi355_stream_t s) {
  if (d->in_dtype != 1 || (d->out_dtype != 0 && d->out_dtype != 1)) return -1;
  const long long nb = d->batch0 * d->batch1;
  if (d->M <= 0 || d->N <= 0 || d->K <= 0 || nb <= 0) return -1;
  // operand A: k-contiguous rows, or m-contiguous columns
  bool at, bt;
  long long aLd, bLd;
  if (d->aCol == 1 && d->aRow % 8 == 0 && d->K % 8 == 0) { at = false; aLd = d->aRow; }
  else if (d->aRow == 1 && d->aCol % 8 == 0 && d->M % 8 == 0) { at = true; aLd = d->aCol; }
  else return -1;
  // operand B (K x N through bRow/bCol): k-contiguous means bRow == 1
  if (d->bRow == 1 && d->bCol % 8 == 0 && d->K % 8 == 0) { bt = false; bLd = d->bCol; }
  else if (d->bCol == 1 && d->bRow % 8 == 0 && d->N % 8 == 0) { bt = true; bLd = d->bRow; }
  else return -1;
  if (!aligned16(a) || !aligned16(b)) return -1;
  if (d->batch0 > 1 && (d->aB0 % 8 || d->bB0 % 8)) return -1;
  if (d->batch1 > 1 && (d->aB1 % 8 || d->bB1 % 8)) return -1;

  TiledArgs g;
  g.a = (const u16*)a; g.b = (const u16*)b; g.c = c;
  g.M = d->M; g.N = d->N; g.K = d->K;
  g.aB0 = d->aB0; g.aB1 = d->aB1; g.aLd = aLd;
  g.bB0 = d->bB0; g.bB1 = d->bB1; g.bLd = bLd;
  g.batch1 = (int)d->batch1;
  g.outBf16 = d->out_dtype == 1;
  auto tiles = [&](int bm, int bn) { return ((d->M + bm - 1) / bm) * ((d->N + bn - 1) / bn) * nb; };
  int bm = 64, bn = 64;
  static const char* force = getenv("MI355X_GEMM_TILE");   // "256x128", "128x128", "128x64", "64x64": tuning aid
  if (force) { sscanf(force, "%dx%d", &bm, &bn); }
  else if (d->M > 128 && d->N > 64 && tiles(256, 128) >= 256) { bm = 256; bn = 128; }
  else if (d->M > 64 && d->N > 64 && tiles(128, 128) >= 512) { bm = 128; bn = 128; }
  else if (d->M > 64 && tiles(128, 64) >= 384) { bm = 128; bn = 64; }
  g.tilesM = (int)((d->M + bm - 1) / bm);
  g.tilesN = (int)((d->N + bn - 1) / bn);
  g.total = (long long)g.tilesM * g.tilesN * nb;
  if (g.total > 0x7FFFFFFFll) return -1;
  hipStream_t st = (hipStream_t)s;
  if (bm == 256) launchLayout<256, 128>(at, bt, g, st);
  else if (bm == 128 && bn == 128) launchLayout<128, 128>(at, bt, g, st);
  else if (bm == 128) launchLayout<128, 64>(at, bt, g, st);
  else launchLayout<64, 64>(at, bt, g, st);
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? 0 : 3;
}
