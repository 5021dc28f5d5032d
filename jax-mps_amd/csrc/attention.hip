// Fused scaled-dot-product attention for bf16 operands: softmax(scale * Q K^T [masked]) V in one
// launch, the logits and probabilities never leave registers.
//
// Replaces, for the shapes that qualify, the chain dot_general -> scale -> mask select -> softmax ->
// convert -> dot_general (-> head-merging transpose) that the reference runs as separate mlx ops, or
// as mlx::fast::scaled_dot_product_attention behind its mps.sdpa custom call
// (src/pjrt_plugin/ops/control_flow.cc:1484-1533).
//
// One workgroup = one (batch, head) and 128 query rows, one wavefront = 32 query rows.  Keys are
// visited in blocks of 32 with a running maximum and sum per query (online softmax), so any number
// of keys works.  Per block and wavefront:
//   S^T[key][query]  = K_blk . Q^T      4 (H = 64) MFMA 32x32x16; K rows from LDS (ds_read_b128), Q fragments held
//                                       in registers
//   scale, mask, running max / sum      a query is one accumulator column: its 32 scores sit in 16
//                                       registers of two lanes (l and l ^ 32), so the row reductions are
//                                       15 register ops and one cross-lane exchange
//   O^T[h][query]   += V_blk^T . P^T    P^T is the accumulator itself: registers 8n .. 8n+7 of a lane are
//                                       the lane's B operand of product n once the 16 keys of that product
//                                       are numbered accordingly, and V^T is read with that same numbering
//                                       from LDS by transposing reads (ds_read_b64_tr_b16).
// K and V of the (batch, head) are staged once in LDS ([key][h] rows, 16-byte slots XOR-swizzled by the row so that
// the 16 rows of a K operand read and the four rows of a transposing V read fall into different banks): after the
// one cooperative load the key loop touches memory only for mask bytes.
#include <hip/hip_runtime.h>

#include <cstdint>

#include "hip_abi.h"

namespace {

typedef unsigned short u16;
typedef unsigned int u32;
typedef float float16v __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef short short4v __attribute__((ext_vector_type(4)));
typedef short short8v __attribute__((ext_vector_type(8)));

struct AttnArgs {
  const u16* q;
  const u16* k;
  const u16* v;
  const unsigned char* mask;   // i1 as bytes, or null
  u16* out;
  long long qB, qN, qT, kB, kN, kS, vB, vN, vS, oB, oN, oT, mB, mN, mT, mS;
  int T, S;
  int maskWords;               // mask rows are contiguous and 4-byte aligned: four keys per load
  float scale, masked;         // score of a masked-out position
};

__device__ __forceinline__ u16 to_bf16(float f) { return __builtin_bit_cast(u16, (__bf16)f); }

template <int H>
__device__ __forceinline__ int swzV(int row) { return H == 64 ? ((row >> 1) & 1) << 2 : (row & 3) << 2; }
template <int H>
__device__ __forceinline__ int swzK(int row) { return H == 64 ? (row >> 1) & 7 : row & 15; }

template <int H>
__global__ void __launch_bounds__(256) attention_bf16(AttnArgs g) {
  constexpr int HC = H / 16;       // 16-wide chunks of the head dim (QK^T products per key block)
  constexpr int HT = H / 32;       // 32-wide tiles of the head dim (output accumulators)
  constexpr int SLOTS = H / 8;     // 16-byte slots per V row
  extern __shared__ __attribute__((aligned(16))) unsigned char vlds[];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int b = blockIdx.z, n = blockIdx.y;
  const int q0 = blockIdx.x * 128 + wave * 32;
  const int keyBlocks = (g.S + 31) / 32;

  // Q fragments and the first mask bytes are requested before K and V are staged, so the latencies overlap
  const int col = lane & 31, half = lane >> 5;
  int query = q0 + col;
  const bool queryOk = query < g.T;
  if (query > g.T - 1) query = g.T - 1;
  const u16* Q = g.q + (long long)b * g.qB + (long long)n * g.qN + (long long)query * g.qT;
  bf16x8 qf[HC];
#pragma unroll
  for (int c = 0; c < HC; ++c) qf[c] = *(const bf16x8*)(Q + c * 16 + half * 8);
  const unsigned char* M = g.mask ? g.mask + (long long)b * g.mB + (long long)n * g.mN + (long long)query * g.mT : nullptr;
  // the 16 mask bytes of a key block (four runs of four consecutive keys) are requested one block ahead; as four
  // 32-bit words when the mask rows allow it
  auto loadMask = [&](int kb, u32 (&mk)[4]) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      int key = kb * 32 + j * 8 + half * 4;
      if (g.maskWords) {
        if (key > g.S - 4) key = g.S - 4;
        mk[j] = *(const u32*)(M + key);
      } else {
        u32 w = 0;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          int ki = key + i;
          if (ki > g.S - 1) ki = g.S - 1;
          w |= (u32)(M[(long long)ki * g.mS] != 0) << (8 * i);
        }
        mk[j] = w;
      }
    }
  };
  u32 mkA[4] = {}, mkB[4] = {};
  if (M) loadMask(0, mkA);
  // ---- K and V of this (batch, head) into LDS, rows past S zero
  const int rows = keyBlocks * 32;
  unsigned char* klds = vlds + rows * (H * 2);
  const u16* K = g.k + (long long)b * g.kB + (long long)n * g.kN;
  const u16* V = g.v + (long long)b * g.vB + (long long)n * g.vN;
#pragma unroll 4
  for (int i = tid; i < rows * SLOTS; i += 256) {
    const int row = i / SLOTS, slot = i % SLOTS;
    uint4 kv = make_uint4(0, 0, 0, 0), vv = make_uint4(0, 0, 0, 0);
    if (row < g.S) {
      kv = *(const uint4*)(K + (long long)row * g.kS + slot * 8);
      vv = *(const uint4*)(V + (long long)row * g.vS + slot * 8);
    }
    *(uint4*)(klds + row * (H * 2) + ((slot ^ swzK<H>(row)) << 4)) = kv;
    *(uint4*)(vlds + row * (H * 2) + ((slot ^ swzV<H>(row)) << 4)) = vv;
  }
  __syncthreads();
  if (q0 >= g.T) return;


  float16v o[HT];
#pragma unroll
  for (int t = 0; t < HT; ++t)
#pragma unroll
    for (int e = 0; e < 16; ++e) o[t][e] = 0.f;
  float mRun = -__builtin_inff(), lRun = 0.f;

  // The loop is bound by vector ALU work, so everything that does not depend on the key block is hoisted:
  // per-lane LDS offsets of the K operand reads and of the transposing V reads (lane d of a 16-lane group
  // addresses key row d >> 2 of a group of four and the 4 head columns 4 * (d & 3) .. + 3 of the group's 16; the
  // swizzle terms only depend on the lane because block and product offsets are multiples of 16 rows), and
  // the exponentials run in base 2 with log2(e) folded into the scale.
  const int d = lane & 15, nhalf = (lane >> 4) & 1;
  int kOff[HC], vOff[HT];
#pragma unroll
  for (int c = 0; c < HC; ++c) kOff[c] = col * (H * 2) + (((c * 2 + half) ^ swzK<H>(col)) << 4);
#pragma unroll
  for (int t = 0; t < HT; ++t) {
    const int row = 4 * half + (d >> 2);
    const int slot = ((t * 32 + nhalf * 16) >> 3) + ((d & 3) >> 1);
    vOff[t] = row * (H * 2) + ((slot ^ swzV<H>(row)) << 4) + ((d & 1) << 3);
  }
  constexpr float kLog2e = 1.44269504088896340736f;
  const float scale2 = g.scale * kLog2e;
  const float masked2 = fmaxf(g.masked * kLog2e, -3.4028234663852886e38f);   // stays finite: a fully masked row is uniform
  const bool ragged = (g.S & 31) != 0;

  auto block = [&](int kb, u32 (&mk)[4], u32 (&mkNext)[4]) {
    if (M && kb + 1 < keyBlocks) loadMask(kb + 1, mkNext);
    const unsigned char* kblk = klds + kb * (32 * H * 2);
    const unsigned char* vblk = vlds + kb * (32 * H * 2);
    // ---- S^T = K_blk . Q^T
    float16v s;
#pragma unroll
    for (int e = 0; e < 16; ++e) s[e] = 0.f;
#pragma unroll
    for (int c = 0; c < HC; ++c) s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(*(const bf16x8*)(kblk + kOff[c]), qf[c], s, 0, 0, 0);
    // ---- scale, mask, block maximum
#pragma unroll
    for (int e = 0; e < 16; ++e) s[e] *= scale2;
    if (M) {
#pragma unroll
      for (int e = 0; e < 16; ++e) s[e] = ((mk[e >> 2] >> (8 * (e & 3))) & 0xFFu) ? s[e] : masked2;
    }
    if (ragged && kb == keyBlocks - 1) {
#pragma unroll
      for (int e = 0; e < 16; ++e)
        if (kb * 32 + (e >> 2) * 8 + half * 4 + (e & 3) >= g.S) s[e] = -__builtin_inff();
    }
    float mBlk = s[0];
#pragma unroll
    for (int e = 1; e < 16; ++e) mBlk = fmaxf(mBlk, s[e]);
    mBlk = fmaxf(mBlk, __shfl_xor(mBlk, 32));
    const float mNew = fmaxf(mRun, mBlk);
    const float alpha = __builtin_amdgcn_exp2f(mRun - mNew);
    float lBlk = 0.f;
#pragma unroll
    for (int e = 0; e < 16; ++e) {
      s[e] = __builtin_amdgcn_exp2f(s[e] - mNew);
      lBlk += s[e];
    }
    lBlk += __shfl_xor(lBlk, 32);
    lRun = lRun * alpha + lBlk;
    mRun = mNew;
    if (kb > 0) {
#pragma unroll
      for (int t = 0; t < HT; ++t)
#pragma unroll
        for (int e = 0; e < 16; ++e) o[t][e] *= alpha;
    }
    // ---- O^T += V_blk^T . P^T: product nn covers the keys 16nn + 8(r / 4) + 4 half + r % 4 (r = 0..7 of a lane)
#pragma unroll
    for (int nn = 0; nn < 2; ++nn) {
      bf16x8 pf;
#pragma unroll
      for (int r = 0; r < 8; ++r) pf[r] = (__bf16)s[8 * nn + r];
#pragma unroll
      for (int t = 0; t < HT; ++t) {
        short4v hv[2];
#pragma unroll
        for (int qq = 0; qq < 2; ++qq)
          hv[qq] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) short4v*)(vblk + vOff[t] + (16 * nn + 8 * qq) * (H * 2)));
        const short8v both = __builtin_shufflevector(hv[0], hv[1], 0, 1, 2, 3, 4, 5, 6, 7);
        o[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, both), pf, o[t], 0, 0, 0);
      }
    }
  };
  for (int kb = 0; kb < keyBlocks; kb += 2) {
    block(kb, mkA, mkB);
    if (kb + 1 < keyBlocks) block(kb + 1, mkB, mkA);
  }
  if (!queryOk) return;
  const float inv = 1.f / lRun;
  u16* O = g.out + (long long)b * g.oB + (long long)n * g.oN + (long long)(q0 + col) * g.oT;
#pragma unroll
  for (int t = 0; t < HT; ++t)
#pragma unroll
    for (int e4 = 0; e4 < 4; ++e4) {
      const int h = t * 32 + e4 * 8 + half * 4;
      uint2 w;
      w.x = (u32)to_bf16(o[t][e4 * 4 + 0] * inv) | ((u32)to_bf16(o[t][e4 * 4 + 1] * inv) << 16);
      w.y = (u32)to_bf16(o[t][e4 * 4 + 2] * inv) | ((u32)to_bf16(o[t][e4 * 4 + 3] * inv) << 16);
      *(uint2*)(O + h) = w;
    }
}

template <int H>
int launch(const AttnArgs& g, const mi355_attention_desc* d, hipStream_t st) {
  const int bytes = ((d->S + 31) / 32) * 32 * H * 4;   // K and V
  static bool configured = false;
  if (!configured) {
    if (hipFuncSetAttribute((const void*)attention_bf16<H>, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024) != hipSuccess) return 3;
    configured = true;
  }
  dim3 grid((unsigned)((d->T + 127) / 128), (unsigned)d->N, (unsigned)d->B);
  attention_bf16<H><<<grid, 256, bytes, st>>>(g);
  return hipGetLastError() == hipSuccess ? 0 : 3;
}

}  // namespace

extern "C" int mi355_attention_supported(const mi355_attention_desc* d) {
  if (d->H != 64 && d->H != 128) return 0;
  if (d->B <= 0 || d->N <= 0 || d->T <= 0 || d->S <= 0 || d->B > 65535 || d->N > 65535) return 0;
  if ((long long)((d->S + 31) / 32) * 32 * d->H * 4 > 128 * 1024) return 0;   // K and V of one head must fit LDS
  // 16-byte loads of head rows, 8-byte stores of the result
  const long long strides[] = {d->qB, d->qN, d->qT, d->kB, d->kN, d->kS, d->vB, d->vN, d->vS};
  for (long long s : strides) if (s % 8 != 0) return 0;
  if (d->oB % 4 != 0 || d->oN % 4 != 0 || d->oT % 4 != 0) return 0;
  return 1;
}

// 0 = launched, -1 = shape or layout does not qualify, other = launch error.
extern "C" int mi355_attention(const mi355_attention_desc* d, const void* q, const void* k, const void* v, const void* mask, void* out,
                               mi355_stream_t s) {
  if (!mi355_attention_supported(d)) return -1;
  if ((((uintptr_t)q | (uintptr_t)k | (uintptr_t)v) & 15) != 0 || ((uintptr_t)out & 7) != 0) return -1;
  AttnArgs g;
  g.q = (const u16*)q; g.k = (const u16*)k; g.v = (const u16*)v; g.mask = (const unsigned char*)mask; g.out = (u16*)out;
  g.qB = d->qB; g.qN = d->qN; g.qT = d->qT;
  g.kB = d->kB; g.kN = d->kN; g.kS = d->kS;
  g.vB = d->vB; g.vN = d->vN; g.vS = d->vS;
  g.oB = d->oB; g.oN = d->oN; g.oT = d->oT;
  g.mB = d->mB; g.mN = d->mN; g.mT = d->mT; g.mS = d->mS;
  g.T = (int)d->T; g.S = (int)d->S;
  g.scale = d->scale; g.masked = d->masked;
  g.maskWords = mask && d->mS == 1 && d->S % 4 == 0 && d->mB % 4 == 0 && d->mN % 4 == 0 && d->mT % 4 == 0 && ((uintptr_t)mask & 3) == 0;
  if (d->H == 64) return launch<64>(g, d, (hipStream_t)s);
  return launch<128>(g, d, (hipStream_t)s);
}
