// Thin C-ABI layer between the host runtime (plain C++) and HIP.  Only
// hip_abi.hip and kernels.hip include HIP headers; everything above talks to the
// GPU through these functions.  All functions return 0 on success or a HIP error
// code; mi355_last_error() describes the most recent failure of the calling thread.
#pragma once

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void* mi355_stream_t;
typedef void* mi355_event_t;
typedef void* mi355_function_t;

const char* mi355_last_error(void);

// device
int mi355_device_count(int* count);
int mi355_device_init(int device, char* name, size_t name_len, char* arch, size_t arch_len, int* compute_units,
                      size_t* total_mem);
int mi355_mem_info(size_t* free_bytes, size_t* total_bytes);

// memory
int mi355_malloc(void** ptr, size_t bytes);
int mi355_free(void* ptr);
int mi355_host_alloc(void** ptr, size_t bytes);   // pinned
int mi355_host_free(void* ptr);
int mi355_memcpy_h2d(void* dst, const void* src, size_t bytes, mi355_stream_t s);
int mi355_memcpy_d2h(void* dst, const void* src, size_t bytes, mi355_stream_t s);
int mi355_memcpy_d2d(void* dst, const void* src, size_t bytes, mi355_stream_t s);

// streams and events (default priority only)
int mi355_stream_create(mi355_stream_t* s);
int mi355_stream_destroy(mi355_stream_t s);
int mi355_stream_sync(mi355_stream_t s);
int mi355_event_create(mi355_event_t* e, int timing);
int mi355_event_destroy(mi355_event_t e);
int mi355_event_record(mi355_event_t e, mi355_stream_t s);
int mi355_stream_wait_event(mi355_stream_t s, mi355_event_t e);   // work enqueued on s after this call waits for what e recorded
int mi355_event_sync(mi355_event_t e);
int mi355_event_query(mi355_event_t e, int* ready);
int mi355_event_elapsed_ms(mi355_event_t a, mi355_event_t b, float* ms);

// Stream capture into an executable graph: work enqueued on `s` between begin and end is recorded,
// not run; mi355_graph_launch replays it.  Used for the bodies of counted loops.
typedef void* mi355_graph_t;
int mi355_capture_begin(mi355_stream_t s);
int mi355_capture_end(mi355_stream_t s, mi355_graph_t* exec, int* num_nodes);
int mi355_graph_launch(mi355_graph_t exec, mi355_stream_t s);
int mi355_graph_destroy(mi355_graph_t exec);

// runtime-compiled kernels: `source` defines extern "C" __global__ void k(...).
// mi355_rtc_compile is thread-safe (no device state); the code object it returns is
// malloc'ed and handed to mi355_module_load, which must run on the thread that owns the device.
// identifies the compiler build and the options mi355_rtc_compile uses (part of the on-disk cache key)
const char* mi355_rtc_fingerprint(void);
int mi355_rtc_compile(const char* source, const char* arch, char** code, size_t* code_size, char* log, size_t log_len);
int mi355_module_load(const char* code, mi355_function_t* fn);
int mi355_launch(mi355_function_t fn, const unsigned grid[3], const unsigned block[3], void** arg_ptrs, int num_args,
                 mi355_stream_t s);

// ahead-of-time kernels (kernels.hip).  dtype codes: 0 f32, 1 bf16, 2 s32, 3 u32.
typedef struct {
  int64_t batch0, batch1, M, N, K;
  int64_t aB0, aB1, aRow, aCol;
  int64_t bB0, bB1, bRow, bCol;
  int in_dtype, out_dtype;
  // act 1 (bf16 results only): after the bias, y = act_a * x * (1 + tanh(act_c * (x + act_b * x^3))) on the stored
  // (rounded) value x, computed in fp32 and rounded again: the tanh form of GELU with the program's own constants;
  // act 2 (small fp32 products only, mi355_gemm_is_small): y = maximum(x, 0)
  int act;
  float act_a, act_b, act_c;
} mi355_gemm_desc;
// `workspace` (may be NULL) holds k-contiguous copies of bf16 operands; see mi355_gemm_workspace_bytes.
// `bias` (may be NULL): N values of the output type added to every row of C after the product has been rounded to
// the output type, i.e. exactly dot_general followed by add(broadcast(bias)).
int mi355_gemm(const mi355_gemm_desc* d, const void* a, const void* b, void* c, const void* bias, void* workspace,
               size_t workspace_bytes, mi355_stream_t s);
size_t mi355_gemm_workspace_bytes(const mi355_gemm_desc* d);
// Small fp32 products (mi355_gemm_is_small) run as one launch without workspace; two of them with the same
// result shape can be summed by the same launch: C = A1 x B1 + A2 x B2 (+ addend) (+ bias).  d2 may be NULL; addend, a
// tensor laid out like C (it may not be C itself), may be NULL.  -1 = not small.
int mi355_gemm_is_small(const mi355_gemm_desc* d);   // 0, or the tile edge (16 / 32) the small-product kernel uses
// n <= 4 independent small products of one tile class in one launch; d2[i] may be NULL.  -1 = the group does not qualify.
int mi355_gemm_small_group(int n, const mi355_gemm_desc* const* d1, const void* const* a1, const void* const* b1,
                           const mi355_gemm_desc* const* d2, const void* const* a2, const void* const* b2, void* const* c,
                           const void* const* bias, const void* const* addend, mi355_stream_t s);
int mi355_gemm_small_sum(const mi355_gemm_desc* d1, const void* a1, const void* b1, const mi355_gemm_desc* d2, const void* a2,
                         const void* b2, void* c, const void* bias, const void* addend, mi355_stream_t s);
// bf16 operands with 16-byte-loadable layouts on 128x128 / 128x64 / 64x64 tiles; -1 = layout does not qualify
// bf16, both operands k-contiguous, K % 64 == 0: LDS ring filled by direct global->LDS loads
int mi355_gemm_bf16_async(const mi355_gemm_desc* d, const void* a, const void* b, void* c, const void* bias, void* workspace,
                          size_t workspace_bytes, mi355_stream_t s);
size_t mi355_gemm_bf16_async_workspace_bytes(const mi355_gemm_desc* d);
int mi355_gemm_bf16_tiled(const mi355_gemm_desc* d, const void* a, const void* b, void* c, mi355_stream_t s);

// softmax(scale * Q K^T, masked positions replaced by `masked`) V for bf16 tensors addressed through element strides
// (head dim contiguous): q[b, n, t, :H], k[b, n, s, :H], v[b, n, s, :H], out[b, n, t, :H]; mask (may be NULL) is one byte
// per position addressed by mB / mN / mT / mS (0 = broadcast), non-zero = keep.
typedef struct {
  int64_t B, N, T, S, H;
  int64_t qB, qN, qT, kB, kN, kS, vB, vN, vS, oB, oN, oT, mB, mN, mT, mS;
  float scale, masked;
} mi355_attention_desc;
int mi355_attention_supported(const mi355_attention_desc* d);
int mi355_attention(const mi355_attention_desc* d, const void* q, const void* k, const void* v, const void* mask, void* out,
                    mi355_stream_t s);

typedef struct {
  int nsp;
  int64_t N, C, O;
  int64_t in[3], k[3], out[3], stride[3], padLo[3], ldil[3], rdil[3], rev[3];
  int64_t featureGroups, batchGroups;
  int64_t lhsB, lhsF, lhsS[3], rhsI, rhsO, rhsS[3], outB, outF, outS[3];
  int dtype;
} mi355_conv_desc;
// `workspace` (may be NULL) is scratch for split-K partial sums; see mi355_conv_workspace_bytes.
int mi355_conv(const mi355_conv_desc* d, const void* lhs, const void* rhs, void* out, void* workspace,
               size_t workspace_bytes, mi355_stream_t s);
size_t mi355_conv_workspace_bytes(const mi355_conv_desc* d);
// Column statistics next to the output: mi355_conv_stats_rows(d) > 0 says the convolution can deliver, for each of that
// many tile rows i and every output feature n, the sum and the sum of squares of its rows' outputs (stat_sum[i * O + n],
// stat_sq[i * O + n], both rows x O floats); folding the tile rows in order gives the statistics of the whole output.
int mi355_conv_stats_rows(const mi355_conv_desc* d);
int mi355_conv_stats(const mi355_conv_desc* d, const void* lhs, const void* rhs, void* out, void* workspace, size_t workspace_bytes,
                     float* stat_sum, float* stat_sq, mi355_stream_t s);
int mi355_conv_direct(const mi355_conv_desc* d, const void* lhs, const void* rhs, void* out, mi355_stream_t s);

typedef struct {
  int64_t numUpdates, rowElems, operandRows;
  int kind;        // 0 add, 1 set, 2 mul, 3 min, 4 max
  int dtype;       // element type code
  int index_bytes; // 4 or 8
} mi355_scatter_desc;
// Deterministic row scatter: updates are applied to each destination row in the order they
// appear in `indices` (stable sort by row, then one pass per row segment).  `result` already
// holds the operand.  `workspace` needs mi355_scatter_workspace_bytes(numUpdates) bytes.
// returned (before anything is enqueued) when a fold launch would need more workgroups than a grid holds; negative so
// that it cannot be mistaken for a HIP error code
#define MI355_SCATTER_GRID_TOO_LARGE (-3)
int mi355_scatter_rows(const mi355_scatter_desc* d, void* result, const void* indices, const void* updates,
                       void* workspace, mi355_stream_t s);
// The same with the operand given as a splat: when `fill` is set, `result` need not hold anything on entry and every
// element starts as `fill_bits` (the element's bit pattern; 16-bit types in the low half).  The fill shares a launch
// with the sort, which keeps one CU busy while the others write.
int mi355_scatter_rows_fill(const mi355_scatter_desc* d, void* result, const void* indices, const void* updates,
                            void* workspace, int fill, uint32_t fill_bits, mi355_stream_t s);
size_t mi355_scatter_workspace_bytes(int64_t num_updates);
// resolves, for the current device, the library-owned workspace of mi355x_scatter_rows_noalloc (include/mi355x_noalloc.h)
int mi355_noalloc_setup(void);

int mi355_copy(void* dst, const void* src, size_t bytes, mi355_stream_t s);   // kernel copy (graph-capturable)
// up to 16 copies between pairwise disjoint buffers in one launch
int mi355_copy_multi(int n, void* const* dst, const void* const* src, const size_t* bytes, mi355_stream_t s);
// The same under a condition the kernel reads from device memory, so that control flow needs no host round trip:
// mode 1 copies when the int at `flag` is non-zero (commit of a loop iteration while the loop is alive); mode 2 copies
// when the branch index at `flag` (index_bytes wide, 0 = one-byte predicate; out of range selects branch count-1,
// reference: ops/control_flow.cc:672-675) equals `want`.  cond == NULL copies unconditionally.
typedef struct {
  const void* flag;
  int mode, index_bytes;
  long long want, count;
} mi355_copy_cond;
int mi355_copy_multi_if(int n, void* const* dst, const void* const* src, const size_t* bytes, const mi355_copy_cond* cond, mi355_stream_t s);
// loop flag (two ints: alive, iterations run while alive): init sets alive to *parent (the enclosing loop's flag) or 1 and
// the count to 0; and folds a one-byte predicate into alive and adds the result to the count
int mi355_flag_init(void* flag, const void* parent, mi355_stream_t s);
int mi355_flag_and(void* flag, const void* pred, mi355_stream_t s);

#ifdef __cplusplus
}
#endif
