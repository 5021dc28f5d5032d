/* Entry points of libpjrt_plugin_mi355x.so beside GetPjrtApi (include/pjrt_c_api.h).
 *
 * mi355x_scatter_rows_noalloc has no counterpart in the reference.  It exists for callers that cannot
 * allocate device memory: code under HIP graph capture, tight serving loops, harnesses that forbid
 * hipMalloc.  It is the ordered row scatter that PJRT_LoadedExecutable_Execute runs for stablehlo.scatter
 * (reference semantics: src/pjrt_plugin/ops/gather_scatter.cc:296-699, with updates applied in the order
 * they appear), with the sort workspace taken from a fixed device array inside the library instead of the
 * executable's arena.  It calls no hipMalloc / hipFree and no allocating library routine.
 */
#ifndef MI355X_NOALLOC_H_
#define MI355X_NOALLOC_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Largest num_updates the fixed workspace holds (16 bytes per update plus 65 KiB of sort counters:
 * about 4.1 MiB of device memory per GPU the library has run on, held until the process ends). */
#define MI355X_NOALLOC_MAX_UPDATES 262144

typedef struct {
  int64_t num_updates;   /* rows of `updates`, entries of `indices` */
  int64_t row_elems;     /* elements per row (operand and updates) */
  int64_t operand_rows;  /* rows of the operand; indices outside [0, operand_rows) are dropped */
  int kind;              /* 0 add, 1 set, 2 multiply, 3 minimum, 4 maximum */
  int dtype;             /* 0 f32, 1 bf16, 2 s32, 3 u32 */
  int index_bytes;       /* 4 (int32) or 8 (int64) */
} mi355x_scatter_desc;

/* result[indices[i], :] = combine(result[indices[i], :], updates[i, :]) for i = 0 .. num_updates-1, every row's
 * updates applied in ascending i (bit-identical to a sequential loop).  `result` (operand_rows x row_elems)
 * already holds the operand and is updated in place; all three pointers are device memory of the current HIP
 * device; the work is enqueued on `hip_stream` (a hipStream_t, NULL = the null stream) and not waited for.
 *
 * Returns 0 on success.  1 = invalid argument, 2 = num_updates above MI355X_NOALLOC_MAX_UPDATES, 3 = the sizes need
 * more workgroups than one launch holds (row_elems above 16 776 960); these three are found before anything is
 * enqueued.  1000 + e = the HIP runtime reported error e (resolving the workspace, or a launch; launches before the
 * failing one may have been enqueued and `result` is then undefined).  If `error` is non-NULL a NUL-terminated
 * description is written into error[0 .. error_len).
 *
 * All calls on one GPU share that GPU's workspace: calls that may run concurrently on one GPU (different
 * streams or threads) race and must be serialised by the caller.  Nothing in the workspace has to start at
 * zero: every call writes all the keys, positions and counters it later reads. */
int mi355x_scatter_rows_noalloc(const mi355x_scatter_desc* desc, void* result, const void* indices, const void* updates,
                                void* hip_stream, char* error, size_t error_len);

#ifdef __cplusplus
}
#endif

#endif /* MI355X_NOALLOC_H_ */
