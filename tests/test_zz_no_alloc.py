"""mi355x_scatter_rows_noalloc (include/mi355x_noalloc.h) against the entry point it is a variant of:
PJRT_LoadedExecutable_Execute of the same row scatter.  Both run the ordered scatter kernels; this one takes
its sort workspace from the library's fixed device array.  Bit-exact, on two calls in a row, the second
with a smaller input (the workspace keeps the first call's contents)."""
import ctypes as C

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

# (rows, cols, updates, combiner, seed) of the calls below, in order; the build step compiles their programs ahead of time
# the first is the largest the fixed workspace holds and the second lies just above the one-workgroup sort's limit: both
# take the general radix sort, whose second key / position arrays and counters are the upper three quarters of the workspace
CASES = [(3000, 32, 262144, "add", 9), (700, 64, 9000, "add", 10), (5000, 768, 8192, "add", 11), (300, 96, 1000, "add", 12),
         (300, 96, 37, "max", 13)]


def _scatter_program(rows, cols, n, kind):
    from jax_mps_amd.shlo.builder import Builder
    b = Builder("scatter_rows_" + kind)
    x = b.arg((rows, cols), "f32")
    i = b.arg((n,), "i32")
    u = b.arg((n, cols), "f32")
    b.ret(b.scatter(x, b.reshape(i, (n, 1)), u, update_window_dims=[1], inserted_window_dims=[0],
                    scatter_dims_to_operand_dims=[0], index_vector_dim=1, body=kind))
    return b.text()


def _device_sync():
    """hipDeviceSynchronize of the HIP runtime the plugin library is bound to (found among the process's mappings,
    so that no second copy of the runtime is loaded)."""
    paths = {line.split()[-1] for line in open("/proc/self/maps") if "libamdhip64" in line}
    assert len(paths) == 1, paths
    hip = C.CDLL(paths.pop())
    hip.hipDeviceSynchronize.restype = C.c_int
    rc = hip.hipDeviceSynchronize()
    assert rc == 0, f"hipDeviceSynchronize returned {rc}"


def _both(client, rows, cols, n, kind, seed):
    from jax_mps_amd import pjrt
    rng = np.random.default_rng(seed)
    operand = rng.standard_normal((rows, cols)).astype(np.float32)
    # skewed indices with long runs of one row, a few out of range (dropped)
    idx = np.minimum(rng.zipf(1.3, size=n) - 1, rows + 2).astype(np.int32)
    idx[::17] = -1
    upd = rng.standard_normal((n, cols)).astype(np.float32)
    print(f"noalloc scatter rows={rows} cols={cols} n={n} kind={kind} seed={seed}", flush=True)
    # existing entry point: the program through PJRT_Client_Compile / PJRT_LoadedExecutable_Execute
    exe = client.compile_and_load(_scatter_program(rows, cols, n, kind))
    bufs = [client.buffer_from_pyval(a) for a in (operand, idx, upd)]
    want = exe.execute(bufs)[0].to_numpy()
    # the variant that allocates nothing: caller-owned result buffer holding the operand, updated in place
    result = client.buffer_from_pyval(operand.copy())
    for b in bufs + [result]:
        b.block_until_ready()
    pjrt.scatter_rows_noalloc(client.plugin, result.device_pointer(), bufs[1].device_pointer(), bufs[2].device_pointer(),
                              num_updates=n, row_elems=cols, operand_rows=rows, kind=kind)
    _device_sync()
    got = result.to_numpy()
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), (rows, cols, n, kind)
    # and against the sequential definition, independent of both
    if kind == "add":
        seq = operand.copy()
        ok = (idx >= 0) & (idx < rows)
        np.add.at(seq, idx[ok], upd[ok])
        assert np.array_equal(got.view(np.uint32), seq.view(np.uint32))


def test_scatter_rows_noalloc_matches_execute_twice(client):
    for rows, cols, n, kind, seed in CASES:      # each smaller than the one before: stale keys of earlier calls stay in the workspace
        _both(client, rows=rows, cols=cols, n=n, kind=kind, seed=seed)


def test_scatter_rows_noalloc_rejects_oversize_and_bad_arguments(client):
    from jax_mps_amd import pjrt
    with pytest.raises(pjrt.PjrtError) as e:
        pjrt.scatter_rows_noalloc(client.plugin, 1, 1, 1, num_updates=262145, row_elems=4, operand_rows=4)
    assert e.value.code == 2 and "MI355X_NOALLOC_MAX_UPDATES" in str(e.value)
    with pytest.raises(pjrt.PjrtError) as e:
        pjrt.scatter_rows_noalloc(client.plugin, 0, 0, 0, num_updates=4, row_elems=4, operand_rows=4)
    assert e.value.code == 1
    with pytest.raises(pjrt.PjrtError) as e:      # rows too long for one launch's grid: refused before any launch
        pjrt.scatter_rows_noalloc(client.plugin, 1, 1, 1, num_updates=4, row_elems=16776961, operand_rows=4)
    assert e.value.code == 3 and "more workgroups" in str(e.value)
    with pytest.raises(pjrt.PjrtError) as e:
        pjrt.scatter_rows_noalloc(client.plugin, 1, 1, 1, num_updates=4, row_elems=4, operand_rows=4, index_bytes=2)
    assert e.value.code == 1
    pjrt.scatter_rows_noalloc(client.plugin, 0, 0, 0, num_updates=0, row_elems=4, operand_rows=4)   # empty: nothing to do
