"""The part of the C API that jaxlib drives around an execution: PJRT_Event_{IsReady, OnReady, Error, Await,
Destroy}, PJRT_Buffer_{CopyToDevice, Delete, IsDeleted} and PJRT_LoadedExecutable_GetDeviceAssignment
(reference: src/pjrt_plugin/pjrt_event.cc:28-183, pjrt_buffer.cc, pjrt_executable.cc:280-313)."""
import ctypes as C
import threading
import time

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _slow_program(n=4096, chain=40):
    """A chain of n x n float32 products: tens of milliseconds of device work per execution, so the completion
    event of an execution is still pending when the host asks about it."""
    from jax_mps_amd.shlo.builder import Builder
    b = Builder("slow_chain")
    x = b.arg((n, n), "f32")
    w = b.arg((n, n), "f32")
    y = x
    for _ in range(chain):
        y = b.matmul(y, w)
    b.ret(y)
    return b.text()


@pytest.fixture(scope="module")
def slow(client):
    n = 4096
    exe = client.compile_and_load(_slow_program(n))
    rng = np.random.default_rng(5)
    x = client.buffer_from_pyval(rng.standard_normal((n, n)).astype(np.float32))
    w = client.buffer_from_pyval((rng.standard_normal((n, n)) / np.sqrt(n)).astype(np.float32))
    exe.execute([x, w])[0].block_until_ready()     # warm: kernels loaded, allocator primed
    return exe, [x, w]


class _Recorder:
    def __init__(self):
        from jax_mps_amd import pjrt
        self.calls = []
        self.fired = threading.Event()

        def cb(error, user_arg):
            self.calls.append((error, user_arg, threading.get_ident(), time.perf_counter()))
            self.fired.set()
        self.cb = pjrt.OnReadyCallback(cb)     # kept alive by this object


def _is_ready(client, event) -> bool:
    from jax_mps_amd import pjrt
    return bool(client.plugin.call("PJRT_Event_IsReady", pjrt.Event_IsReady_Args(event=event)).is_ready)


def test_on_ready_fires_once_after_completion_on_the_service_thread(client, slow):
    from jax_mps_amd import pjrt
    exe, args = slow
    p = client.plugin
    rec = _Recorder()
    t0 = time.perf_counter()
    outs, event = exe.execute(args, return_event=True)
    assert event, "Execute must hand out a device-complete event"
    ready_at_once = _is_ready(client, event)
    p.call("PJRT_Event_OnReady", pjrt.Event_OnReady_Args(event=event, callback=rec.cb, user_arg=0x1234))
    t_registered = time.perf_counter()
    assert rec.fired.wait(60), "the OnReady callback never fired"
    assert _is_ready(client, event)
    p.call("PJRT_Event_Await", pjrt.Event_Args(event=event))
    assert p.call("PJRT_Event_Error", pjrt.Event_Error_Args(event=event)) is not None      # no error: call() would raise
    time.sleep(0.05)
    assert len(rec.calls) == 1, rec.calls
    error, user_arg, tid, t_fired = rec.calls[0]
    assert error is None and user_arg == 0x1234
    print(f"execute returned after {1e3 * (t_registered - t0):.2f} ms, ready at once: {ready_at_once}, "
          f"callback after {1e3 * (t_fired - t0):.2f} ms", flush=True)
    # asynchronous: Execute and OnReady returned before tens of milliseconds of device work were done, and the
    # callback ran on the completion thread
    assert not ready_at_once, "Execute returned only after the device had finished: the call is not asynchronous"
    assert tid != threading.get_ident()
    assert t_fired >= t_registered
    # an event that is already complete runs the callback inline, before OnReady returns
    rec2 = _Recorder()
    p.call("PJRT_Event_OnReady", pjrt.Event_OnReady_Args(event=event, callback=rec2.cb, user_arg=7))
    assert len(rec2.calls) == 1 and rec2.calls[0][2] == threading.get_ident() and rec2.calls[0][0] is None
    p.call("PJRT_Event_Destroy", pjrt.Event_Args(event=event))
    assert np.isfinite(outs[0].to_numpy()).all()


def test_on_ready_survives_destroying_the_event_first(client, slow):
    from jax_mps_amd import pjrt
    exe, args = slow
    p = client.plugin
    rec = _Recorder()
    outs, event = exe.execute(args, return_event=True)
    p.call("PJRT_Event_OnReady", pjrt.Event_OnReady_Args(event=event, callback=rec.cb, user_arg=99))
    p.call("PJRT_Event_Destroy", pjrt.Event_Args(event=event))
    assert rec.fired.wait(60)
    outs[0].block_until_ready()
    time.sleep(0.05)
    assert len(rec.calls) == 1 and rec.calls[0][0] is None and rec.calls[0][1] == 99


def test_many_callbacks_fire_in_registration_order(client, slow):
    from jax_mps_amd import pjrt
    exe, args = slow
    p = client.plugin
    order, done = [], threading.Event()

    def cb(error, user_arg):
        order.append(user_arg)
        if len(order) == 8:
            done.set()
    keep = pjrt.OnReadyCallback(cb)
    events = []
    for k in range(4):
        outs, event = exe.execute(args, return_event=True)
        events.append(event)
        p.call("PJRT_Event_OnReady", pjrt.Event_OnReady_Args(event=event, callback=keep, user_arg=2 * k + 1))
        p.call("PJRT_Event_OnReady", pjrt.Event_OnReady_Args(event=event, callback=keep, user_arg=2 * k + 2))
    assert done.wait(120)
    assert order == list(range(1, 9)), order
    for e in events:
        p.call("PJRT_Event_Destroy", pjrt.Event_Args(event=e))


def test_buffer_ready_event_and_is_ready(client):
    from jax_mps_amd import pjrt
    p = client.plugin
    buf = client.buffer_from_pyval(np.arange(1024, dtype=np.float32))
    a = p.call("PJRT_Buffer_ReadyEvent", pjrt.Buffer_ReadyEvent_Args(buffer=buf.handle))
    p.call("PJRT_Event_Await", pjrt.Event_Args(event=a.event))
    assert _is_ready(client, a.event)
    p.call("PJRT_Event_Error", pjrt.Event_Error_Args(event=a.event))
    p.call("PJRT_Event_Destroy", pjrt.Event_Args(event=a.event))


def test_copy_to_device_is_an_independent_copy(client):
    x = np.random.default_rng(3).standard_normal((257, 33)).astype(np.float32)
    src = client.buffer_from_pyval(x)
    dst = src.copy_to_device()
    assert dst.device_pointer() != src.device_pointer() and dst.device_pointer() != 0
    assert dst.shape() == (257, 33) and dst.dtype_code() == src.dtype_code()
    src.mark_deleted()
    assert np.array_equal(dst.to_numpy(), x)


def test_buffer_delete_releases_the_memory(client):
    from jax_mps_amd import pjrt
    before = client.memory_stats()["bytes_in_use"]
    buf = client.buffer_from_pyval(np.zeros(8 * 1024 * 1024, np.float32))       # 32 MiB
    held = client.memory_stats()["bytes_in_use"]
    assert held - before >= 32 * 1024 * 1024
    assert not buf.is_deleted()
    buf.mark_deleted()
    assert buf.is_deleted()
    assert client.memory_stats()["bytes_in_use"] <= held - 32 * 1024 * 1024
    assert buf.device_pointer() == 0
    with pytest.raises(pjrt.PjrtError) as e:
        buf.to_numpy()
    assert e.value.code == 9      # FAILED_PRECONDITION
    exe = client.compile_and_load("module { func.func public @main(%a: tensor<8388608xf32>) -> tensor<8388608xf32> { %0 = stablehlo.add %a, %a : tensor<8388608xf32>\n return %0 : tensor<8388608xf32> } }")
    with pytest.raises(pjrt.PjrtError):
        exe.execute([buf])
    buf.mark_deleted()            # idempotent
    buf.delete()                  # PJRT_Buffer_Destroy after Delete frees the handle only
    assert client.memory_stats()["bytes_in_use"] <= held - 32 * 1024 * 1024


def test_donated_inputs_are_consumed_only_when_the_caller_allows_it(client):
    """An argument the program declares donated (`tf.aliasing_output`, what jax.jit(..., donate_argnums) emits) is
    consumed by Execute unless the caller lists it in non_donatable_input_indices: the buffer is deleted afterwards and
    its memory recycled, so a train loop that threads its state does not grow (the reference ignores donation:
    pjrt_executable.cc:198-246)."""
    text = ("module { func.func public @main(%w: tensor<1048576xf32> {tf.aliasing_output = 0 : i32}, %g: tensor<1048576xf32>) -> tensor<1048576xf32> {\n"
            " %0 = stablehlo.subtract %w, %g : tensor<1048576xf32>\n return %0 : tensor<1048576xf32> } }")
    exe = client.compile_and_load(text)
    w0 = np.arange(1 << 20, dtype=np.float32)
    g = client.buffer_from_pyval(np.ones(1 << 20, np.float32))
    w = client.buffer_from_pyval(w0)
    kept = exe.execute([w, g])[0]                       # pjrt.py lists every input as non-donatable by default
    assert not w.is_deleted() and np.array_equal(w.to_numpy(), w0)
    base = client.memory_stats()["bytes_in_use"]
    for step in range(5):
        new = exe.execute([w, g], donate=True)[0]
        assert w.is_deleted() and not g.is_deleted()    # only the declared argument is taken
        w = new
    assert np.array_equal(w.to_numpy(), w0 - 5)
    assert client.memory_stats()["bytes_in_use"] <= base      # each step's input went back to the allocator
    assert np.array_equal(kept.to_numpy(), w0 - 1)
    # the same buffer passed for two arguments is never taken
    both = client.buffer_from_pyval(w0)
    out = exe.execute([both, both], donate=True)[0]
    assert not both.is_deleted() and not out.to_numpy().any()


def _read_varint(data, i):
    v, shift = 0, 0
    while True:
        b = data[i]
        i += 1
        v |= (b & 0x7F) << shift
        shift += 7
        if not b & 0x80:
            return v, i


def test_device_assignment_is_one_replica_one_computation_on_device_zero(client):
    """The serialized xla.DeviceAssignmentProto: replica_count = 1 (field 1), computation_count = 1 (field 2),
    one computation_devices entry (field 3) holding replica_device_ids = [0] (reference: pjrt_executable.cc:290-313)."""
    exe = client.compile_and_load("module { func.func public @main(%a: tensor<4xf32>) -> tensor<4xf32> { return %a : tensor<4xf32> } }")
    data = exe.device_assignment_bytes()
    fields, i = {}, 0
    while i < len(data):
        tag, i = _read_varint(data, i)
        num, wire = tag >> 3, tag & 7
        if wire == 0:
            v, i = _read_varint(data, i)
        else:
            assert wire == 2
            n, i = _read_varint(data, i)
            v, i = data[i:i + n], i + n
        fields.setdefault(num, []).append(v)
    assert fields[1] == [1] and fields[2] == [1] and len(fields[3]) == 1
    inner = fields[3][0]
    tag, j = _read_varint(inner, 0)
    assert tag >> 3 == 1
    if tag & 7 == 2:      # packed repeated int64
        n, j = _read_varint(inner, j)
        ids = []
        end = j + n
        while j < end:
            v, j = _read_varint(inner, j)
            ids.append(v)
    else:
        v, j = _read_varint(inner, j)
        ids = [v]
    assert ids == [0]
