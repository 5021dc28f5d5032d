"""The C-ABI boundary without a GPU: the library loads, exports exactly the declared symbol, and its
function table has the populated / NULL entries the header (and the reference's table,
src/pjrt_plugin/pjrt_api.cc:232-393) prescribes.  No compute calls here."""
import ctypes as C
import re
import subprocess
from pathlib import Path

import pytest

from jax_mps_amd import pjrt

ROOT = Path(__file__).resolve().parents[1]
HEADER = (ROOT / "include" / "pjrt_c_api.h").read_text()


@pytest.fixture(scope="module")
def plugin():
    return pjrt.Plugin()


def test_exports_only_the_declared_symbols():
    """Every function include/*.h declares is exported, and nothing else of ours is."""
    declared = re.findall(r"^const PJRT_Api\* (\w+)\(void\);", HEADER, flags=re.M)
    assert declared == ["GetPjrtApi"]
    noalloc = (ROOT / "include" / "mi355x_noalloc.h").read_text()
    declared += re.findall(r"^int (mi355x_\w+)\(", noalloc, flags=re.M)
    assert declared == ["GetPjrtApi", "mi355x_scatter_rows_noalloc"]
    # every defined dynamic symbol of whatever kind (functions, kernel handles, weak template instantiations, data):
    # the reference's build hides all but its entry point (CMakeLists.txt:303-318) and so does the linker script
    # csrc/exports.map; only the HIP toolchain's own __hip_* bookkeeping symbols would be tolerated
    out = subprocess.run(["nm", "-D", "--defined-only", pjrt.default_library_path()], capture_output=True, text=True, check=True).stdout
    syms = {line.split()[-1] for line in out.splitlines() if line.strip()}
    ours = {s for s in syms if not s.startswith("__hip_")}
    assert ours == set(declared), sorted(ours ^ set(declared))[:20]


def test_noalloc_descriptor_mirrors_the_header():
    noalloc = (ROOT / "include" / "mi355x_noalloc.h").read_text()
    body = noalloc[noalloc.index("typedef struct {"):noalloc.index("} mi355x_scatter_desc;")]
    fields = re.findall(r"^\s*(?:int64_t|int) (\w+);", body, flags=re.M)
    assert fields == [f[0] for f in pjrt.ScatterDesc._fields_]
    assert C.sizeof(pjrt.ScatterDesc) == 40


def test_table_header_and_version(plugin):
    api = plugin.api
    assert api.struct_size == C.sizeof(pjrt.Api)
    assert api.pjrt_api_version.major_version == int(re.search(r"#define PJRT_API_MAJOR (\d+)", HEADER).group(1))
    assert api.pjrt_api_version.minor_version == int(re.search(r"#define PJRT_API_MINOR (\d+)", HEADER).group(1))
    assert api.extension_start   # profiler extension stub is chained


def test_python_table_mirrors_the_header():
    body = HEADER[HEADER.index("typedef struct PJRT_Api {"):HEADER.index("} PJRT_Api;")]
    fields = re.findall(r"_PJRT_API_STRUCT_FIELD\((\w+)\);|PJRT_Unimplemented_Fn\* (\w+);", body)
    names = [a or b for a, b in fields]
    assert names == pjrt.API_ENTRIES
    nulls = {b for a, b in fields if b}
    assert nulls == pjrt.NULL_ENTRIES


def test_every_entry_is_populated_or_null_as_declared(plugin):
    for name in pjrt.API_ENTRIES:
        ptr = getattr(plugin.api, name)
        if name in pjrt.NULL_ENTRIES:
            assert not ptr, f"{name} must be NULL"
        else:
            assert ptr, f"{name} must be populated"


def test_static_identity_entries(plugin):
    # entries that need no device
    a = plugin.call("PJRT_Plugin_Initialize", pjrt.Plugin_Initialize_Args())
    assert a is not None


def test_plugin_attributes_advertise_the_stablehlo_versions(plugin):
    """jaxlib reads stablehlo_current_version / stablehlo_minimum_version to choose the version it serialises the
    portable artifact for (the reference advertises none: pjrt_client.cc:42-46)."""
    a = plugin.call("PJRT_Plugin_Attributes", pjrt.Plugin_Attributes_Args())
    arr = C.cast(a.attributes, C.POINTER(pjrt.NamedValue))
    got = {}
    for i in range(a.num_attributes):
        nv = arr[i]
        assert nv.type == 2      # PJRT_NamedValue_kInt64List
        got[C.string_at(nv.name, nv.name_size).decode()] = [C.cast(nv.int64_array_value, C.POINTER(C.c_int64))[k] for k in range(nv.value_size)]
    assert set(got) == {"stablehlo_current_version", "stablehlo_minimum_version"}
    assert len(got["stablehlo_current_version"]) == 3 and got["stablehlo_minimum_version"] <= got["stablehlo_current_version"]


def test_client_create_without_gpu_is_a_clean_error(plugin):
    """No CPU fallback: without a device PJRT_Client_Create returns a PJRT_Error (code INTERNAL)."""
    import torch
    if torch.cuda.is_available():
        pytest.skip("a GPU is present; the error path needs a machine without one")
    with pytest.raises(pjrt.PjrtError) as e:
        pjrt.Client(plugin)
    assert "no HIP device" in str(e.value) or "HIP" in str(e.value)
    assert e.value.code == 13


def test_unimplemented_entries_return_the_code(plugin):
    class A(C.Structure):
        _fields_ = [("struct_size", C.c_size_t), ("extension_start", C.c_void_p), ("pad", C.c_void_p * 8)]
    for name in ("PJRT_Compile", "PJRT_Executable_OptimizedProgram", "PJRT_TopologyDescription_Serialize"):
        with pytest.raises(pjrt.PjrtError) as e:
            plugin.call(name, A())
        assert e.value.code == 12, name


def test_serialization_entries_reject_bad_arguments(plugin):
    """Serialize / DeserializeAndLoad are implemented; without valid arguments they answer INVALID_ARGUMENT, not a crash."""
    with pytest.raises(pjrt.PjrtError) as e:
        plugin.call("PJRT_Executable_Serialize", pjrt.Executable_Serialize_Args(executable=None))
    assert e.value.code == 3
    with pytest.raises(pjrt.PjrtError) as e:
        plugin.call("PJRT_Executable_DeserializeAndLoad", pjrt.Executable_DeserializeAndLoad_Args(
            client=None, serialized_executable=b"junk", serialized_executable_size=4))
    assert e.value.code == 3
