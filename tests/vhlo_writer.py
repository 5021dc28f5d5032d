"""Writes a StableHLO module as a VHLO portable artifact in MLIR bytecode (test infrastructure).

The plugin's bytecode reader (jax-mps_amd/csrc/bytecode.cc) has no artifact written by jaxlib to be tested on
(neither jax nor the MLIR libraries exist here), so this writer produces them: the module is parsed by the
oracle's parser, its ops are renamed to their versioned vhlo names with vhlo attributes and types, and the
result is laid out as an MLIR bytecode file (string / dialect / attribute-type / offset / IR sections, prefix
varints, values numbered per region).  Encoding tables follow the builtin and vhlo dialects' bytecode encodings
as restated in bytecode.cc; both sides share that restatement, so a test through this writer checks the container
logic and the mapping of every op's attributes, not the numeric codes themselves.
"""
from __future__ import annotations

import struct
from typing import Dict, List, Tuple

import numpy as np

from shlo_oracle import parse_with_attributes, f32_to_bf16_bits

# ---- code tables (mirror bytecode.cc) ------------------------------------------------------------------------------
B_DICT, B_STRING, B_INTEGER, B_UNKNOWN_LOC = 1, 2, 8, 15
BT_INTEGER = 0
(A_ARRAY, A_BOOL, A_CMP_DIR, A_CMP_TYPE, A_API, A_DICT, A_FFT, A_FLOAT, A_INT, A_OOA, A_PRECISION, A_RNG_ALG, A_RNG_DIST, A_STRING, A_TENSOR,
 A_TRANSPOSE, A_TYPE, A_TYPE_EXT) = range(18)
T_CODES = {"i1": 0, "bf16": 2, "f16": 3, "f32": 4, "f64": 5, "index": 9, "i8": 11, "i16": 12, "i32": 13, "i64": 14, "ui8": 16, "ui16": 17,
           "ui32": 18, "ui64": 19}
T_FUNCTION, T_TENSOR, T_TOKEN = 8, 20, 22
CMP_DIR = ["EQ", "NE", "GE", "GT", "LE", "LT"]
CMP_TYPE = ["NOTYPE", "FLOAT", "TOTALORDER", "SIGNED", "UNSIGNED"]
PRECISION = ["DEFAULT", "HIGH", "HIGHEST"]
RNG_ALG = ["DEFAULT", "THREE_FRY", "PHILOX"]
NP_OF = {"f32": np.float32, "f64": np.float64, "f16": np.float16, "i8": np.int8, "i16": np.int16, "i32": np.int32, "i64": np.int64,
         "ui8": np.uint8, "ui16": np.uint16, "ui32": np.uint32, "ui64": np.uint64}
# ops whose vhlo name carries a version other than 1
VERSIONS = {"dot_general": 2, "gather": 2, "scatter": 2}


def varint(v: int) -> bytes:
    assert 0 <= v < (1 << 64)
    for nbytes in range(1, 9):
        if v < (1 << (7 * nbytes)):
            return ((v << nbytes) | (1 << (nbytes - 1))).to_bytes(nbytes, "little")
    return b"\x00" + v.to_bytes(8, "little")


def svarint(v: int) -> bytes:
    return varint(((v << 1) ^ (v >> 63)) & ((1 << 64) - 1))


def with_flag(v: int, flag: bool) -> bytes:
    return varint((v << 1) | int(flag))


class Writer:
    def __init__(self, text: str, version: int = 6, isolated_funcs: bool = False, pack_bools: bool = True, module_properties: bool = False):
        self.funcs, module_attributes = parse_with_attributes(text)
        # builtin.module keeps its attributes as builtin ones; the device counts are the two the plugin reads
        self.module_counts = [(k, int(module_attributes[k])) for k in ("mhlo.num_partitions", "mhlo.num_replicas") if k in module_attributes]
        self.version = version
        self.isolated_funcs = isolated_funcs
        self.module_properties = module_properties and version >= 5   # builtin.module carries native properties from version 5 on
        self.pack_bools = pack_bools
        self.strings: Dict[str, int] = {}
        self.attrs: Dict[tuple, int] = {}      # key -> provisional id, in first-use order
        self.attr_keys: List[tuple] = []
        self.types: Dict[tuple, int] = {}
        self.type_keys: List[tuple] = []
        self.op_names: Dict[Tuple[str, str], int] = {}
        self.arg_attrs_override: Dict[Tuple[str, int], list] = {}   # (function, argument) -> [(name, vhlo attribute)]

    # ---- interning: keys are nested tuples; children are interned before their parents ---------------------------------
    def s(self, text: str) -> int:
        return self.strings.setdefault(text, len(self.strings))

    def attr(self, key: tuple) -> int:
        if key not in self.attrs:
            self.attrs[key] = len(self.attr_keys)
            self.attr_keys.append(key)
        return self.attrs[key]

    def type(self, key: tuple) -> int:
        if key not in self.types:
            self.types[key] = len(self.type_keys)
            self.type_keys.append(key)
        return self.types[key]

    def op_name(self, dialect: str, name: str) -> int:
        return self.op_names.setdefault((dialect, name), len(self.op_names))

    # attribute / type constructors: (dialect, kind, payload...)
    def t_scalar(self, dtype: str):
        return ("vhlo", "scalar", dtype)

    def t_of(self, tt):
        if tt.dtype == "token":
            return ("vhlo", "token")
        return ("vhlo", "tensor", tuple(int(d) for d in tt.shape), self.t_scalar(tt.dtype))

    def a_str(self, text: str):
        return ("vhlo", "string", text)

    def a_int(self, v: int, dtype="i64"):
        return ("vhlo", "int", int(v), self.t_scalar(dtype))

    def a_bool(self, v: bool):
        return ("vhlo", "bool", bool(v))

    def a_ints(self, vals, dtype="i64", shape=None):
        arr = np.asarray(list(vals), dtype=NP_OF[dtype]).reshape(shape if shape is not None else (len(list(vals)),))
        return self.a_tensor(arr, dtype)

    def a_tensor(self, arr: np.ndarray, dtype: str):
        shape = tuple(int(d) for d in arr.shape)
        flat = np.ascontiguousarray(arr).reshape(-1)
        splat = flat.size > 1 and bool((flat == flat[0]).all()) and not (dtype in ("f32", "bf16", "f16", "f64") and np.isnan(flat.astype(np.float64)).any())
        if dtype == "i1":
            vals = flat.astype(bool)
            if splat:
                blob = b"\xff" if vals[0] else b"\x00"          # the form MLIR keeps boolean splats in
            elif self.pack_bools:
                blob = np.packbits(vals, bitorder="little").tobytes()
            else:
                blob = vals.astype(np.uint8).tobytes()
        elif dtype == "bf16":
            bits = f32_to_bf16_bits(flat.astype(np.float32))
            blob = (bits[:1] if splat else bits).tobytes()
        else:
            data = flat.astype(NP_OF[dtype])
            blob = (data[:1] if splat else data).tobytes()
        return ("vhlo", "tensor_attr", ("vhlo", "tensor", shape, self.t_scalar(dtype)), blob)

    def a_enum(self, code: int, names: List[str], value: str):
        return ("vhlo", "enum", code, names.index(value))

    def a_array(self, elems):
        return ("vhlo", "array", tuple(elems))

    def a_dict(self, pairs):
        return ("vhlo", "dict", tuple(pairs))

    def a_type(self, tkey):
        return ("vhlo", "type_attr", tkey)

    # ---- op attribute mapping (oracle's parsed forms -> vhlo attribute names) --------------------------------------------
    def op_attrs(self, op, short: str) -> Dict[str, tuple]:
        a = op.attrs
        out: Dict[str, tuple] = {}

        def flag(v):
            return v in (True, "true")
        if short == "constant":
            t = op.out_types[0]
            out["value"] = self.a_tensor(np.asarray(a["value"]).reshape(t.shape), t.dtype)
        elif short == "iota":
            out["iota_dimension"] = self.a_int(a["iota_dimension"])
        elif short == "broadcast_in_dim":
            out["broadcast_dimensions"] = self.a_ints(a.get("dims", a.get("broadcast_dimensions", [])))
        elif short == "transpose":
            out["permutation"] = self.a_ints(a.get("dims", a.get("permutation")))
        elif short == "reverse":
            out["dimensions"] = self.a_ints(a.get("dims", a.get("dimensions")))
        elif short == "concatenate":
            out["dimension"] = self.a_int(a.get("dim", a.get("dimension")))
        elif short == "slice":
            for k in ("start_indices", "limit_indices", "strides"):
                out[k] = self.a_ints(a[k])
        elif short == "dynamic_slice":
            out["slice_sizes"] = self.a_ints(a.get("sizes", a.get("slice_sizes")))
        elif short == "pad":
            out["edge_padding_low"] = self.a_ints(a.get("low", a.get("edge_padding_low")))
            out["edge_padding_high"] = self.a_ints(a.get("high", a.get("edge_padding_high")))
            out["interior_padding"] = self.a_ints(a.get("interior", a.get("interior_padding")))
        elif short == "compare":
            out["comparison_direction"] = self.a_enum(A_CMP_DIR, CMP_DIR, a["comparison_direction"])
            out["compare_type"] = self.a_enum(A_CMP_TYPE, CMP_TYPE, a.get("compare_type", "NOTYPE"))
        elif short == "reduce":
            out["dimensions"] = self.a_ints(a["dimensions"])
        elif short == "dot_general":
            lb, rb = a.get("batching_dims", ([], []))
            lc, rc = a.get("contracting_dims", ([], []))
            out["lhs_batching_dimensions"] = self.a_ints(lb)
            out["rhs_batching_dimensions"] = self.a_ints(rb)
            out["lhs_contracting_dimensions"] = self.a_ints(lc)
            out["rhs_contracting_dimensions"] = self.a_ints(rc)
            out["precision_config"] = self.a_array([self.a_enum(A_PRECISION, PRECISION, "DEFAULT")] * 2)
        elif short == "gather":
            dn = a["dimension_numbers"][1]
            for k in ("offset_dims", "collapsed_slice_dims", "operand_batching_dims", "start_indices_batching_dims", "start_index_map"):
                out[k] = self.a_ints(dn.get(k, []))
            out["index_vector_dim"] = self.a_int(dn["index_vector_dim"])
            out["slice_sizes"] = self.a_ints(a["slice_sizes"])
            out["indices_are_sorted"] = self.a_bool(flag(a.get("indices_are_sorted", False)))
        elif short == "scatter":
            dn = a["scatter_dimension_numbers"][1]
            for k in ("update_window_dims", "inserted_window_dims", "input_batching_dims", "scatter_indices_batching_dims", "scatter_dims_to_operand_dims"):
                out[k] = self.a_ints(dn.get(k, []))
            out["index_vector_dim"] = self.a_int(dn["index_vector_dim"])
            out["indices_are_sorted"] = self.a_bool(flag(a.get("indices_are_sorted", False)))
            out["unique_indices"] = self.a_bool(flag(a.get("unique_indices", False)))
        elif short == "convolution":
            ls, rs, os_ = a["dim_numbers"]
            win = a.get("window", {})
            nsp = len(ls) - 2
            sp = [str(k) for k in range(nsp)]
            out["input_batch_dimension"] = self.a_int(ls.index("b"))
            out["input_feature_dimension"] = self.a_int(ls.index("f"))
            out["input_spatial_dimensions"] = self.a_ints([ls.index(x) for x in sp])
            out["kernel_input_feature_dimension"] = self.a_int(rs.index("i"))
            out["kernel_output_feature_dimension"] = self.a_int(rs.index("o"))
            out["kernel_spatial_dimensions"] = self.a_ints([rs.index(x) for x in sp])
            out["output_batch_dimension"] = self.a_int(os_.index("b"))
            out["output_feature_dimension"] = self.a_int(os_.index("f"))
            out["output_spatial_dimensions"] = self.a_ints([os_.index(x) for x in sp])
            out["window_strides"] = self.a_ints(win.get("stride", [1] * nsp))
            out["padding"] = self.a_ints(np.asarray(win.get("pad", [[0, 0]] * nsp)).reshape(-1), shape=(nsp, 2))
            out["lhs_dilation"] = self.a_ints(win.get("lhs_dilate", [1] * nsp))
            out["rhs_dilation"] = self.a_ints(win.get("rhs_dilate", [1] * nsp))
            out["window_reversal"] = self.a_tensor(np.asarray([flag(x) for x in win.get("reverse", [False] * nsp)], dtype=bool), "i1")
            out["feature_group_count"] = self.a_int(a.get("feature_group_count", 1))
            out["batch_group_count"] = self.a_int(a.get("batch_group_count", 1))
            out["precision_config"] = self.a_array([self.a_enum(A_PRECISION, PRECISION, "DEFAULT")] * 2)
        elif short == "reduce_precision":
            out["exponent_bits"] = self.a_int(a["exponent_bits"], "i32")
            out["mantissa_bits"] = self.a_int(a["mantissa_bits"], "i32")
        elif short == "sort":
            out["dimension"] = self.a_int(a.get("dimension", -1))
            out["is_stable"] = self.a_bool(flag(a.get("is_stable", False)))
        elif short in ("reduce_window", "select_and_scatter"):
            rank = len(op.in_types[0].shape)
            for k in ("window_dimensions", "window_strides", "base_dilations", "window_dilations"):
                if k in a and not (short == "select_and_scatter" and k.endswith("dilations")):
                    out[k] = self.a_ints(a[k])
            if "padding" in a:
                pad = a["padding"][0] if isinstance(a["padding"], tuple) else a["padding"]
                out["padding"] = self.a_ints(np.asarray(pad).reshape(-1), shape=(rank, 2))
        elif short == "rng_bit_generator":
            out["rng_algorithm"] = self.a_enum(A_RNG_ALG, RNG_ALG, a["rng_algorithm"])
        elif short == "custom_call":
            out["call_target_name"] = self.a_str(a["call_target_name"])
            out["has_side_effect"] = self.a_bool(False)
            config = a.get("backend_config", "")
            out["backend_config"] = self.a_str(config if isinstance(config, str) else "")
        elif short == "composite":
            out["name"] = self.a_str(a["name"])
            out["decomposition"] = self.a_str(str(a["decomposition"]).lstrip("@"))
            out["version"] = self.a_int(0, "i32")
            out["composite_attributes"] = self.a_dict([])
        elif short == "all_reduce":
            # vhlo.all_reduce_v1: replica_groups (tensor), channel_id (integer; 0 = no channel), use_global_device_ids (bool)
            groups = a["replica_groups"]
            out["replica_groups"] = self.a_tensor(np.asarray(groups[0] if isinstance(groups, tuple) else groups), "i64")
            handle = a.get("channel_handle")
            out["channel_id"] = self.a_int(handle[1]["handle"] if handle else 0)
            out["use_global_device_ids"] = self.a_bool(flag(a.get("use_global_device_ids", False)))
        elif short == "call":
            out["callee"] = self.a_str(str(a["callee"]).lstrip("@"))
        elif a and short not in ("while", "case", "return", "optimization_barrier", "select", "clamp"):
            raise NotImplementedError(f"vhlo writer: attributes of {op.name}: {sorted(a)}")
        return out

    # ---- encoders --------------------------------------------------------------------------------------------------------
    def collect(self, key):
        """Interns `key` and everything it refers to (children first)."""
        if key[0] == "builtin":
            kind = key[1]
            if kind == "string":
                self.s(key[2])
            elif kind == "dict":
                for name, value in key[2]:
                    self.collect(("builtin", "string", name))
                    self.collect(value)
            elif kind == "int":
                self.type(key[3])
            self.attr(key)
            return
        kind = key[1]
        if kind in ("scalar", "token"):
            self.type(key)
        elif kind == "tensor":
            self.collect(key[3])
            self.type(key)
        elif kind == "function":
            for t in key[2] + key[3]:
                self.collect(t)
            self.type(key)
        elif kind == "string":
            self.s(key[2])
            self.attr(key)
        elif kind in ("int",):
            self.collect(key[3])
            self.attr(key)
        elif kind in ("bool", "enum"):
            self.attr(key)
        elif kind == "tensor_attr":
            self.collect(key[2])
            self.attr(key)
        elif kind == "array":
            for e in key[2]:
                self.collect(e)
            self.attr(key)
        elif kind == "dict":
            for n, v in key[2]:
                self.collect(n)
                self.collect(v)
            self.attr(key)
        elif kind == "type_attr":
            self.collect(key[2])
            self.attr(key)
        else:
            raise AssertionError(key)

    def encode_attr(self, key, aidx, tidx) -> bytes:
        if key[0] == "builtin":
            if key[1] == "string":
                return varint(B_STRING) + varint(self.strings[key[2]])
            if key[1] == "dict":
                out = varint(B_DICT) + varint(len(key[2]))
                for name, value in key[2]:
                    out += varint(aidx[("builtin", "string", name)]) + varint(aidx[value])
                return out
            if key[1] == "unknown_loc":
                return varint(B_UNKNOWN_LOC)
            if key[1] == "int":
                return varint(B_INTEGER) + varint(tidx[key[3]]) + svarint(key[2])
            raise AssertionError(key)
        kind = key[1]
        if kind == "string":
            return varint(A_STRING) + varint(self.strings[key[2]])
        if kind == "int":
            dtype = key[3][2]
            bits = {"i1": 1, "i8": 8, "ui8": 8}.get(dtype, 64)
            return varint(A_INT) + varint(tidx[key[3]]) + (bytes([key[2] & 0xFF]) if bits <= 8 else svarint(key[2]))
        if kind == "bool":
            return varint(A_BOOL) + varint(int(key[2]))
        if kind == "enum":
            return varint(key[2]) + varint(key[3])
        if kind == "tensor_attr":
            return varint(A_TENSOR) + varint(tidx[key[2]]) + varint(len(key[3])) + key[3]
        if kind == "array":
            return varint(A_ARRAY) + varint(len(key[2])) + b"".join(varint(aidx[e]) for e in key[2])
        if kind == "dict":
            return varint(A_DICT) + varint(len(key[2])) + b"".join(varint(aidx[n]) + varint(aidx[v]) for n, v in key[2])
        if kind == "type_attr":
            return varint(A_TYPE) + varint(tidx[key[2]])
        raise AssertionError(key)

    def encode_type(self, key, tidx) -> bytes:
        kind = key[1]
        if key[0] == "builtin":
            assert kind == "integer"
            return varint(BT_INTEGER) + varint(key[2] << 2)      # width, signless
        if kind == "scalar":
            return varint(T_CODES[key[2]])
        if kind == "token":
            return varint(T_TOKEN)
        if kind == "tensor":
            return varint(T_TENSOR) + varint(len(key[2])) + b"".join(svarint(d) for d in key[2]) + varint(tidx[key[3]])
        if kind == "function":
            return (varint(T_FUNCTION) + varint(len(key[2])) + b"".join(varint(tidx[t]) for t in key[2]) +
                    varint(len(key[3])) + b"".join(varint(tidx[t]) for t in key[3]))
        raise AssertionError(key)

    # ---- IR --------------------------------------------------------------------------------------------------------------
    def vhlo_name(self, op) -> str:
        n = op.name
        for prefix in ("stablehlo.", "func."):
            if n.startswith(prefix):
                n = n[len(prefix):]
        if n.startswith("chlo."):
            raise NotImplementedError("chlo ops are not part of a vhlo artifact")
        return n

    def prepare_region(self, region, plans):
        """First pass: intern every attribute / type / op name of the region, remember each op's attribute dictionary."""
        for t in region.arg_types:
            self.collect(self.t_of(t))
        for op in region.ops:
            short = self.vhlo_name(op)
            name = f"{short}_v{VERSIONS.get(short, 1)}"
            self.op_name("vhlo", name)
            attrs = self.op_attrs(op, short)
            dict_key = None
            if attrs:
                dict_key = ("builtin", "dict", tuple(sorted(attrs.items())))
                self.collect(dict_key)
            for t in op.out_types:
                self.collect(self.t_of(t))
            plans[id(op)] = (name, dict_key)
            for r in op.regions:
                self.prepare_region(r, plans)

    def emit_region(self, region, plans, names, base, aidx, tidx, loc) -> bytes:
        """One region with one block; `names` maps value names to ids of the enclosing scope, `base` is the first free id."""
        names = dict(names)
        num_values = len(region.args) + sum(len(op.results) for op in region.ops)
        nxt = base
        out = varint(1) + varint(num_values)
        out += with_flag(len(region.ops), bool(region.args))
        if region.args:
            out += varint(len(region.args))
            for a, t in zip(region.args, region.arg_types):
                out += with_flag(tidx[self.t_of(t)], False) if self.version >= 4 else varint(tidx[self.t_of(t)]) + varint(loc)
                names[a] = nxt
                nxt += 1
            if self.version >= 3:
                out += b"\x00"      # no use-list orders
        for op in region.ops:
            name, dict_key = plans[id(op)]
            mask = (1 if dict_key else 0) | (2 if op.results else 0) | (4 if op.operands else 0) | (16 if op.regions else 0)
            out += varint(self.op_names[("vhlo", name)]) + bytes([mask]) + varint(loc)
            if dict_key:
                out += varint(aidx[dict_key])
            if op.results:
                assert len(op.results) == len(op.out_types), (op.name, op.results, op.out_types)
                out += varint(len(op.results)) + b"".join(varint(tidx[self.t_of(t)]) for t in op.out_types)
            if op.operands:
                out += varint(len(op.operands)) + b"".join(varint(names[o]) for o in op.operands)
            for r in op.results:
                names[r] = nxt
                nxt += 1
            if op.regions:
                out += with_flag(len(op.regions), False)
                for r in op.regions:
                    out += self.emit_region(r, plans, names, base + num_values, aidx, tidx, loc)
        return out

    def section(self, sid: int, data: bytes) -> bytes:
        return bytes([sid]) + varint(len(data)) + data

    def write(self) -> bytes:
        plans: Dict[int, tuple] = {}
        loc_key = ("builtin", "unknown_loc")
        self.attr(loc_key)
        self.op_name("builtin", "module")
        self.op_name("vhlo", "func_v1")
        func_plans = []
        for name, f in self.funcs.items():
            ftype = ("vhlo", "function", tuple(self.t_of(t) for t in f.body.arg_types), tuple(self.t_of(t) for t in f.result_types))
            attrs = {"sym_name": self.a_str(name), "function_type": self.a_type(ftype),
                     "sym_visibility": self.a_str("public" if name == "main" else "private"),
                     "arg_attrs": self.a_array([self.a_dict([(self.a_str(k), v) for k, v in self.arg_attrs_override.get((name, i), [])])
                                                for i in range(len(f.body.args))]),
                     "res_attrs": self.a_array([self.a_dict([])] * len(f.result_types))}
            dict_key = ("builtin", "dict", tuple(sorted(attrs.items())))
            self.collect(dict_key)
            self.prepare_region(f.body, plans)
            func_plans.append((f, dict_key))
        module_dict = None
        if self.module_counts:
            i32 = ("builtin", "integer", 32)
            module_dict = ("builtin", "dict", tuple((k, ("builtin", "int", v, i32)) for k, v in self.module_counts))
            self.collect(module_dict)
        # final numbering: attributes and types grouped by dialect (builtin first, then vhlo)
        order = [k for k in self.attr_keys if k[0] == "builtin"] + [k for k in self.attr_keys if k[0] == "vhlo"]
        aidx = {k: i for i, k in enumerate(order)}
        self.type_keys = [k for k in self.type_keys if k[0] == "builtin"] + [k for k in self.type_keys if k[0] == "vhlo"]
        tidx = {k: i for i, k in enumerate(self.type_keys)}
        loc = aidx[loc_key]
        attr_blobs = [self.encode_attr(k, aidx, tidx) for k in order]
        type_blobs = [self.encode_type(k, tidx) for k in self.type_keys]
        # sections
        dialects = ["builtin", "vhlo"]
        for d in dialects:
            self.s(d)
        for (_, n) in self.op_names:
            self.s(n)
        strings = sorted(self.strings, key=self.strings.get)
        string_sec = varint(len(strings)) + b"".join(varint(len(s.encode()) + 1) for s in reversed(strings)) + b"".join(s.encode() + b"\x00" for s in strings)
        dialect_sec = varint(len(dialects))
        for d in dialects:
            dialect_sec += with_flag(self.strings[d], False) if self.version >= 1 else varint(self.strings[d])
        # op names grouped by dialect; the index of a name is its position in this order
        by_dialect = {d: [n for (dd, n) in self.op_names if dd == d] for d in dialects}
        final_names = {}
        if self.version >= 4:
            dialect_sec += varint(len(self.op_names))
        for di, d in enumerate(dialects):
            dialect_sec += varint(di) + varint(len(by_dialect[d]))
            for n in by_dialect[d]:
                final_names[(d, n)] = len(final_names)
                dialect_sec += with_flag(self.strings[n], True) if self.version >= 5 else varint(self.strings[n])
        self.op_names = final_names
        nb = sum(1 for k in order if k[0] == "builtin")
        offset_sec = varint(len(order)) + varint(len(type_blobs))
        offset_sec += varint(0) + varint(nb) + b"".join(with_flag(len(b), True) for b in attr_blobs[:nb])
        if len(order) > nb:
            offset_sec += varint(1) + varint(len(order) - nb) + b"".join(with_flag(len(b), True) for b in attr_blobs[nb:])
        nbt = sum(1 for k in self.type_keys if k[0] == "builtin")
        if nbt:
            offset_sec += varint(0) + varint(nbt) + b"".join(with_flag(len(b), True) for b in type_blobs[:nbt])
        if len(type_blobs) > nbt:
            offset_sec += varint(1) + varint(len(type_blobs) - nbt) + b"".join(with_flag(len(b), True) for b in type_blobs[nbt:])
        attr_sec = b"".join(attr_blobs) + b"".join(type_blobs)
        # IR: top-level block with the module op, whose (isolated) region is a section of its own from version 2 on
        module_region = varint(1) + varint(0) + with_flag(len(func_plans), False)
        for f, dict_key in func_plans:
            module_region += varint(self.op_names[("vhlo", "func_v1")]) + bytes([1 | 16]) + varint(loc) + varint(aidx[dict_key])
            module_region += with_flag(1, self.isolated_funcs)
            body = self.emit_region(f.body, plans, {}, 0, aidx, tidx, loc)
            module_region += self.section(4, body) if (self.isolated_funcs and self.version >= 2) else body
        ir = with_flag(1, False) + varint(self.op_names[("builtin", "module")]) + bytes([16 | (1 if module_dict else 0) | (0x40 if self.module_properties else 0)]) + varint(loc)
        if module_dict:
            ir += varint(aidx[module_dict])
        if self.module_properties:
            ir += varint(0)                  # index into the properties section
        ir += with_flag(1, True)
        ir += self.section(4, module_region) if self.version >= 2 else module_region
        out = b"ML\xefR" + varint(self.version) + b"StableHLO_v1.9.0\x00"
        out += self.section(0, string_sec) + self.section(1, dialect_sec) + self.section(2, attr_sec) + self.section(3, offset_sec) + self.section(4, ir)
        if self.module_properties:
            # one entry: the module's two optional inherent attributes (symbol name, visibility), both absent
            out += self.section(8, varint(1) + varint(2) + b"\x00\x00")
        return out


def to_vhlo_bytecode(text: str, **kw) -> bytes:
    return Writer(text, **kw).write()
