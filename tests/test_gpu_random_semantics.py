"""Seeded random programs in four families that hand-written cases cover thinly, each checked bit for bit against the
CPU oracle on the GPU:

* integers: the eight integer types with corner values (limits, 0, 1, small numbers), wrapping sums, differences and
  products, division and remainder by non-zero divisors, shifts by up to twice the width, bit operations, comparisons,
  conversions between the types and through float32, bit casts, clamps, wrapping reductions, sorts;
* floats: float32 inputs half drawn from special values (signed zeros, infinities, NaN, subnormals, the largest finite
  numbers, halves, the integer limits) through every exactly rounded operation (arithmetic, square root, rounding modes,
  max / min, comparisons, selects, clamps, conversions to integers and to 16-bit floats and back, remainders), compared
  bit for bit with the sign of zeros (NaN payloads aside);
* data movement: ranks 1 to 4 through transposes, reshapes, strided slices, positive / negative / interior padding,
  reversals, concatenations, broadcasts, dynamic slices and updates at computed (clamped) offsets, row gathers;
* gather and scatter with random dimension numbers (offset, collapsed and inserted dims, index maps in any order, the
  index vector at any position, indices from two below to two above the range, add / set / max / min / mul combiners).
"""
import random

import numpy as np
import pytest

from shlo_oracle import Oracle

pytestmark = pytest.mark.gpu

INT_SEEDS = list(range(6100, 6125))
FLOAT_SEEDS = list(range(6200, 6225))
MOVE_SEEDS = list(range(6300, 6325))
GATHER_SEEDS = list(range(6400, 6425))

INTS = ["i8", "i16", "i32", "i64", "ui8", "ui16", "ui32", "ui64"]
NP = {"i8": np.int8, "i16": np.int16, "i32": np.int32, "i64": np.int64, "ui8": np.uint8, "ui16": np.uint16, "ui32": np.uint32, "ui64": np.uint64,
      "f32": np.float32}
BITS = {"i8": 8, "i16": 16, "i32": 32, "i64": 64, "ui8": 8, "ui16": 16, "ui32": 32, "ui64": 64}
SPECIAL = np.array([0.0, -0.0, 1.0, -1.0, np.inf, -np.inf, np.nan, 1e-45, -1e-45, 1.1754944e-38, 3.4028235e38, -3.4028235e38, 0.5, -0.5, 1.5, 2.5, -2.5,
                    2147483648.0, -2147483904.0, 4294967296.0, 255.5, 256.0, -129.0, 65504.0, 65520.0, 1e-8, 3.0, 0.1, 0.49999997, 8388609.0], np.float32)


# ------------------------------------------------------------------ integers
def build_integers(seed):
    from jax_mps_amd.shlo.builder import Builder
    rnd = random.Random(seed)
    b = Builder(f"random_integers_{seed}")
    R, C = rnd.choice([(8, 16), (64, 64), (3, 130), (33, 7)])
    pools, arg_types, masks = {}, [], []

    def arg(dt):
        arg_types.append(dt)
        v = b.arg((R, C), dt)
        pools.setdefault(dt, []).append(v)
        return v

    def get(dt):
        c = pools.get(dt, [])
        if c and rnd.random() < 0.8:
            return rnd.choice(c[-4:])
        if len(arg_types) < 6 or not c:
            return arg(dt)
        return rnd.choice(c)

    def put(v):
        pools.setdefault(v.dtype, []).append(v)

    for _ in range(rnd.randint(4, 24)):
        dt = rnd.choice(INTS)
        k = rnd.random()
        x, y = get(dt), get(dt)
        if k < 0.10: put(b.add(x, y))
        elif k < 0.18: put(b.sub(x, y))
        elif k < 0.26: put(b.mul(x, y))
        elif k < 0.33: put((b.div if rnd.random() < 0.5 else b.remainder)(x, b.or_(y, 1)))
        elif k < 0.41:
            amt = b.and_(y, b.constant(2 * BITS[dt] - 1, dt))
            put(b._binary(rnd.choice(["shift_left", "shift_right_logical", "shift_right_arithmetic"]), x, amt))
        elif k < 0.47: put(rnd.choice([b.and_, b.or_, b.xor])(x, y))
        elif k < 0.51: put(b.not_(x))
        elif k < 0.56: put(rnd.choice([b.maximum, b.minimum])(x, y))
        elif k < 0.60 and not dt.startswith("u"): put(rnd.choice([b.neg, b.abs, b.sign])(x))
        elif k < 0.64: put(b._unary(rnd.choice(["popcnt", "count_leading_zeros"]), x))
        elif k < 0.70: masks.append(b.compare(x, y, rnd.choice(["LT", "LE", "GT", "GE", "EQ", "NE"])))
        elif k < 0.75 and masks: put(b.select(rnd.choice(masks[-3:]), x, y))
        elif k < 0.83: put(b.convert(x, rnd.choice(INTS)))
        elif k < 0.86: put(b.convert(b.mul(b.convert(b.and_(x, b.constant(63, dt)), "f32"), 2.0), rnd.choice(INTS)))
        elif k < 0.89: put(b.bitcast_convert(x, [t for t in INTS if BITS[t] == BITS[dt] and t != dt][0]))
        elif k < 0.92: put(b.clamp(b.constant(3, dt), x, b.constant(100, dt)))
        elif k < 0.95:
            d = rnd.choice([0, 1])
            put(b.broadcast_in_dim(rnd.choice([b.reduce_sum, b.reduce_max, b.reduce_min])(x, [d]), (R, C), [1 - d]))
        elif k < 0.97: put(b.iota((R, C), rnd.choice([0, 1]), dt))
        elif k < 0.985: put(b.sort([x], dimension=rnd.choice([0, 1]))[0])
        else: put(b.reverse(x, [rnd.choice([0, 1])]))
        if masks and rnd.random() < 0.1:
            put(b.convert(masks[-1], rnd.choice(INTS)))
    outs = [vs[-1] for vs in pools.values() if not vs[-1].name.startswith("%arg")]
    if masks:
        outs.append(masks[-1])
    if not outs:
        outs = [b.add(get("i32"), 1)]
    b.ret(*outs[:6])
    rng = np.random.default_rng(seed)
    ins = []
    for dt in arg_types:
        info = np.iinfo(NP[dt])
        kind = rng.integers(0, 3)
        if kind == 1:
            a = rng.integers(max(info.min, -5), min(info.max, 5), (R, C), dtype=NP[dt], endpoint=True)
        else:
            a = rng.integers(info.min, info.max, (R, C), dtype=NP[dt], endpoint=True)
            if kind == 2:
                a.flat[::3] = rng.choice(np.array([info.min, info.max, 0, 1], dtype=NP[dt]), size=a.flat[::3].shape)
        ins.append(a)
    return b.text(), ins, arg_types


# ------------------------------------------------------------------ floats on special values
def build_floats(seed):
    from jax_mps_amd.shlo.builder import Builder
    rnd = random.Random(seed)
    b = Builder(f"random_floats_{seed}")
    R, C = rnd.choice([(8, 16), (4, 64), (33, 7)])
    xs = [b.arg((R, C), "f32") for _ in range(3)]
    F, M, I = list(xs), [], []

    def f():
        return rnd.choice(F[-6:])
    for _ in range(rnd.randint(3, 16)):
        k = rnd.random()
        x, y = f(), f()
        if k < 0.09: F.append(b.add(x, y))
        elif k < 0.16: F.append(b.sub(x, y))
        elif k < 0.23: F.append(b.mul(x, y))
        elif k < 0.30: F.append(b.div(x, y))
        elif k < 0.34: F.append(b.sqrt(x))
        elif k < 0.40: F.append(rnd.choice([b.abs, b.neg, b.sign, b.floor])(x))
        elif k < 0.46: F.append(b._unary(rnd.choice(["ceil", "round_nearest_even", "round_nearest_afz"]), x))
        elif k < 0.54: F.append(rnd.choice([b.maximum, b.minimum])(x, y))
        elif k < 0.61: M.append(b.compare(x, y, rnd.choice(["LT", "LE", "GT", "GE", "EQ", "NE"])))
        elif k < 0.67 and M: F.append(b.select(rnd.choice(M[-3:]), x, y))
        elif k < 0.71: F.append(b.clamp(b.constant(-2.0, "f32"), x, b.constant(300.0, "f32")))
        elif k < 0.78: I.append(b.convert(x, rnd.choice(["i32", "ui8", "i64", "i8", "ui32", "i16"])))
        elif k < 0.84: F.append(b.convert(b.convert(x, rnd.choice(["bf16", "f16"])), "f32"))
        elif k < 0.90: F.append(b.remainder(x, y))
        elif k < 0.95 and I: F.append(b.convert(rnd.choice(I[-2:]), "f32"))
        else: F.append(b.bitcast_convert(b.bitcast_convert(x, "i32"), "f32"))
    outs = [v for v in F[-3:] if not v.name.startswith("%arg")] + M[-2:] + I[-2:]
    if not outs:
        outs = [b.add(xs[0], xs[1])]
    b.ret(*outs)
    rng = np.random.default_rng(seed)
    ins = []
    for _ in range(3):
        a = rng.uniform(-4, 4, (R, C)).astype(np.float32)
        pick = rng.random((R, C)) < 0.5
        a[pick] = rng.choice(SPECIAL, size=int(pick.sum()))
        ins.append(a)
    return b.text(), ins, ["f32"] * 3


# ------------------------------------------------------------------ data movement
def build_movement(seed):
    from jax_mps_amd.shlo.builder import Builder
    rnd = random.Random(seed)
    b = Builder(f"random_movement_{seed}")
    dt = rnd.choice(["f32", "f32", "i32", "i8", "i64", "ui16"])
    rank = rnd.choice([1, 2, 3, 3, 4])
    shape = tuple(rnd.choice([1, 2, 3, 4, 5, 7, 8, 16, 33]) for _ in range(rank))
    while int(np.prod(shape)) > 40000:
        shape = tuple(max(1, d // 2) for d in shape)
    x = b.arg(shape, dt)
    idx_arg = b.arg((4,), "i32")
    at = lambda q: b.reshape(b.slice(idx_arg, [q % 4], [q % 4 + 1]), ())
    vals = [x]
    for _ in range(rnd.randint(2, 12)):
        v = rnd.choice(vals[-3:])
        sh = tuple(v.shape)
        r = len(sh)
        k = rnd.random()
        if k < 0.14 and r >= 2:
            perm = list(range(r))
            rnd.shuffle(perm)
            w = b.transpose(v, perm)
        elif k < 0.26:
            nel = int(np.prod(sh))
            cands = [(nel,)]
            for d in (2, 3, 4, 7, 8):
                if nel % d == 0:
                    cands += [(d, nel // d), (nel // d, d)]
                if nel % (d * 2) == 0:
                    cands += [(2, d, nel // (2 * d))]
            if r >= 2:
                cands.append((sh[0] * sh[1],) + sh[2:])
            w = b.reshape(v, rnd.choice(cands))
        elif k < 0.38:
            st = [rnd.randint(0, d - 1) for d in sh]
            w = b.slice(v, st, [rnd.randint(s + 1, d) for s, d in zip(st, sh)], [rnd.choice([1, 1, 2, 3]) for _ in sh])
        elif k < 0.50:
            lo = [rnd.choice([0, 0, 1, 2, -1]) for _ in sh]
            hi = [rnd.choice([0, 0, 1, 3, -1]) for _ in sh]
            it = [rnd.choice([0, 0, 0, 1, 2]) for _ in sh]
            if not all(d + max(d - 1, 0) * i + l + h > 0 for d, l, h, i in zip(sh, lo, hi, it)):
                continue
            w = b.pad(v, b.constant(7, dt), lo, hi, it)
        elif k < 0.58:
            w = b.reverse(v, [d for d in range(r) if rnd.random() < 0.5] or [0])
        elif k < 0.68:
            d = rnd.randrange(r)
            w = b.concatenate([v, b.reverse(v, [d]), v] if rnd.random() < 0.3 else [v, v], d)
        elif k < 0.76 and r <= 3:
            pos = rnd.randint(0, r)
            w = b.broadcast_in_dim(v, sh[:pos] + (rnd.choice([2, 3, 5]),) + sh[pos:], [d if d < pos else d + 1 for d in range(r)])
        elif k < 0.84:
            w = b.dynamic_slice(v, [at(q) for q in range(r)], [rnd.randint(1, d) for d in sh])
        elif k < 0.92:
            blk = b.slice(b.reverse(v, [0]), [0] * r, [rnd.randint(1, d) for d in sh])
            w = b.dynamic_update_slice(v, blk, [at(q + 1) for q in range(r)])
        elif r == 2:
            ii = b.remainder(b.add(b.iota((rnd.choice([1, 3, 9]),), 0), at(0)), sh[0])
            w = b.take_rows(v, b.select(b.compare(ii, 0, "LT"), b.add(ii, sh[0]), ii))
        else:
            continue
        if 0 < int(np.prod(w.shape)) <= 200000:
            vals.append(w)
    b.ret(*vals[-3:])
    rng = np.random.default_rng(seed)
    ins = [(np.arange(int(np.prod(shape))) % 120 + 1).reshape(shape).astype({**NP, "f32": np.float32}[dt]), rng.integers(-3, 12, (4,)).astype(np.int32)]
    return b.text(), ins, [dt, "i32"]


# ------------------------------------------------------------------ gather and scatter with random dimension numbers
def build_gather_scatter(seed):
    from jax_mps_amd.shlo.builder import Builder
    rnd = random.Random(seed)
    b = Builder(f"random_gather_scatter_{seed}")
    dt = rnd.choice(["f32", "f32", "i32"])
    idt = rnd.choice(["i32", "i32", "i64"])
    r = rnd.randint(1, 4)
    oshape = tuple(rnd.randint(2, 6) for _ in range(r))
    k = rnd.randint(1, r)
    index_map = rnd.sample(range(r), k)
    collapsed = sorted(d for d in range(r) if d in index_map and rnd.random() < 0.6)
    brank = rnd.randint(0, 2)
    bshape = tuple(rnd.randint(1, 4) for _ in range(brank))
    ivd = rnd.randint(0, brank)
    ishape = bshape[:ivd] + (k,) + bshape[ivd:]
    slice_sizes = [1 if d in collapsed else rnd.randint(1, oshape[d]) for d in range(r)]
    nwin = r - len(collapsed)
    orank = brank + nwin
    offset_dims = sorted(rnd.sample(range(orank), nwin))
    operand, indices = b.arg(oshape, dt), b.arg(ishape, idt)
    rng = np.random.default_rng(seed)
    ins = [(np.arange(int(np.prod(oshape))) % 50 + 1).reshape(oshape).astype(NP[dt]),
           rng.integers(-2, max(oshape[d] for d in index_map) + 2, size=ishape).astype(NP[idt])]
    dts = [dt, idt]
    if rnd.random() < 0.66:
        g = b.gather(operand, indices, offset_dims=offset_dims, collapsed_slice_dims=collapsed, start_index_map=index_map, index_vector_dim=ivd,
                     slice_sizes=slice_sizes)
        b.ret(g, b.add(g, g))
    else:
        win = [slice_sizes[d] for d in range(r) if d not in collapsed]
        ushape, wi, bi = [], 0, 0
        for d in range(orank):
            if d in offset_dims:
                ushape.append(win[wi]); wi += 1
            else:
                ushape.append(bshape[bi]); bi += 1
        upd = b.arg(tuple(ushape), dt)
        body = rnd.choice(["add", "add", "set", "max", "min", "mul"]) if dt != "f32" else rnd.choice(["add", "add", "max", "min"])
        b.ret(b.scatter(operand, indices, upd, update_window_dims=offset_dims, inserted_window_dims=collapsed, scatter_dims_to_operand_dims=index_map,
                        index_vector_dim=ivd, body=body))
        ins.append(rng.integers(-4, 5, size=tuple(ushape)).astype(NP[dt]))
        dts.append(dt)
    return b.text(), ins, dts


BUILDERS = {"integers": (build_integers, INT_SEEDS), "floats": (build_floats, FLOAT_SEEDS), "movement": (build_movement, MOVE_SEEDS),
            "gather_scatter": (build_gather_scatter, GATHER_SEEDS)}
CASES = [(family, seed) for family, (_, seeds) in BUILDERS.items() for seed in seeds]


def all_programs():
    """(name, text) of every program of this file, for whoever compiles kernels ahead of time."""
    return [(f"random_{family}_{seed}", BUILDERS[family][0](seed)[0]) for family, seed in CASES]


@pytest.mark.parametrize("family,seed", CASES)
def test_random_semantics(client, family, seed):
    from jax_mps_amd import runner
    text, ins, dts = BUILDERS[family][0](seed)
    print(family, "seed", seed, flush=True)
    exe = client.compile_and_load(text)
    got = [runner.download(o) for o in exe.execute(runner.upload(client, ins, dts))]
    with np.errstate(all="ignore"):
        want = Oracle(text).run(*ins)
    assert len(got) == len(want)
    for k, (g, w) in enumerate(zip(got, want)):
        g, w = np.asarray(g), np.asarray(w)
        assert g.shape == w.shape, f"{family} seed {seed}, output {k}: shape {g.shape} for {w.shape}"
        if w.dtype.kind == "f":
            g, w = g.astype(np.float32), w.astype(np.float32)
            nan = np.isnan(g) & np.isnan(w)      # NaN payloads may differ; everything else bit for bit, the sign of zeros too
            bad = (g.view(np.uint32) != w.view(np.uint32)) & ~nan
        else:
            bad = g.astype(w.dtype) != w
        assert not bad.any(), f"{family} seed {seed}, output {k} ({w.dtype}): {int(bad.sum())} of {w.size} differ, first at {int(np.flatnonzero(bad.ravel())[0])}"
