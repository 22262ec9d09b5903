"""Seeded random loop nests -- row reductions with post-processing, element-wise 2-D updates, two-phase
row normalisations and time loops over ping-pong buffers -- compiled under several parallelisations and
compared with the Python interpreter running the very same function (the reference's own test method,
e.g. test/test_slicing.py:111-115)."""
import linecache

import numpy as np
import pytest

import parpy_amd as parpy
import parpy_amd.operators as ops
from parpy_amd.compile import hiprtc_compile

HIP = parpy.CompileBackend.Hip


def opts_for(p):
    o = parpy.par(p)
    o.backend = HIP
    return o


def build(name, src):
    fname = f"<{name}>"
    linecache.cache[fname] = (len(src), None, src.splitlines(True), fname)
    ns = {"parpy": parpy, "ops": ops}
    exec(compile(src, fname, "exec"), ns)
    return ns[name]


def term(rng):
    return str(rng.choice(["x[i, j]", "y[j]", "(x[i, j] * y[j])", "(x[i, j] + z[i])", "abs(x[i, j])", "(x[i, j] - 0.5)",
                           "ops.max(x[i, j], y[j])", "(x[i, j] * x[i, j])", "ops.exp(ops.min(x[i, j], 1.0))"]))


def make_program(rng, case):
    kind = case % 4
    name = f"prog_{case}"
    if kind == 0:      # row reduction, then something with the result
        op = str(rng.choice(["+", "max", "min"]))
        init = {"+": "0.0", "max": "-ops.inf", "min": "ops.inf"}[op]
        upd = f"acc + {term(rng)}" if op == "+" else f"ops.{op}(acc, {term(rng)})"
        post = str(rng.choice(["acc", "(acc * z[i])", "(acc if acc > z[i] else z[i])", "ops.sqrt(abs(acc))", "(acc + 1.0)"]))
        src = (f"def {name}(x, y, z, out, out2, N, M):\n    parpy.label('outer')\n    for i in range(N):\n"
               f"        acc = ops.float32({init})\n        parpy.label('inner')\n        for j in range(M):\n            acc = {upd}\n"
               f"        out[i] = {post}\n")
    elif kind == 1:    # element-wise 2-D update
        src = (f"def {name}(x, y, z, out, out2, N, M):\n    parpy.label('outer')\n    for i in range(N):\n"
               f"        parpy.label('inner')\n        for j in range(M):\n            out2[i, j] = {term(rng)} + {term(rng)}\n")
    elif kind == 2:    # two phases over the row with a reduction in between
        red = str(rng.choice(["max", "sum"]))
        use = str(rng.choice(["x[i, :] - m", "x[i, :] * m", "ops.max(x[i, :], m)"]))
        src = (f"def {name}(x, y, z, out, out2, N, M):\n    parpy.label('outer')\n    for i in range(N):\n"
               f"        parpy.label('inner')\n        m = ops.{red}(x[i, :])\n        parpy.label('inner')\n        out2[i, :] = {use}\n"
               f"        parpy.label('inner')\n        out[i] = ops.sum(out2[i, :])\n")
    else:              # time loop over two buffers selected by parity, inner loop parallel
        steps = int(rng.integers(2, 6))
        mix = str(rng.choice(["0.5 * (src[i, j] + src[i, (j + 1) % M])", "ops.max(src[i, j], src[i, (j + M - 1) % M]) - 0.25",
                              "src[i, j] * y[j] + z[i]"]))
        src = (f"def {name}(x, y, z, out, out2, N, M):\n    parpy.label('outer')\n    for i in range(N):\n"
               f"        for t in range({steps}):\n            src = x\n            dst = out2\n            if t & 1:\n"
               f"                src = out2\n                dst = x\n            parpy.label('inner')\n            for j in range(M):\n"
               f"                dst[i, j] = {mix}\n        parpy.label('inner')\n        s1 = ops.sum(x[i, :])\n"
               f"        parpy.label('inner')\n        s2 = ops.sum(out2[i, :])\n        out[i] = s1 + s2\n")
    return name, src, kind


def par_specs(kind, N, M):
    specs = [{'outer': parpy.threads(N)}]
    for inner in (64, 256):
        p = parpy.threads(inner)
        specs.append({'outer': parpy.threads(N), 'inner': p.reduce() if kind == 0 else p})
    if kind in (0, 1):
        p = parpy.threads(2048)
        specs.append({'outer': parpy.threads(N), 'inner': p.reduce() if kind == 0 else p})
    return specs


def inputs(rng, N, M):
    x = rng.uniform(-1, 1, (N, M)).astype(np.float32)
    y = rng.uniform(-1, 1, M).astype(np.float32)
    z = rng.uniform(-1, 1, N).astype(np.float32)
    return x, y, z, np.zeros(N, dtype=np.float32), np.zeros((N, M), dtype=np.float32)


CASES = list(range(32))


# ---------------------------------------------------------------- further shapes
def more_program(rng, case):
    kind = case % 4
    name = f"more_{case}"
    if kind == 0:      # three levels: rows, columns, a reduction over a third dimension
        upd = str(rng.choice(["acc + w[i, j, k] * v[k]", "ops.max(acc, w[i, j, k] + v[k])", "acc + abs(w[i, j, k] - v[k])"]))
        init = "-ops.inf" if "max" in upd else "0.0"
        src = (f"def {name}(w, v, x, idx, out2, N, M, K):\n    parpy.label('outer')\n    for i in range(N):\n"
               f"        parpy.label('mid')\n        for j in range(M):\n            acc = ops.float32({init})\n"
               f"            parpy.label('inner')\n            for k in range(K):\n                acc = {upd}\n            out2[i, j] = acc\n")
    elif kind == 1:    # data-dependent while loop per element (integer work)
        src = (f"def {name}(w, v, x, idx, out2, N, M, K):\n    parpy.label('outer')\n    for i in range(N):\n"
               f"        parpy.label('mid')\n        for j in range(M):\n            n = idx[j] + i + 1\n            c = 0\n"
               f"            while n != 1 and c < 50:\n                if n % 2 == 0:\n                    n = n // 2\n"
               f"                else:\n                    n = 3 * n + 1\n                c = c + 1\n            out2[i, j] = ops.float32(c)\n")
    elif kind == 2:    # a branch on a per-row value with the same parallel structure on both sides
        a, b = str(rng.choice(["x[i, j] * 2.0", "x[i, j] + v[0]", "abs(x[i, j])"])), str(rng.choice(["-x[i, j]", "x[i, j] * x[i, j]", "0.25"]))
        src = (f"def {name}(w, v, x, idx, out2, N, M, K):\n    parpy.label('outer')\n    for i in range(N):\n"
               f"        if x[i, 0] > 0.0:\n            parpy.label('mid')\n            for j in range(M):\n                out2[i, j] = {a}\n"
               f"        else:\n            parpy.label('mid')\n            for j in range(M):\n                out2[i, j] = {b}\n")
    else:              # gather through an index array
        src = (f"def {name}(w, v, x, idx, out2, N, M, K):\n    parpy.label('outer')\n    for i in range(N):\n"
               f"        parpy.label('mid')\n        for j in range(M):\n            out2[i, j] = x[i, idx[j]] + x[(i + 1) % N, idx[(j + 3) % M]]\n")
    return name, src, kind


MORE = list(range(12))


def more_inputs(rng, N, M, K):
    return (rng.uniform(-1, 1, (N, M, K)).astype(np.float32), rng.uniform(-1, 1, K).astype(np.float32),
            rng.uniform(-1, 1, (N, M)).astype(np.float32), rng.permutation(M).astype(np.int64), np.zeros((N, M), dtype=np.float32))


def more_specs(kind, N, M):
    specs = [{'outer': parpy.threads(N)}, {'outer': parpy.threads(N), 'mid': parpy.threads(M)}, {'outer': parpy.threads(N), 'mid': parpy.threads(64)}]
    if kind == 0:
        specs += [{'outer': parpy.threads(N), 'mid': parpy.threads(M), 'inner': parpy.threads(64).reduce()},
                  {'outer': parpy.threads(N), 'inner': parpy.threads(128).reduce()}]
    return specs


@pytest.mark.parametrize("case", MORE)
def test_more_random_programs_compile(case):
    rng = np.random.default_rng(2000 + case)
    name, src, kind = more_program(rng, case)
    f = build(name, src)
    N, M, K = 4, 24, 40
    for p in more_specs(kind, N, M):
        s = parpy.print_compiled(f, list(more_inputs(rng, N, M, K)) + [N, M, K], opts_for(p))
        hiprtc_compile(s[:s.index("// host side")], opts_for({}))


@pytest.mark.gpu
@pytest.mark.parametrize("case", MORE)
def test_more_random_programs_on_device(case):
    rng = np.random.default_rng(2000 + case)
    name, src, kind = more_program(rng, case)
    f = build(name, src)
    for N, M, K in [(4, 24, 40), (3, 130, 70)]:
        base = more_inputs(rng, N, M, K)
        want = [a.copy() for a in base]
        with np.errstate(all="ignore"):
            f(*want, N, M, K)
        for p in more_specs(kind, N, M):
            got = [a.copy() for a in base]
            parpy.jit(f)(*got, N, M, K, opts=opts_for(p))
            assert np.allclose(got[-1], want[-1], rtol=1e-4, atol=1e-4), (src, N, M, K, sorted(p), np.abs(got[-1] - want[-1]).max())


@pytest.mark.parametrize("case", CASES)
def test_random_programs_compile(case):
    rng = np.random.default_rng(1000 + case)
    name, src, kind = make_program(rng, case)
    f = build(name, src)
    N, M = 7, 96
    for p in par_specs(kind, N, M)[:2]:
        s = parpy.print_compiled(f, list(inputs(rng, N, M)) + [N, M], opts_for(p))
        hiprtc_compile(s[:s.index("// host side")], opts_for({}))


@pytest.mark.gpu
@pytest.mark.parametrize("case", CASES)
def test_random_programs_on_device(case):
    rng = np.random.default_rng(1000 + case)
    name, src, kind = make_program(rng, case)
    f = build(name, src)
    for N, M in [(5, 64), (9, 200), (3, 2048)]:
        base = inputs(rng, N, M)
        want = [a.copy() for a in base]
        with np.errstate(all="ignore"):
            f(*want, N, M)
        for p in par_specs(kind, N, M):
            got = [a.copy() for a in base]
            parpy.jit(f)(*got, N, M, opts=opts_for(p))
            for g, w, label in zip(got, want, "xyz oO"):
                assert np.allclose(g, w, rtol=1e-4, atol=1e-4, equal_nan=True), (src, N, M, sorted(p), label, np.abs(g - w).max())


# ---------------------------------------------------------------- strided iterations with quotients and remainders
def strided_program(rng, case, T):
    """A parallel loop of 2T..8T iterations meant for T threads: thread g gets g, g + T, ...  Elements are picked by
    quotients and remainders of the iteration number, some by divisors of T (the same element in all iterations of a
    thread, or the counter's element) and some not; one term is a selection whose test guards an index."""
    name = f"strided_{case}"
    div = [1, 2, 4, T // 4, T // 2, T, 2 * T, 3, 5, 7]

    def c():
        return int(rng.choice(div))

    def idx():
        kind = int(rng.integers(0, 6))
        if kind == 0:
            return f"(i // {c()}) % {c()}"
        if kind == 1:
            return f"i % {c()}"
        if kind == 2:
            return f"(i % {c()}) // {int(rng.choice([1, 2, 3, 4]))}"
        if kind == 3:
            return f"((i // 4) % {max(T // 4, 1)}) + {int(rng.integers(0, 4))} * {max(T // 4, 1)}"
        if kind == 4:
            return f"(i // {int(rng.choice([T, 2 * T, T // 2]))}) * 3 + i % 3"
        return f"(i + {int(rng.integers(1, 9))}) % {c()}"

    def term():
        kind = int(rng.integers(0, 5))
        if kind == 0:
            return f"a[{idx()}]"
        if kind == 1:
            return f"b[{idx()}] * a[{idx()}]"
        if kind == 2:
            return f"ops.float32(({idx()}) % 11)"
        if kind == 3:
            g = int(rng.choice([T // 2, T // 4 * 3]))
            return f"(s[i % {T}] if i % {T} < {g} else b[{idx()}])"
        return f"ops.max(a[{idx()}], b[i // {T}])"
    body = " + ".join(term() for _ in range(int(rng.integers(2, 5))))
    # (stored transposed -- thread g writes out[g * per + k] -- so that the loop keeps its strided form: a unit-stride
    # store would have the iterations regrouped four to a thread)
    src = (f"def {name}(a, b, s, out, N):\n    parpy.label('i')\n    for i in range(N):\n"
           f"        out[(i % {T}) * (N // {T}) + i // {T}] = {body}\n")
    return name, src


STRIDED = list(range(24))


def strided_inputs(rng, T, per):
    N = T * per
    # `s` is only as long as the widest guard allows (3 T / 4 elements): an unguarded read runs past it
    return (rng.uniform(-1, 1, 16 * T + 64).astype(np.float32), rng.uniform(-1, 1, 16 * T + 64).astype(np.float32),
            rng.uniform(-1, 1, T // 4 * 3).astype(np.float32), np.zeros(N, dtype=np.float32)), N


@pytest.mark.parametrize("case", STRIDED[:8])
def test_strided_programs_compile(case):
    rng = np.random.default_rng(3000 + case)
    T = int(rng.choice([64, 128, 256]))
    name, src = strided_program(rng, case, T)
    f = build(name, src)
    arrays, N = strided_inputs(rng, T, 4)
    for share in (True, False):
        o = opts_for({'i': parpy.threads(T)})
        o.opt_share_iterations = share
        s = parpy.print_compiled(f, list(arrays) + [N], o)
        hiprtc_compile(s[:s.index("// host side")], opts_for({}))


@pytest.mark.gpu
@pytest.mark.parametrize("case", STRIDED)
def test_strided_programs_on_device(case):
    rng = np.random.default_rng(3000 + case)
    T = int(rng.choice([64, 128, 256]))
    name, src = strided_program(rng, case, T)
    f = build(name, src)
    for per, tpb in [(2, None), (4, None), (8, 64), (3, None)]:
        arrays, N = strided_inputs(rng, T, per)
        want = [a.copy() for a in arrays]
        f(*want, N)
        # (with 64-bit index arithmetic as well: quotients and remainders of sums that provably fit 31 bits are
        # computed in 32 bits, and no 64-bit quotient is ever cut down to a 32-bit element offset)
        for share, narrow in ((True, True), (False, True), (True, False)):
            got = [a.copy() for a in arrays]
            p = parpy.threads(T) if tpb is None else parpy.threads(T).tpb(tpb)
            o = opts_for({'i': p})
            o.opt_share_iterations = share
            o.opt_narrow_index = narrow
            parpy.jit(f)(*got, N, opts=o)
            # (products and sums may be contracted into fused multiply-adds on the device: not bit-equal)
            assert np.allclose(got[-1], want[-1], rtol=1e-5, atol=1e-6), (src, T, per, tpb, share, narrow, np.abs(got[-1] - want[-1]).max())


# ---------------------------------------------------------------- index scalars that are assigned again between accesses
def walking_program(rng, case):
    """Groups of four accesses whose subscripts read alike (`4 * q + c`) while `q` moves between them, on loads, on
    stores, or on both: every access has to keep the element that the sequential program names."""
    name = f"walking_{case}"
    steps = [int(rng.integers(0, 3)) for _ in range(3)]          # how far q moves after each access (0: stays)
    loads = case % 3 != 1
    stores = case % 3 != 0
    lines = [f"def {name}(a, b, N):", "    parpy.label('i')", "    for i in range(N):", "        q = i"]
    for c in range(4):
        src = f"a[4 * q + {c}]" if loads else f"a[4 * i + {c}]"
        dst = f"b[4 * q + {c}]" if stores else f"b[4 * i + {c}]"
        lines.append(f"        x{c} = {src} + {c}.0")
        lines.append(f"        {dst} = x{c}")
        if c < 3 and steps[c]:
            lines.append(f"        q = q + {steps[c]}")
    return name, "\n".join(lines) + "\n"


WALKING = list(range(9))


@pytest.mark.parametrize("case", WALKING[:3])
def test_walking_programs_compile(case):
    rng = np.random.default_rng(4000 + case)
    name, src = walking_program(rng, case)
    f = build(name, src)
    s = parpy.print_compiled(f, [np.zeros(4 * 300, dtype=np.float32), np.zeros(4 * 300, dtype=np.float32), 256], opts_for({'i': parpy.threads(256)}))
    hiprtc_compile(s[:s.index("// host side")], opts_for({}))


@pytest.mark.gpu
@pytest.mark.parametrize("case", WALKING)
def test_walking_programs_on_device(case):
    rng = np.random.default_rng(4000 + case)
    name, src = walking_program(rng, case)
    f = build(name, src)
    N = 256
    # component c of an iteration goes to element 4 * (i + offset_c) + c: no two iterations store to the same element,
    # so the parallel run has one defined result; elements nobody stores to keep the marker value
    a = rng.uniform(-1, 1, 4 * (N + 8)).astype(np.float32)
    want = np.full(4 * (N + 8), -7.0, dtype=np.float32)
    f(a.copy(), want, N)
    got = np.full(4 * (N + 8), -7.0, dtype=np.float32)
    parpy.jit(f)(a.copy(), got, N, opts=opts_for({'i': parpy.threads(N)}))
    assert np.array_equal(got, want), (src, np.abs(got - want).max())


# ---------------------------------------------------------------- stepping programs: rows that swap every step, a look-up every few steps
def stepping_program(rng, case, period=None):
    """A sequential loop of steps over two rows that swap roles (`src` / `dst` chosen by the step's parity), every
    element of the new row a sum of products of elements of the old one (its own and two picked by a random index
    pattern) times a table value selected by a per-step observation, groups of 1, 2 or 4 consecutive elements per
    iteration; every few steps the largest element of the new row is looked up and the next step divides by it; at the
    end the row is summed.  The shape of the rescaled forward pass, with everything that the memory passes key on
    (group size, index patterns, look-up period, thread count) drawn at random."""
    name = f"stepping_{case}"
    V = int(rng.choice([1, 2, 4]))
    P = int(rng.choice([1, 2, 3, 4, 8]))
    if period is not None:
        P = period
    G = "(M // %d)" % V

    def pred():
        kind = int(rng.integers(0, 6))
        if kind == 0:
            return "q"
        if kind == 1:
            return f"({G} * {int(rng.integers(0, V))} + q)" if V > 1 else f"((q + 7) % M)"
        if kind == 2:
            return f"((q + {int(rng.integers(1, 9))}) % {G})"
        if kind == 3:
            return f"(({V} * q + {int(rng.integers(1, 5))}) % M)"
        if kind == 4:
            return "(q // 2)"
        return "(M - 1 - q)"
    if case % 3 == 2:
        return name, _max_plus_steps(name, rng, V, P, pred), V
    lines = [f"def {name}(x, w, w2, tab, obs, a, b, out, N, M, T):", "    parpy.label('outer')", "    for i in range(N):",
             "        parpy.label('inner')", "        for j in range(M):", "            a[i, j] = x[i, j]",
             "        r = ops.float32(1.0)", "        for t in range(1, T):", "            src = b", "            dst = a",
             "            if t & 1:", "                src = a", "                dst = b", "            o = obs[i, t]",
             "            parpy.label('inner')", f"            for q in range(M // {V}):",
             f"                p1 = src[i, {pred()}]", f"                p2 = src[i, {pred()}]"]
    if int(rng.integers(0, 2)) or V == 1:
        for u in range(V):
            lines.append(f"                dst[i, {V} * q + {u}] = ((p1 * w[q, {u}] + p2 * w[q, {(u + 1) % V}] + src[i, {V} * q + {u}] * w2[{V} * q + {u}]) * r) * tab[o, {V} * q + {u}]")
    else:
        lines += [f"                for u in range({V}):",
                  f"                    s = p1 * w[q, u] + p2 * w[q, ({V} - 1) - u] + src[i, {V} * q + u] * w2[{V} * q + u]",
                  f"                    dst[i, {V} * q + u] = (s * r) * tab[o, {V} * q + u]"]
    lines += ["            r = ops.float32(1.0)", f"            if t % {P} == 0:", "                cur = a", "                if t & 1:",
              "                    cur = b", "                parpy.label('inner')", "                top = ops.max(cur[i, :])",
              "                r = ops.float32(1.0) / top",
              "        fin = a", "        if T & 1 == 0:", "            fin = b", "        parpy.label('inner')",
              "        total = ops.sum(fin[i, :])", "        out[i] = total * r"]
    return name, "\n".join(lines) + "\n", V


def _max_plus_steps(name, rng, V, P, pred):
    """The same stepping structure in the (max, +) semiring: the best of three sums instead of a sum of three
    products, the looked-up maximum subtracted instead of divided by (a Viterbi-like pass)."""
    lines = [f"def {name}(x, w, w2, tab, obs, a, b, out, N, M, T):", "    parpy.label('outer')", "    for i in range(N):",
             "        parpy.label('inner')", "        for j in range(M):", "            a[i, j] = x[i, j]",
             "        r = ops.float32(0.0)", "        for t in range(1, T):", "            src = b", "            dst = a",
             "            if t & 1:", "                src = a", "                dst = b", "            o = obs[i, t]",
             "            parpy.label('inner')", f"            for q in range(M // {V}):",
             f"                p1 = src[i, {pred()}]", f"                p2 = src[i, {pred()}]"]
    for u in range(V):
        lines.append(f"                dst[i, {V} * q + {u}] = ops.max(ops.max(p1 + w[q, {u}], p2 + w[q, {(u + 1) % V}]), src[i, {V} * q + {u}] + w2[{V} * q + {u}]) - r + tab[o, {V} * q + {u}]")
    lines += ["            r = ops.float32(0.0)", f"            if t % {P} == 0:", "                cur = a", "                if t & 1:",
              "                    cur = b", "                parpy.label('inner')", "                top = ops.max(cur[i, :])",
              "                r = top",
              "        fin = a", "        if T & 1 == 0:", "            fin = b", "        parpy.label('inner')",
              "        total = ops.max(fin[i, :])", "        out[i] = total - r"]
    return "\n".join(lines) + "\n"


STEPPING = list(range(12))


def stepping_inputs(rng, N, M, T, V):
    return (rng.uniform(0.5, 1.0, (N, M)).astype(np.float32), rng.uniform(0.1, 0.5, (M // V, V)).astype(np.float32),
            rng.uniform(0.1, 0.5, M).astype(np.float32), rng.uniform(0.5, 1.0, (5, M)).astype(np.float32),
            rng.integers(0, 5, (N, T)).astype(np.int8), np.zeros((N, M), dtype=np.float32), np.zeros((N, M), dtype=np.float32),
            np.zeros(N, dtype=np.float32))


@pytest.mark.parametrize("case", STEPPING[:4])
def test_stepping_programs_compile(case):
    rng = np.random.default_rng(6000 + case)
    name, src, V = stepping_program(rng, case)
    f = build(name, src)
    N, M, T = 3, 256, 11
    arrays = stepping_inputs(rng, N, M, T, V)
    for threads in (64, 256):
        s = parpy.print_compiled(f, list(arrays) + [N, M, T], opts_for({'outer': parpy.threads(N), 'inner': parpy.threads(threads)}))
        hiprtc_compile(s[:s.index("// host side")], opts_for({}))


def test_rows_shared_by_several_workgroups_stay_in_global_memory():
    """With more threads on the inner level than one workgroup holds, a step is a launch of several workgroups per
    row: none of them may stage the whole row in LDS and write it back (it would overwrite what the others computed).
    With one workgroup per row the same program keeps its rows in LDS."""
    for case in STEPPING[:3]:
        rng = np.random.default_rng(6000 + case)
        name, src, V = stepping_program(rng, case, period=1)
        f = build(name, src)
        N, M, T = 2, 2048, 9
        arrays = stepping_inputs(rng, N, M, T, V)
        for expand in (True, False):
            o = opts_for({'outer': parpy.threads(N), 'inner': parpy.threads(2048)})
            o.opt_expand_short_loops = expand
            s = parpy.print_compiled(f, list(arrays) + [N, M, T], o)
            assert "lds_a" not in s and "lds_b" not in s, (case, expand)
            o = opts_for({'outer': parpy.threads(N), 'inner': parpy.threads(512)})
            o.opt_expand_short_loops = expand
            s = parpy.print_compiled(f, list(arrays) + [N, M, T], o)
            assert "lds_a" in s and "lds_b" in s, (case, expand)


@pytest.mark.gpu
@pytest.mark.parametrize("case", STEPPING)
def test_stepping_programs_on_device(case):
    rng = np.random.default_rng(6000 + case)
    name, src, V = stepping_program(rng, case)
    f = build(name, src)
    for N, M, T, threads in [(3, 256, 11, 64), (2, 1024, 18, 256), (2, 64, 7, 64), (1, 4096, 10, 1024)]:
        arrays = stepping_inputs(rng, N, M, T, V)
        want = [a.copy() for a in arrays]
        f(*want, N, M, T)
        got = [a.copy() for a in arrays]
        parpy.jit(f)(*got, N, M, T, opts=opts_for({'outer': parpy.threads(N), 'inner': parpy.threads(threads)}))
        for g, w_, label in zip(got[-3:], want[-3:], ("a", "b", "out")):
            assert np.allclose(g, w_, rtol=2e-4, atol=1e-6), (src, N, M, T, threads, label, np.abs(g - w_).max())


@pytest.mark.gpu
@pytest.mark.parametrize("expand", [True, False], ids=["expanded", "inner loop kept"])
@pytest.mark.parametrize("case", STEPPING)
def test_stepping_programs_over_several_workgroups(case, expand):
    """2048 threads per row: every step is a launch of its own, the rows stay in global memory (a row that several
    workgroups work on must not be staged in LDS by each of them).  A look-up that is not made in every step sits
    under a conditional, where a reduction over several workgroups cannot be placed: refused with a message."""
    rng = np.random.default_rng(6000 + case)
    name, src, V = stepping_program(rng, case, period=1)
    f = build(name, src)
    N, M, T = 2, 2048, 9
    arrays = stepping_inputs(rng, N, M, T, V)
    o = opts_for({'outer': parpy.threads(N), 'inner': parpy.threads(2048)})
    o.opt_expand_short_loops = expand
    if case == 0:
        _, src3, _ = stepping_program(np.random.default_rng(6000 + case), case, period=3)
        with pytest.raises(RuntimeError, match="spans several workgroups"):
            parpy.print_compiled(build(name + "_every_third", src3.replace(name, name + "_every_third")), list(arrays) + [N, M, T], o)
    want = [a.copy() for a in arrays]
    f(*want, N, M, T)
    got = [a.copy() for a in arrays]
    parpy.jit(f)(*got, N, M, T, opts=o)
    for g, w_, label in zip(got[-3:], want[-3:], ("a", "b", "out")):
        assert np.allclose(g, w_, rtol=2e-4, atol=1e-6), (src, label, np.abs(g - w_).max())


# ---------------------------------------------------------------- gathers and per-thread dot products
def gather_program(case):
    """One thread per non-zero or per row with a sequential loop inside: sampled dot products with the second operand
    read by columns or by rows, sums over ragged CSR rows, a maximum over a gathered row segment -- what the lane-group
    and transposed-staging rewrites work on."""
    name = f"gather_{case}"
    kind = case % 4
    if kind == 0:
        body = ["    parpy.label('i')", "    for i in range(NNZ):", "        acc = ops.float32(0.0)", "        for k in range(K):",
                "            acc = acc + A[rows[i], k] * B[k, cols[i]]", "        out[i] = acc * vals[i]"]
    elif kind == 1:
        body = ["    parpy.label('i')", "    for i in range(NNZ):", "        acc = ops.float32(0.0)", "        for k in range(K):",
                "            acc = acc + A[rows[i], k] * BT[cols[i], k]", "        out[i] = acc + vals[i]"]
    elif kind == 2:
        body = ["    parpy.label('i')", "    for i in range(NR):", "        acc = ops.float32(0.0)", "        for j in range(ptr[i], ptr[i + 1]):",
                "            acc = acc + vals2[j] * x[cidx[j]]", "        y[i] = acc"]
    else:
        body = ["    parpy.label('i')", "    for i in range(NNZ):", "        m = ops.float32(-ops.inf)", "        for k in range(K):",
                "            m = ops.max(m, A[rows[i], k] - BT[cols[i], k])", "        out[i] = m"]
    src = f"def {name}(A, B, BT, rows, cols, vals, out, ptr, cidx, vals2, x, y, NNZ, K, NR):\n" + "\n".join(body) + "\n"
    return name, src, kind


def gather_inputs(rng, K, NNZ, NR, NRa=64, NC=128):
    A = rng.uniform(-1, 1, (NRa, K)).astype(np.float32)
    B = rng.uniform(-1, 1, (K, NC)).astype(np.float32)
    rows = np.sort(rng.integers(0, NRa, NNZ)).astype(np.int64)
    cols = rng.integers(0, NC, NNZ).astype(np.int64)
    lens = rng.integers(0, 40, NR)
    ptr = np.concatenate([[0], np.cumsum(lens)]).astype(np.int64)
    nn = max(int(ptr[-1]), 1)
    return [A, B, np.ascontiguousarray(B.T), rows, cols, rng.uniform(-1, 1, NNZ).astype(np.float32), np.zeros(NNZ, dtype=np.float32), ptr,
            rng.integers(0, NC, nn).astype(np.int64), rng.uniform(-1, 1, nn).astype(np.float32), rng.uniform(-1, 1, NC).astype(np.float32),
            np.zeros(NR, dtype=np.float32)]


@pytest.mark.gpu
@pytest.mark.parametrize("case", range(4))
def test_gather_programs_on_device(case):
    name, src, kind = gather_program(case)
    f = build(name, src)
    rng = np.random.default_rng(7000 + case)
    for K, NNZ, NR, tpb in [(1, 63, 1, None), (15, 1000, 50, 128), (128, 5000, 1000, None), (33, 64, 300, 64), (200, 1000, 7, None)]:
        base = gather_inputs(rng, K, NNZ, NR)
        want = [a.copy() for a in base]
        f(*want, NNZ, K, NR)
        n_it = NR if kind == 2 else NNZ
        for lanes in (True, False):
            got = [a.copy() for a in base]
            o = opts_for({'i': parpy.threads(n_it) if tpb is None else parpy.threads(n_it).tpb(tpb)})
            o.opt_lane_split = lanes
            parpy.jit(f)(*got, NNZ, K, NR, opts=o)
            assert np.allclose(got[6], want[6], rtol=1e-4, atol=1e-4) and np.allclose(got[11], want[11], rtol=1e-4, atol=1e-4), (src, K, NNZ, NR, tpb, lanes)


# ---------------------------------------------------------------- phases: consecutive parallel loops over the rows of a few arrays
def phases_program(rng, case):
    """Three to six consecutive parallel loops over one row each of the arrays u, v, w, every loop storing to its own
    element of one array and reading the others at its own element or at a shifted, mirrored or halved one, the whole
    optionally repeated by a sequential loop: what decides whether a row section may stay in a thread's registers
    between two loops and whether the barrier between them orders anything."""
    name = f"phases_{case}"
    arrays = ["u", "v", "w"]

    def at(arr):
        kind = int(rng.integers(0, 7))
        if kind <= 2:
            return f"{arr}[i, j]"
        if kind == 3:
            return f"{arr}[i, (j + {int(rng.integers(1, 70))}) % M]"
        if kind == 4:
            return f"{arr}[i, M - 1 - j]"
        if kind == 5:
            return f"{arr}[i, j // 2]"
        return f"{arr}[i, (j * 2) % M]"

    def phase(indent):
        dst = str(rng.choice(arrays))
        others = [a for a in arrays if a != dst] + [dst]
        a1, a2 = str(rng.choice(others)), str(rng.choice(others))
        # the destination array is only read at the thread's own element in the loop that stores to it
        t1 = f"{a1}[i, j]" if a1 == dst else at(a1)
        t2 = f"{a2}[i, j]" if a2 == dst else at(a2)
        op = str(rng.choice(["+", "-", "*"]))
        scale = str(rng.choice(["0.5", "0.25", "1.0"]))
        return [f"{indent}parpy.label('inner')", f"{indent}for j in range(M):", f"{indent}    {dst}[i, j] = ({t1} {op} {t2}) * {scale}"]
    steps = int(rng.integers(0, 4))
    lines = [f"def {name}(u, v, w, out, N, M):", "    parpy.label('outer')", "    for i in range(N):"]
    ind = "        "
    if steps:
        lines.append(f"        for t in range({steps + 1}):")
        ind = "            "
    for _ in range(int(rng.integers(3, 7))):
        lines += phase(ind)
    lines += ["        parpy.label('inner')", "        s1 = ops.sum(u[i, :])", "        parpy.label('inner')", "        s2 = ops.max(w[i, :])",
              "        out[i] = s1 + s2"]
    return name, "\n".join(lines) + "\n"


PHASES = list(range(16))


@pytest.mark.parametrize("case", PHASES[:4])
def test_phases_programs_compile(case):
    rng = np.random.default_rng(8000 + case)
    name, src = phases_program(rng, case)
    f = build(name, src)
    N, M = 3, 1000
    arrays = [rng.uniform(-1, 1, (N, M)).astype(np.float32) for _ in range(3)] + [np.zeros(N, dtype=np.float32)]
    for threads in (64, 256):
        s = parpy.print_compiled(f, arrays + [N, M], opts_for({'outer': parpy.threads(N), 'inner': parpy.threads(threads)}))
        hiprtc_compile(s[:s.index("// host side")], opts_for({}))


@pytest.mark.gpu
@pytest.mark.parametrize("case", PHASES)
def test_phases_programs_on_device(case):
    rng = np.random.default_rng(8000 + case)
    name, src = phases_program(rng, case)
    f = build(name, src)
    for N, M, threads in [(3, 1000, 64), (2, 1024, 256), (5, 70, 64), (1, 4096, 1024), (2, 4096, 2048)]:
        arrays = [rng.uniform(-1, 1, (N, M)).astype(np.float32) for _ in range(3)] + [np.zeros(N, dtype=np.float32)]
        want = [a.copy() for a in arrays]
        f(*want, N, M)
        got = [a.copy() for a in arrays]
        parpy.jit(f)(*got, N, M, opts=opts_for({'outer': parpy.threads(N), 'inner': parpy.threads(threads)}))
        for g, w_, label in zip(got, want, "uvwo"):
            assert np.allclose(g, w_, rtol=1e-4, atol=1e-5), (src, N, M, threads, label, np.abs(g - w_).max())


# ---------------------------------------------------------------- slice statements
SLICE_SHAPES = {"x4": (5, 6, 7, 8), "x3": (6, 7, 8), "y3": (9, 8, 7), "x2": (7, 8), "y2": (8, 7), "x1": (8,), "y1": (70,), "o3": (6, 7, 8), "o2": (7, 8), "o1": (8,), "p1": (70,), "s0": (4,)}
SLICE_INPUTS = ["x4", "x3", "y3", "x2", "y2", "x1", "y1"]
SLICE_OUTPUTS = ["o3", "o2", "o1", "p1"]
def slice_operand(prng, arr, extents, in_loop):
    """A subscript of `arr` whose slice dimensions have the given extents, in order; None when it does not fit."""
    shape = SLICE_SHAPES[arr]
    n = len(extents)
    if len(shape) < n: return None
    pos = sorted(prng.choice(len(shape), size=n, replace=False).tolist())
    parts = []
    k = 0
    for d, ext in enumerate(shape):
        if k < n and d == pos[k]:
            e = extents[k]; k += 1
            if e > ext: return None
            lo = int(prng.integers(0, ext - e + 1))
            if e == ext and prng.random() < 0.6: parts.append(":")
            elif lo == 0 and prng.random() < 0.5: parts.append(f":{e}")
            elif lo + e == ext and prng.random() < 0.5: parts.append(f"{lo}:")
            else: parts.append(f"{lo}:{lo + e}")
        else:
            if in_loop and ext >= 4 and prng.random() < 0.4: parts.append(f"i % {ext}")
            else: parts.append(str(int(prng.integers(0, ext))))
    return f"{arr}[{', '.join(parts)}]"
def slice_program(prng, case):
    name = f"slices_{case}"
    lines = [f"def {name}(x4, x3, y3, x2, y2, x1, y1, o3, o2, o1, p1, s0):"]
    nstmts = int(prng.integers(1, 4))
    labels = []
    groups = []
    in_loop = prng.random() < 0.4
    ind = "    "
    if in_loop:
        lines += ["    parpy.label('outer')", "    for i in range(4):"]
        ind = "        "
        labels.append("outer")
    for sidx in range(nstmts):
        n = int(prng.integers(1, 4))
        extents = [int(prng.choice([1, 3, 5, 6, 7, 8])) for _ in range(n)]
        kind = int(prng.integers(0, 3))     # 0 element-wise, 1 full reduction, 2 reduction along an axis
        ops_in = []
        for _ in range(int(prng.integers(1, 4))):
            for _try in range(20):
                o = slice_operand(prng, str(prng.choice(SLICE_INPUTS)), extents, in_loop)
                if o: ops_in.append(o); break
        if not ops_in: continue
        expr = ops_in[0]
        for o in ops_in[1:]:
            expr = f"({expr} {str(prng.choice(['+', '-', '*']))} {o})"
        if prng.random() < 0.3: expr = f"({expr} * 0.5)"
        lab = [f"L{sidx}_{d}" for d in range(n)]
        stmt = None
        if kind == 0:
            for _try in range(30):
                dst = slice_operand(prng, str(prng.choice(SLICE_OUTPUTS)), extents, False)
                if dst: stmt = f"{dst} = {expr}"; break
        elif kind == 1:
            red = str(prng.choice(["sum", "max", "min"]))
            lab = lab[:int(prng.integers(0, 2))]          # a full reduction takes at most one label
            stmt = f"s0[{int(prng.integers(0, 4))}] = ops.{red}({expr})"
        elif n >= 2:
            ax = int(prng.integers(0, n))
            rest = [e for d, e in enumerate(extents) if d != ax]
            red = str(prng.choice(["sum", "max", "min"]))
            for _try in range(30):
                dst = slice_operand(prng, str(prng.choice(SLICE_OUTPUTS)), rest, False)
                if dst: stmt = f"{dst} = ops.{red}({expr}, axis={ax})"; break
        if stmt is None: continue
        for l in lab: lines.append(f"{ind}parpy.label('{l}')")
        lines.append(f"{ind}{stmt}")
        groups.append(lab)
    if not groups: lines.append(f"{ind}parpy.label('Z')\n{ind}o1[:] = x1[:]"); groups.append(["Z"])
    return name, "\n".join(lines) + "\n", (in_loop, groups)


SLICES = list(range(24))


@pytest.mark.gpu
@pytest.mark.parametrize("case", SLICES)
def test_slice_programs_on_device(case):
    """One to three slice statements over arrays of one to four dimensions: element-wise assignments, full reductions
    and reductions along an axis, with integer indices (some of them the counter of an enclosing sequential loop),
    bounded and full slices, a label per slice dimension of which a random subset is parallel."""
    prng = np.random.default_rng(9000 + case)
    name, src, (in_loop, groups) = slice_program(prng, case)
    f = build(name, src)
    base = ([prng.uniform(-1, 1, SLICE_SHAPES[a]).astype(np.float32) for a in SLICE_INPUTS] +
            [np.zeros(SLICE_SHAPES[a], dtype=np.float32) for a in SLICE_OUTPUTS] + [np.zeros(4, dtype=np.float32)])
    want = [a.copy() for a in base]
    f(*want)
    for pick in (0, 1, 2):
        par = {}
        for g in groups:
            chosen = g if pick == 0 else g[:1] if pick == 1 else g[-1:]
            for l in chosen:
                par[l] = parpy.threads(int(prng.choice([4, 8, 64, 128])))
        if not par:
            continue
        got = [a.copy() for a in base]
        try:
            parpy.jit(f)(*got, opts=opts_for(par))
        except RuntimeError as e:
            # different thread counts on statements that end up in one kernel are refused, as in the reference
            assert "inconsistent parallel structure" in str(e), (src, e)
            continue
        for g_, w_, label in zip(got[7:], want[7:], SLICE_OUTPUTS + ["s0"]):
            assert np.allclose(g_, w_, rtol=1e-4, atol=1e-4), (src, sorted(par), label, np.abs(g_ - w_).max())
