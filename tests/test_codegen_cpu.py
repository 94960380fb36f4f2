"""Code generator checks that need no GPU: every kernel is generated and
compiled to a gfx950 code object through the C ABI (hiprtc), and the generated
text is inspected for the properties the design relies on."""
import numpy as np
import pytest

import appy_amd as appy
from appy_amd.backends.hip import codegen as cg
from appy_amd.backends.hip import dtypes as T
from appy_amd.backends.hip import selfcheck
from appy_amd.backends.hip.kernelgen import Spec


def compiled(loop_source, **vals):
    vals.setdefault("np", np)
    f, src = cg.codegen(loop_source, "kernel_loop_1", vals, {"dump_code": False})
    return f, src


def body_of(src):
    return src[src.index("// kernel for"):]


def test_all_workload_patterns_compile_for_gfx950():
    assert selfcheck.compile_all_patterns() >= 6


def test_vec_add_uses_128_bit_accesses_and_restrict():
    a = np.zeros(8, np.float32)
    f, src = compiled("#pragma parallel for simd\nfor i in range(a_shape_0):\n    c[i] = a[i] + b[i]", c=a, a=a, b=a, a_shape_0=8)
    k = body_of(src)
    assert "appy::vload<float, 4>" in k and "appy::vstore<float, 4>" in k
    assert "float* __restrict__ c" in k and "const float* __restrict__ a" in k
    assert f.analysis.kind == "flat" and not f.analysis.outer_reductions
    assert f.kernels[f.default_spec].code[:4] == b"\x7fELF"


def test_shared_reduction_ends_in_one_atomic_per_workgroup():
    s = np.zeros(1)
    a = np.zeros(8, np.float32)
    f, src = compiled("#pragma parallel for simd shared(s)\nfor i in range(n):\n    s[0] += a[i]", s=s, a=a, n=8)
    k = body_of(src)
    assert k.count("atomic_combine") == 1 and "block_reduce<appy::OpAdd, 256, double>" in k
    assert "double __acc0" in k                      # accumulates in the dtype of the shared buffer
    assert "if (threadIdx.x == 0)" in k
    red = f.analysis.outer_reductions[0]
    assert (red.key, red.op, red.ty.name) == ("s[0]", "+", "float64")
    assert f.grid_for(f.default_spec, 1 << 28, kernel=f.kernels[f.default_spec]) == 512   # 4 MiB window: 512 x 256 lanes x 2 x 16 B
    mid = {"s": s, "a": np.broadcast_to(np.float32(0), (1 << 22,))}
    sp = f.choose_spec(1 << 22, {}, mid)                 # served by the caches: few workgroups of 1024 lanes
    assert (sp.block, sp.unroll, sp.stream_loads) == (1024, 2, False)
    assert f.grid_for(sp, 1 << 22, kernel=f.kernel_for(sp)) == 128
    big = {"s": s, "a": np.broadcast_to(np.float32(0), (1 << 28,))}
    sp = f.choose_spec(1 << 28, {}, big)
    assert (sp.block, sp.unroll, sp.stream_loads) == (512, 2, True)
    assert f.grid_for(sp, 1 << 28, kernel=f.kernel_for(sp)) == 384


def test_masked_sum_loads_mask_bytes_as_vectors():
    s = np.zeros(1)
    a = np.zeros(8, np.float32)
    m = np.zeros(8, bool)
    _, src = compiled("#pragma parallel for simd shared(s)\nfor i in range(n):\n    s[0] += a[i] if m[i] else 0.0",
                      s=s, a=a, m=m, n=8)
    k = body_of(src)
    assert "appy::vload<unsigned char, 4>" in k and "appy::vload<float, 4>" in k


def test_weak_scalars_follow_numpy_promotion():
    a32 = np.zeros(8, np.float32)
    _, src = compiled("#pragma parallel for simd\nfor i in range(n):\n    c[i] = alpha * a[i] + 1.5", c=a32, a=a32, alpha=2.0, n=8)
    k = body_of(src)
    assert "(float)(alpha)" in k and "(float)(1.5)" in k       # Python floats adopt float32
    a_i = np.zeros(8, np.int32)
    c64 = np.zeros(8)
    _, src = compiled("#pragma parallel for simd\nfor i in range(n):\n    c[i] = a[i] * 0.5", c=c64, a=a_i, n=8)
    assert "(double)" in body_of(src)                          # int32 * Python float -> float64
    assert T.promote(T.F32, T.WEAK_FLOAT) == T.F32
    assert T.promote(T.I32, T.WEAK_FLOAT) == T.F64
    assert T.promote(T.I32, T.WEAK_INT) == T.I32
    assert T.true_divide(T.I32, T.I32) == T.F64
    assert T.join(T.WEAK_FLOAT, T.F32) == T.F32


def test_local_accumulator_takes_the_numpy_type():
    A = np.zeros((4, 8), np.float32)
    x = np.zeros(8, np.float32)
    y = np.zeros(4, np.float32)
    text = ("#pragma parallel for\nfor i in range(r):\n    yi = 0.0\n    #pragma simd\n"
            "    for j in range(c):\n        yi += A[i, j] * x[j]\n    y[i] = yi")
    f, src = compiled(text, A=A, x=x, y=y, r=4, c=8)
    k = body_of(src)
    assert "float yi" in k and "team_reduce<appy::OpAdd" in k
    assert f.analysis.kind == "team"
    assert "if (__lane == 0) { y[i]" in k                      # one store per row


def test_team_width_follows_the_row_length():
    f, _ = selfcheck_loop("spmv")
    arrays = {"A_data": np.zeros(16 * 1000, np.float32)}
    assert f.choose_spec(1000, {}, arrays).width == 4           # 16 non-zeros, 4 per lane
    arrays = {"A_data": np.zeros(97 * 1000, np.float32)}
    assert f.choose_spec(1000, {}, arrays).width == 32
    g, _ = selfcheck_loop("gemv")
    assert g.choose_spec(16384, {"A_shape_1": 16384}, {}).width == 32


def selfcheck_loop(name):
    selfcheck.compile_all_patterns()
    for key, (loop, src) in cg.code_cache.items():
        if name == "spmv" and "x[A_indices[j]]" in key[0]:
            return loop, src
        if name == "gemv" and "A[i, j] * x[j]" in key[0]:
            return loop, src
        if name == "spmm" and "B[A_indices[k], :]" in key[0]:
            return loop, src
    raise AssertionError(name)


def test_csr_rows_are_sorted_by_length_from_32768_rows_on():
    """Loops whose simd loop has bounds read per row take the binned shape when there are many
    rows; the analysis names the gathered operand whose stripes long rows are cut at."""
    f, _ = selfcheck_loop("spmv")
    assert f.analysis.ragged is not None and f.analysis.ragged[1] == ("x", "A_indices")
    arrays = {"A_data": np.zeros(16 * 40_000, np.float32)}
    sp = f.choose_spec(40_000, {}, arrays)
    assert sp.rows == "mixed" and sp.vec == 4
    assert f.choose_spec(30_000, {}, arrays).rows == ""                          # too few rows to be worth a pass
    assert f.choose_spec(40_000, {}, arrays, restrict=False).rows == ""          # arguments that share memory
    g, _ = selfcheck_loop("gemv")
    assert g.analysis.ragged is None and g.choose_spec(1 << 20, {"A_shape_1": 64}, {}).rows == ""    # rows of equal length
    m, _ = selfcheck_loop("spmm")
    assert m.analysis.ragged is None                                             # its ragged loop is sequential
    # the kernels of the binned launch
    bins = body_of(f.kernel_for(Spec("team", block=1024, vec=1, width=1, aux="bins")).src.text)
    assert "__trip <= __t0 ? 0 : __trip <= __t1 ? 1 : __trip <= __t2 ? 2 : 3" in bins and "__zero[threadIdx.x] = 0" in bins
    assert "x[" not in bins.split("{", 1)[1]                                     # only the set-up of a row runs here
    mixed = body_of(f.kernel_for(Spec("team", block=256, vec=4, width=64, stream_loads=True, rows="mixed")).src.text)
    assert "team_reduce_dyn<appy::OpAdd, float>" in mixed and "+= __W" in mixed
    assert "__c != __base || (__trip > __tlo && __trip <= __thi)" in mixed
    plan = body_of(f.kernel_for(Spec("team", block=256, vec=1, width=8, rows="list", parts=8, aux="plan")).src.text)
    assert "A_indices[__mid] < __target" in plan and "team_running_max<8>" in plan and "atomicAdd(&__load[threadIdx.x]" in plan
    parts = body_of(f.kernel_for(Spec("team", block=256, vec=4, width=16, phase=1, rows="list", parts=8)).src.text)
    assert "(appy::i64)(blockIdx.x & 7) + 8 * __pass : __pass" in parts and "__bnd[(__chunk + 1) * __cap + __t]" in parts
    assert "__most * 16 <= __tot * 3" in parts                  # parts tied to XCDs only while their loads are even
    fold = body_of(f.kernel_for(Spec("team", block=256, vec=4, width=1, phase=2, rows="list", parts=8)).src.text)
    assert "__c < __nsplit" in fold and "y[i] = s" in fold
    with pytest.raises(ValueError):
        Spec("team", width=16, phase=1, rows="list", parts=12)                   # parts go to the eight XCDs in turn
    with pytest.raises(ValueError):
        Spec("flat", rows="mixed")


def test_sums_of_gathered_terms_can_be_grouped_by_the_stripe_they_read():
    """`s += A[j] * x[idx[j]]` and its relatives qualify; terms that read a value of their row, a
    second gathered operand, or operands that are not four bytes wide do not."""
    f, _ = selfcheck_loop("spmv")
    g = f.analysis.grouping
    assert g is not None and (g["x"], g["idx"], g["carried"], g["name"]) == ("x", "A_indices", "A_data", "s")
    i32, f32 = np.zeros(9, np.int32), np.zeros(16, np.float32)

    def csr(term, init="0.0", pre="", **more):
        src = ("#pragma parallel for\nfor i in range(m):\n" + pre + f"    s = {init}\n    #pragma simd\n"
               f"    for j in range(p[i], p[i + 1]):\n        s += {term}\n    y[i] = s")
        vals = dict(p=i32, c=np.zeros(16, np.int32), v=f32, x=f32, y=np.zeros(8, np.float32), m=8)
        vals.update(more)
        return compiled(src, **vals)[0].analysis

    assert csr("x[c[j]]").grouping["carried"] is None
    assert csr("alpha * (v[j] * x[c[j]])", alpha=0.5).grouping["carried"] == "v"
    assert csr("x[c[j]] * x[c[j]]").grouping is not None                     # the same load twice
    assert csr("f * v[j] * x[c[j]]", pre="    f = y[i]\n").grouping is None  # a value of the row
    assert csr("v[j] * x[c[j]] * j").grouping is None                         # the position itself
    assert csr("v[j] * w[j] * x[c[j]]", w=f32).grouping is None               # two operands to carry
    assert csr("v[j] * x[c[j]] + z[c[j]]", z=f32).grouping is None            # two gathered operands
    assert csr("v[j] * x[c[j]]", x=np.zeros(16, np.float64)).grouping is None
    # 64-bit indices: only the kernel that writes the pairs of a row plan reads them (and narrows them); the launches that
    # group the elements every time are not staged for them
    wide = csr("v[j] * x[c[j]]", c=np.zeros(16, np.int64))
    assert wide.grouping is not None and wide.arrays["c"].ty.name == "int64"
    # the kernels
    src = ("#pragma parallel for\nfor i in range(m):\n    s = 0.0\n    #pragma simd\n"
           "    for j in range(p[i], p[i + 1]):\n        s += v[j] * x[c[j]]\n    y[i] = s")
    fw, _ = compiled(src, p=i32, c=np.zeros(16, np.int64), v=f32, x=f32, y=np.zeros(8, np.float32), m=8)
    for spec in (Spec("team", block=256, vec=1, width=64, parts=8, aux="group", block_rows=256),
                 Spec("team", block=256, vec=1, width=64, parts=8, aux="group", block_rows=256, skip_long=True),
                 Spec("team", block=256, vec=1, width=64, aux="rkeys", block_rows=256)):
        kn = fw.kernel_for(spec)
        assert ("appy::narrow_indices(appy::vload<long long, 4>(" in kn.src.text) == (spec.aux == "group")
        assert kn.code                                                        # compiles for gfx950
    group = body_of(f.kernel_for(Spec("team", block=256, vec=1, width=64, parts=8, aux="group", block_rows=256)).src.text)
    assert "__lp[__r + 1] == __hq[__r]" in group and "__flag[0] = 1" in group and "__hint[0] = 2" in group
    assert "x[" not in group.split("{", 1)[1]                                 # the gathered operand is not read here
    cells = body_of(f.kernel_for(Spec("team", block=256, vec=1, width=64, parts=16, aux="cells", block_rows=256, guard=1)).src.text)
    assert "if ((__flag[0] != 0) == true) return;" in cells and "for (int __pass = 0; __pass < 2; ++__pass)" in cells
    assert "atomicAdd(&__acc[" in cells and "(__cv * __cx)" in cells and "A_indptr[" not in cells.split("{", 1)[1]
    sums = body_of(f.kernel_for(Spec("team", block=256, vec=4, width=1, phase=2, guard=1)).src.text)
    assert "reinterpret_cast<float*>(__scratch)[(0 * __nsplit + __c) * (__hi - __lo) + (i - __lo)]" in sums and "y[i] = s" in sums
    # with long rows in the matrix: the grouping kernel walks the elements of the other rows only, the sums are not
    # added for long rows, and the kernels that cut the long rows wait on the same flag
    kept = body_of(f.kernel_for(Spec("team", block=256, vec=1, width=64, parts=8, aux="group", block_rows=256, skip_long=True)).src.text)
    assert "__kt[__i] = __n > __rowmax ? 0 : __n;" in kept and "__kp[__row + 1] <= __t + __q" in kept and "__hint[0] = 2" not in kept
    sums_kept = body_of(f.kernel_for(Spec("team", block=256, vec=4, width=1, phase=2, guard=1, skip_long=True)).src.text)
    assert "if (__trip <= __rowmax) {" in sums_kept
    parts = body_of(f.kernel_for(Spec("team", block=256, vec=4, width=16, phase=1, rows="list", parts=8, guard=1)).src.text)
    assert "if ((__flag[0] != 0) == true) return;" in parts
    with pytest.raises(ValueError):
        Spec("team", block=256, vec=4, width=4, skip_long=True)
    rest = body_of(f.kernel_for(Spec("team", block=256, vec=4, width=4, guard=2)).src.text)
    assert "if ((__flag[0] != 0) == false) return;" in rest
    with pytest.raises(ValueError):
        Spec("team", block=256, width=64, parts=24, aux="group", block_rows=256)
    with pytest.raises(ValueError):
        Spec("flat", guard=1)
    # sums of float64 are not taken: the loop keeps its rows sorted by length
    d = csr("v[j] * x[c[j]]", v=np.zeros(16, np.float64))
    assert d.grouping is None


def test_spmm_row_lives_in_registers():
    loop, _ = selfcheck_loop("spmm")
    spec = Spec("team", block=256, vec=4, width=32, extent=128)
    k = body_of(loop.kernel_for(spec).src.text)
    assert "row accumulators" in k
    inner = k[k.index("for (appy::i64 k ="):]
    loop_body = inner[: inner.index("appy::vstore")]
    assert "y[" not in loop_body and "appy::vload<float, 4>(y" not in loop_body     # no traffic to y inside the k loop
    assert k.count("appy::vstore<float, 4>(y") == 1
    # without a compile-time extent the generic (memory read-modify-write) form is used
    k2 = body_of(loop.kernel_for(Spec("team", block=256, vec=4, width=32)).src.text)
    assert "row accumulators" not in k2


def test_array_statement_lowering():
    A = np.zeros((4, 8))
    x = np.zeros(8)
    y = np.zeros(4)
    f, src = compiled("#pragma parallel for\nfor i in range(r):\n    y[i] = np.sum(alpha * A[i, :] * x[:])", A=A, x=x, y=y, r=4, alpha=1.5)
    k = body_of(src)
    assert "A_shape_1" in k and "team_reduce<appy::OpAdd" in k
    assert f.derived_shapes["A_shape_1"] == ("A", 1)
    _, src = compiled("#pragma parallel for\nfor i in range(r):\n    y[i] = A[i, :] @ x[:]", A=A, x=x, y=y, r=4)
    assert "team_reduce<appy::OpAdd" in body_of(src)
    _, src = compiled("#pragma parallel for\nfor i in range(r):\n    A[i, 2:6] = x[0:4] + 1.0", A=A, x=x, r=4)
    assert "(6LL - 2LL)" in body_of(src)


def test_non_simd_parallel_loop_with_control_flow():
    a = np.zeros(8)
    m = np.zeros(8, bool)
    b = np.zeros(1)
    f, src = compiled("#pragma parallel for shared(b)\nfor i in range(n):\n    if m[i]:\n        b[0] += a[i]", a=a, m=m, b=b, n=8)
    k = body_of(src)
    assert "atomic_combine" in k and "appy::vload<unsigned char, 2>" in k   # control flow per lane, vector loads all the same


def test_out_of_range_loop_is_caught_on_the_host():
    a = np.zeros(8, np.float32)
    f, _ = compiled("#pragma parallel for simd\nfor i in range(n):\n    c[i] = a[i + 1]", c=a, a=a, n=8)
    with pytest.raises(IndexError):
        f.prepare({"c": a, "a": a, "n": 8})


def test_scalars_in_host_checked_subscripts_are_part_of_a_replayed_call_s_identity():
    """`a[2 * i + off]` is compared with the extent of `a` on the host before a launch.  A repeat
    of the call that only launches again must not carry another `off` past that check."""
    a = np.zeros(64, np.float32)
    b = np.zeros(8, np.float32)
    f, _ = compiled("#pragma parallel for simd\nfor i in range(n):\n    b[i] = a[2 * i + off] * f", a=a, b=b, n=8, off=0, f=2.0)
    assert [(nm, d, t) for nm, d, t in f.analysis.affine_checks] == [("a", 0, "2 * i + off")]
    names = [f.arg_names[i] for i in f._value_only]
    assert "off" not in names and "n" not in names and names == ["f"]
    with pytest.raises(IndexError):
        f.prepare({"a": a, "b": b, "n": 8, "off": 60, "f": 2.0})


def test_lds_staging_is_an_option_and_refuses_unsafe_loops():
    g, _ = selfcheck_loop("gemv")
    k = body_of(g.kernel_for(Spec("team", block=256, vec=4, width=32, lds_tile=2048)).src.text)
    assert "__shared__" in k and "__tile_x[2048]" in k and k.count("__syncthreads()") == 2
    assert "appy::lds_vload<float, 4>" in k and "__lane == 0 && __active" in k
    # a loop that stores from inside its simd loop keeps the plain form (no clamped duplicate rows)
    a = np.zeros((4, 8), np.float32)
    x = np.zeros(8, np.float32)
    text = "#pragma parallel for\nfor i in range(r):\n    #pragma simd\n    for j in range(c):\n        a[i, j] = a[i, j] + x[j]"
    f, _ = compiled(text, a=a, x=x, r=4, c=8)
    k2 = body_of(f.kernel_for(Spec("team", block=256, vec=4, width=32, lds_tile=2048)).src.text)
    assert "__shared__" not in k2


def test_spec_validation():
    for bad in (dict(kind="warp"), dict(kind="flat", block=100), dict(kind="flat", vec=3), dict(kind="team", width=48),
                dict(kind="team", width=128), dict(kind="flat", unroll=0), dict(kind="team", lds_tile=1000002)):
        with pytest.raises(ValueError):
            Spec(**bad)


def test_dump_code_to_file_and_kernel_names(tmp_path):
    out = tmp_path / "kernel.hip"

    @appy.jit(dry_run=True, dump_code_to_file=str(out))
    def scale(a, f):
        #pragma parallel for simd
        for i in range(a.shape[0]):
            a[i] = a[i] * f

    a = np.arange(8, dtype=np.float32)
    scale(a, 2.0)
    text = out.read_text()
    assert 'extern "C" __global__' in text and "_scale_kernel_loop_1(" in text     # kernels carry the function's name
    assert np.array_equal(a, np.arange(8, dtype=np.float32) * 2)                    # dry_run interpreted the loop


def test_by_value_scalar_assigned_in_the_loop_is_private():
    a = np.zeros(8)
    f, src = compiled("#pragma parallel for simd\nfor i in range(n):\n    t = t + 1.0\n    a[i] = t", a=a, t=5.0, n=8)
    k = body_of(src)
    assert "const double t__arg" in k and "double t = t__arg;" in k       # every iteration starts from the caller's value


def test_codegen_is_cached_per_signature_not_per_shape():
    text = "#pragma parallel for simd\nfor i in range(n):\n    c[i] = a[i] + 1"
    f1, _ = compiled(text, c=np.zeros(8, np.float32), a=np.zeros(8, np.float32), n=8)
    f2, _ = compiled(text, c=np.zeros(800, np.float32), a=np.zeros(800, np.float32), n=800)
    f3, _ = compiled(text, c=np.zeros(8), a=np.zeros(8), n=8)
    assert f1 is f2 and f3 is not f1


def test_concurrent_code_generation_is_safe():
    import threading

    text = "#pragma parallel for simd\nfor i in range(n):\n    c[i] = a[i] * 3 + b[i]"
    got = []

    def work():
        a = np.zeros(8, np.float32)
        got.append(cg.codegen(text, "kernel_loop_9", {"c": a, "a": a, "b": a, "n": 8}, {})[0])

    ts = [threading.Thread(target=work) for _ in range(8)]
    [t.start() for t in ts]
    [t.join() for t in ts]
    assert len(got) == 8 and all(g is got[0] for g in got)


def test_loop_bounds_may_use_plain_builtins():
    a = np.zeros(8, np.float32)
    f, _ = compiled("#pragma parallel for simd\nfor i in range(min(n, m) - 1):\n    c[i] = a[i] + 1", c=a, a=a, n=8, m=5)
    import appy_amd.backends.hip.codegen as mod
    assert eval(f._hi_code, mod._HOST_EVAL_GLOBALS, {"n": 8, "m": 5}) == 4


def test_negative_literal_index_counts_from_the_end():
    a = np.zeros(8, np.float32)
    f, src = compiled("#pragma parallel for simd\nfor i in range(n):\n    c[i] = a[i] + a[-1] + b[-2, i]", c=a, a=a,
                      b=np.zeros((4, 8), np.float32), n=8)
    k = body_of(src)
    assert "a[(a_shape_0 - 1LL)]" in k and "(b_shape_0 - 2LL) * b_stride_0" in k
    assert "const appy::i64 a_shape_0" in k and "const appy::i64 b_shape_0" in k


def test_few_very_long_rows_get_a_workgroup_each():
    g, _ = selfcheck_loop("gemv")
    sp = g.choose_spec(100, {"A_shape_1": 1 << 20}, {})
    assert (sp.width, sp.block) == (1024, 1024)
    sp = g.choose_spec(2000, {"A_shape_1": 1 << 16}, {})
    assert (sp.width, sp.block) == (256, 256)
    k = body_of(g.kernel_for(sp).src.text)
    assert "appy::workgroup_reduce_all<appy::OpAdd, 256, float>" in k and "threadIdx.x & 255" in k
    assert g.choose_spec(16384, {"A_shape_1": 16384}, {}).width == 32      # many rows: wavefront teams
    with pytest.raises(ValueError):
        Spec("team", block=256, width=128)


def test_few_very_long_csr_rows_get_a_workgroup_each():
    g, _ = selfcheck_loop("spmv")
    arrays = {"A_data": np.zeros(37 * 40_000, np.float32)}       # ~40000 non-zeros per row on average
    sp = g.choose_spec(37, {}, arrays)
    assert (sp.width, sp.block) == (1024, 1024)



def test_while_break_continue_become_c_loops():
    src = (
        "#pragma parallel for\n"
        "for i in range(0, n, 1):\n"
        "    k = 0\n"
        "    while k < 10 and a[i] > 0.0:\n"
        "        k += 1\n"
        "        if k == 3:\n"
        "            continue\n"
        "        if k > 7:\n"
        "            break\n"
        "    out[i] = k\n"
    )
    a = np.zeros(8, np.float32)
    out = np.zeros(8, np.int64)
    f, code = compiled(src, n=8, a=a, out=out)
    k = body_of(f.kernel_for(f.choose_spec(8, {"n": 8}, {"a": a, "out": out})).src.text)
    assert "while (true) {" in k and "if (!(" in k and "continue;" in k and "break;" in k

    # `continue` directly in a parallel loop ends the iteration: a do/while(0) block per iteration,
    # and the store after it is not merged into a vector store
    skip = "#pragma parallel for simd\nfor i in range(0, n, 1):\n    if a[i] > 0.0:\n        continue\n    out[i] = 1\n"
    f2, _ = compiled(skip, n=8, a=a, out=out)
    k2 = body_of(f2.kernel_for(f2.default_spec).src.text)
    assert "do {" in k2 and "} while (0);" in k2 and "vstore" not in k2 and "continue;" not in k2
    assert ("out", 0, 0) in f2.analysis.guarded_checks
    # a parallel loop cannot be left
    bad = "#pragma parallel for\nfor i in range(0, n, 1):\n    if a[i] > 0.0:\n        break\n    out[i] = 1\n"
    with pytest.raises(NotImplementedError, match="break"):
        compiled(bad, n=8, a=a, out=out)


def test_guarded_loads_are_hoisted_only_when_the_host_can_vouch_for_them():
    from appy_amd.backends.hip.kernelgen import guarded_nodes
    import ast
    import dataclasses

    src = ("#pragma parallel for simd\nfor i in range(0, n, 1):\n"
           "    y[i] = (x[i - 1] if i > 0 else 0.0) + x[i] + (m[i] and x[i + 1] > 0.0)\n")
    x = np.zeros(64)
    m = np.zeros(64, bool)
    f, _ = compiled(src, n=64, x=x, y=x.copy(), m=m)
    assert ("x", 0, 0) in f.analysis.bound_checks and ("m", 0, 0) in f.analysis.bound_checks
    assert ("x", 0, -1) in f.analysis.guarded_checks and ("x", 0, 1) in f.analysis.guarded_checks
    assert ("x", 0, -1) not in f.analysis.bound_checks
    sp = f.default_spec
    fast = body_of(f.kernel_for(sp).src.text)
    safe = body_of(f.kernel_for(dataclasses.replace(sp, hoist_guarded=False)).src.text)
    assert fast.count("appy::vload<double") > safe.count("appy::vload<double") >= 1
    assert "x[(i - 1LL)]" in safe and "x[(i - 1LL)]" not in fast.split("__rest0")[0]
    assert dataclasses.replace(sp, hoist_guarded=False).tag().endswith("_g")

    tree = ast.parse("a[0] if c[1] else b[2]\nfor k in r:\n    d[3]\nwhile e[4]:\n    pass\nif g[5]:\n    h[6]\nz = p[7] and q[8]")
    names = {n.value.id for n in ast.walk(tree) if isinstance(n, ast.Subscript) and id(n) in guarded_nodes(tree.body)}
    assert names == {"a", "b", "d", "e", "h", "q"}


def test_bfloat16_tensors_follow_pytorch_promotion():
    torch = pytest.importorskip("torch")
    a = torch.zeros(8, dtype=torch.bfloat16)
    h = torch.zeros(8, dtype=torch.float16)
    w = torch.zeros(8, dtype=torch.float32)
    o = torch.zeros(8, dtype=torch.bfloat16)
    src = ("#pragma parallel for simd\nfor i in range(0, n, 1):\n"
           "    t = a[i] * 2.5 + 1\n"
           "    u = a[i] + h[i]\n"
           "    v = a[i] * w[i]\n"
           "    r = np.sqrt(a[i]) / a[i]\n"
           "    o[i] = max(t, a[i]) + u + v + r\n")
    f, code = compiled(src, n=8, a=a, h=h, w=w, o=o)
    k = body_of(code)
    assert "const __bf16* __restrict__ a" in k and "appy::vload<__bf16, 4>" in k
    assert "__bf16 t" in k and "float u" in k and "float v" in k and "__bf16 r" in k
    assert "(__bf16)(" in k and "sqrtf(" in k
    assert T.promote(T.BF16, T.WEAK_FLOAT) == T.BF16 and T.promote(T.BF16, T.I64) == T.BF16
    assert T.promote(T.BF16, T.from_dtype(np.float16)) == T.F32 and T.promote(T.F64, T.BF16) == T.F64
    assert T.BF16.size == 2 and T.BF16.is_float


def test_check_bounds_option_generates_a_kernel_that_cannot_leave_its_arrays():
    src = ("#pragma parallel for\nfor i in range(0, n, 1):\n    s = 0.0\n    #pragma simd\n"
           "    for j in range(lo[i], hi[i]):\n        s += v[j] * x[c[j]]\n    y[i + 1] = s\n")
    v = np.zeros(8, np.float32)
    c = np.zeros(8, np.int32)
    f, _ = cg.codegen(src, "kernel_loop_1", {"n": 4, "lo": c, "hi": c, "v": v, "x": v, "c": c, "y": v, "np": np},
                      {"check_bounds": True})
    sp = f.choose_spec(4, {"n": 4}, {"lo": c, "hi": c, "v": v, "x": v, "c": c, "y": v})
    assert sp.checked and sp.vec == 1 and sp.tag().endswith("_chk")
    ksrc = f.kernel_for(sp).src
    k = body_of(ksrc.text)
    assert "int* __oob" in k and "vload" not in k
    assert k.count("appy::at(") >= 5 and "appy::inside(" in k and "appy::report(__oob" in k
    assert set(ksrc.sites) == {"lo[i]", "hi[i]", "v[j]", "c[j]", "x[c[j]]", "y[i + 1]"}
    assert [p.role for p in ksrc.params].count("oob") == 1
    with pytest.raises(ValueError):
        Spec("flat", vec=4, checked=True)


def test_column_reductions_take_the_strip_shape():
    src = ("#pragma parallel for\nfor i in range(0, n, 1):\n    s = 0.0\n    m = -1e30\n"
           "    for j in range(0, r, 1):\n        s += A[j, i] * y[j]\n        m = max(m, A[j, i])\n"
           "    x[i] += beta * s + m\n")
    A = np.zeros((512, 300), np.float32)
    y = np.zeros(512, np.float32)
    x = np.zeros(300, np.float32)
    f, _ = compiled(src, n=300, r=512, A=A, y=y, x=x, beta=1.5)
    assert f.analysis.kind == "flat" and f.analysis.strip is not None
    sp = f.choose_spec(300, {"n": 300, "r": 512, "beta": 1.5}, {"A": A, "y": y, "x": x})
    assert (sp.kind, sp.block) == ("strip", 1024)
    assert f.grid_for(sp, 300) == 5
    k = body_of(f.kernel_for(sp).src.text)
    assert "__shared__ double __strip_slots[16][64];" in k
    assert "j += 16" in k and k.count("__syncthreads();") == 4 and "if (__wave == 0 && __active)" in k
    assert "appy::OpMax::f<float>(__part_m" in k and "if (__active) {" in k
    # short inner loops stay with one lane per iteration
    assert f.choose_spec(300, {"n": 300, "r": 8, "beta": 1.5}, {"A": A, "y": y, "x": x}).kind == "flat"
    # several shared-out loops, one of them under a sequential loop with the same bounds for every column
    multi = ("#pragma parallel for\nfor j in range(0, n, 1):\n    s = 0.0\n    #pragma simd\n    for c in range(0, r, 1):\n"
             "        s += Q[c, k] * A[c, j]\n    R[k, j] = s\n    for t in range(0, 3, 1):\n        #pragma simd\n"
             "        for c in range(0, r, 1):\n            A[c, j] = A[c, j] - Q[c, k] * s\n")
    Q = np.zeros((512, 300), np.float32)
    R = np.zeros((300, 300), np.float32)
    h, _ = compiled(multi, n=300, r=512, k=2, A=A, Q=Q, R=R)
    assert h.analysis.kind == "team" and len(h.analysis.strip) == 2
    hs = h.choose_spec(300, {"n": 300, "r": 512, "k": 2}, {"A": A, "Q": Q, "R": R})
    assert hs.kind == "strip"
    hk = body_of(h.kernel_for(hs).src.text)
    assert hk.count("c += 16") == 2 and "if (__wave == 0 && __active) { R[" in hk and hk.count("__syncthreads();") == 3
    # barriers under bounds or conditions that differ between columns: not a strip
    for bad in ("    for t in range(0, j, 1):\n        #pragma simd\n        for c in range(0, r, 1):\n            A[c, j] = A[c, j] * 2.0\n",
                "    if Q[0, j] > 0.0:\n        #pragma simd\n        for c in range(0, r, 1):\n            A[c, j] = A[c, j] * 2.0\n"):
        b, _ = compiled("#pragma parallel for\nfor j in range(0, n, 1):\n" + bad, n=300, r=512, A=A, Q=Q)
        assert b.analysis.strip is None
    # a running value that the loop looks at is not a column reduction
    g, _ = compiled("#pragma parallel for\nfor i in range(0, n, 1):\n    s = 0.0\n    for j in range(0, r, 1):\n"
                    "        s = s * 0.5 + A[j, i]\n    x[i] = s\n", n=300, r=512, A=A, x=x)
    assert g.analysis.strip is None


def test_triangular_simd_loops_get_teams_sized_by_their_mean_length():
    src = ("#pragma parallel for\nfor i in range(0, n, 1):\n    #pragma simd\n    for j in range(0, i + 1, 1):\n"
           "        C[i, j] = C[i, j] * beta\n")
    C = np.zeros((1200, 1200))
    f, _ = compiled(src, n=1200, C=C, beta=1.2)
    assert f.choose_spec(1200, {"n": 1200, "beta": 1.2, "__appy_mid": 600}, {"C": C}).width == 32
    assert f.choose_spec(1200, {"n": 1200, "beta": 1.2}, {"C": C}).width == 32     # nothing known: a middling team (64 / V)
    assert f.choose_spec(16, {"n": 16, "beta": 1.2, "__appy_mid": 8}, {"C": C}).width == 8


def test_small_element_types_move_16_bytes_per_lane_too():
    a8 = np.zeros(64, np.uint8)
    f, src = compiled("#pragma parallel for simd\nfor i in range(n):\n    c[i] = a[i] + b[i]", c=a8.copy(), a=a8, b=a8, n=64)
    assert f.default_spec.vec == 16 and "appy::vload<unsigned char, 16>" in body_of(src) and ".sf" in body_of(src)
    a16 = np.zeros(64, np.float16)
    g, src = compiled("#pragma parallel for simd\nfor i in range(n):\n    c[i] = a[i] * 2", c=a16.copy(), a=a16, n=64)
    assert g.default_spec.vec == 8 and "appy::vstore<_Float16, 8>" in body_of(src)
    # the widest element decides: a byte mask next to float32 data keeps 4 elements per lane
    m = np.zeros(64, bool)
    x = np.zeros(64, np.float32)
    h, _ = compiled("#pragma parallel for simd\nfor i in range(n):\n    c[i] = x[i] if m[i] else 0.0", c=x.copy(), x=x, m=m, n=64)
    assert h.default_spec.vec == 4


def test_updates_of_elements_shared_between_iterations_are_atomic():
    h = np.zeros(16, np.int64)
    b = np.zeros(64, np.int32)
    w = np.zeros(64, np.float32)
    f, src = compiled("#pragma parallel for simd\nfor i in range(n):\n    hist[b[i]] += 1\n    top[0, b[i]] = max(top[0, b[i]], w[i])\n"
                      "    own[i] += w[i]\n", hist=h, b=b, w=w, top=np.zeros((1, 16), np.float32), own=w.copy(), n=64)
    k = body_of(src)
    assert "appy::atomic_combine<appy::OpAdd, long long>::run(&hist[" in k
    assert "appy::atomic_combine<appy::OpMax, float>::run(&top[" in k
    assert "atomic_combine<appy::OpAdd, float>" not in k and "vstore<float, 2>(own" in k     # own[i] belongs to the iteration
    g, src = compiled("#pragma parallel for\nfor i in range(n):\n    #pragma simd\n    for j in range(m):\n        col[j] -= A[i, j]\n",
                      col=np.zeros(32), A=np.zeros((8, 32)), n=8, m=32)
    assert "appy::atomic_combine<appy::OpAdd, double>::run(&col[" in body_of(src) and "(-" in body_of(src)
    # 8- and 16-bit elements: compare-and-swap on the 32-bit word that holds the element
    h16, src = compiled("#pragma parallel for simd\nfor i in range(n):\n    hist[b[i]] += 1\n    seen[b[i]] = seen[b[i]] or True\n",
                        hist=np.zeros(16, np.int16), seen=np.zeros(16, bool), b=b, n=64)
    assert "appy::atomic_combine<appy::OpAdd, short>::run(&hist[" in body_of(src)
    assert "appy::atomic_combine<appy::OpMax, unsigned char>::run(&seen[" in body_of(src)


def test_in_place_slice_update_from_a_shifted_slice_of_the_same_row_is_refused():
    A = np.zeros((8, 16))
    B = np.zeros((8, 16))
    with pytest.raises(RuntimeError, match="another offset"):
        compiled("#pragma parallel for\nfor i in range(n):\n    A[i, 1:] = 0.5 * (A[i, :-1] + B[i, :-1])\n", A=A, B=B, n=8)
    # same offsets, other rows, other arrays: fine
    compiled("#pragma parallel for\nfor i in range(1, n):\n    A[i, 1:] = A[i, 1:] + A[i - 1, :-1] + B[i, :-1]\n", A=A, B=B, n=8)


def test_clear_cache_option_regenerates_the_loop():
    a = np.zeros(8, np.float32)
    src = "#pragma parallel for simd\nfor i in range(n):\n    a[i] = 1.0"
    f1, _ = cg.codegen(src, "kernel_loop_1", {"a": a, "n": 8}, {})
    f2, _ = cg.codegen(src, "kernel_loop_1", {"a": a, "n": 8}, {})
    f3, _ = cg.codegen(src, "kernel_loop_1", {"a": a, "n": 8}, {"clear_cache": True})
    assert f1 is f2 and f3 is not f1


def test_generated_code_objects_hold_no_packed_fp32_instructions():
    """Kernels are compiled with the packed-fp32 feature switched off; the ISA of a
    float-heavy generated kernel (own code object) must show none of those forms."""
    import os
    import re
    import subprocess
    import tempfile

    objdump = "/opt/rocm/llvm/bin/llvm-objdump"
    if not os.path.exists(objdump):
        pytest.skip("llvm-objdump not found")
    x = np.zeros(64, np.float32)
    src = ("#pragma parallel for simd\nfor i in range(n):\n    xi = x[i]\n    x3 = xi * xi * xi\n"
           "    y[i] = 0.5 * xi * (1 + 0.044715 * x3) + xi * 2.0 + x3 * 3.0 + z[i] * xi\n")
    f, _ = compiled(src, x=x, y=x.copy(), z=x.copy(), n=64)
    with tempfile.NamedTemporaryFile(suffix=".co") as fh:
        fh.write(f.kernels[f.default_spec].code)
        fh.flush()
        isa = subprocess.run([objdump, "-d", fh.name], capture_output=True, text=True, check=True).stdout
    assert "v_mul_f32" in isa or "v_fma" in isa or "v_add_f32" in isa
    assert not re.search(r"v_pk_(add|mul|fma)_f32", isa)
    assert "global_load_dwordx4" in isa and "global_store_dwordx4" in isa


def test_byte_multiply_add_chains_are_not_folded_into_dot_products():
    """Kernels are compiled without the 8-bit dot-product instructions: the compiler's fold of
    `u * u + max(u, u * u)` over uint8 into v_dot4_u32_u8 computed another value (and the
    16-byte form of the loop crashed instruction selection).  The loop must compile and its ISA
    must keep the maximum."""
    import os
    import subprocess
    import tempfile

    objdump = "/opt/rocm/llvm/bin/llvm-objdump"
    if not os.path.exists(objdump):
        pytest.skip("llvm-objdump not found")
    u = np.zeros(64, np.uint8)
    src = "#pragma parallel for simd\nfor i in range(n):\n    out[i] = (-(u[i] * u[i])) - max((u[i] * u[i]), u[i])\n"
    for dt in (np.uint8, np.float64):
        f, _ = compiled(src, u=u, out=np.zeros(64, dt), n=64)
        with tempfile.NamedTemporaryFile(suffix=".co") as fh:
            fh.write(f.kernels[f.default_spec].code)
            fh.flush()
            isa = subprocess.run([objdump, "-d", fh.name], capture_output=True, text=True, check=True).stdout
        assert "v_dot4" not in isa and "v_max_u" in isa


def test_independent_inner_loops_collapse_into_the_parallel_loop():
    """`parallel i / for j / simd k` with few `i`: when the `j` iterations are provably
    independent the pairs (i, j) become the iteration space of the team kernel."""
    A, B = np.zeros((20, 22, 70)), np.zeros((20, 22, 70))
    env = dict(A_shape_0=20, A_shape_1=22, A_shape_2=70)
    stencil = ("#pragma parallel for\nfor i in range(1, A_shape_0 - 1):\n    for j in range(1, A_shape_1 - 1):\n"
               "        #pragma simd\n        for k in range(1, A_shape_2 - 1):\n"
               "            B[i, j, k] = A[i, j, k - 1] + A[i, j + 1, k] + A[i - 1, j, k]\n")
    f, _ = compiled(stencil, A=A, B=B, **env)
    assert f.analysis.collapse is not None
    spec = f.choose_spec(18, dict(env), dict(A=A, B=B))
    assert spec.kind == "team" and spec.collapse
    k = body_of(f.kernel_for(spec).src.text)
    assert "__c < (__hi - __lo) * __nj" in k and "const appy::i64 i = __lo + (__c) / __nj;" in k
    assert "const appy::i64 j = __jlo + (__c) % __nj;" in k and "for (appy::i64 j" not in k
    # many parallel iterations: nothing to gain
    assert not f.choose_spec(20000, dict(env, A_shape_0=20002), dict(A=A, B=B)).collapse

    def collapsible(body, **extra):
        src = "#pragma parallel for\nfor i in range(n):\n    for j in range(m):\n" + body
        g, _ = compiled(src, A=A, B=B, y=np.zeros((20, 22)), n=20, m=22, p=70, **extra)
        return g.analysis.collapse is not None

    simd = "        #pragma simd\n        for k in range(p):\n"
    assert collapsible("        s = 0.0\n" + simd + "            s += A[i, j, k]\n        y[i, j] = s\n")
    # a value carried from one j to the next
    assert not collapsible("        s = y[i, 0]\n" + simd + "            s += A[i, j, k]\n        y[i, 0] = s\n")
    # the loop reads a slab that another j writes
    assert not collapsible(simd + "            A[i, j, k] = A[i, j - 1, k] + 1.0\n")
    # a scalar that lives across iterations of j
    assert not collapsible(simd + "            B[i, j, k] = A[i, j, k] + t\n        t = t + 1.0\n", t=0.5)
    # leaving the loop early
    assert not collapsible("        if y[i, j] > 0:\n            break\n" + simd + "            B[i, j, k] = A[i, j, k]\n")
    # bounds that depend on the parallel variable
    src = "#pragma parallel for\nfor i in range(n):\n    for j in range(i):\n" + simd + "            B[i, j, k] = A[i, j, k]\n"
    g, _ = compiled(src, A=A, B=B, n=20, p=70)
    assert g.analysis.collapse is None


def test_rows_that_an_iteration_reads_twice_are_not_loaded_non_temporally():
    from appy_amd.backends.hip.kernelgen import Spec

    x = np.zeros((8, 64), np.float32)
    src = ("#pragma parallel for\nfor i in range(n):\n    m = -1e30\n    #pragma simd\n    for k in range(p):\n"
           "        m = max(m, x[i, k])\n    s = 0.0\n    #pragma simd\n    for k in range(p):\n"
           "        s += np.exp(x[i, k] - m)\n    #pragma simd\n    for k in range(p):\n        out[i, k] = w[i, k] / s\n")
    f, _ = compiled(src, x=x, w=x.copy(), out=x.copy(), n=8, p=64)
    assert f.analysis.reread == {"x"}
    k = body_of(f.kernel_for(Spec("team", block=256, vec=4, width=16, stream_loads=True)).src.text)
    assert "appy::vload<float, 4>(x +" in k and "vload_stream<float, 4>(x +" not in k
    assert "appy::vload_stream<float, 4>(w +" in k          # read once: streams past the caches


def test_rows_without_slices_and_reductions_spelled_as_methods_are_lowered_to_simd_loops():
    import ast

    from appy_amd.backends.hip import array_expr
    from appy_amd.frontend import loop_ir

    A, x, out = np.zeros((4, 9)), np.zeros(9), np.zeros(4)
    src = ("#pragma parallel for\nfor i in range(n):\n    B[i] = A[i] * 2\n    out[i] = A[i].mean() + np.dot(A[i], x)\n"
           "    k[i] = np.argmax(A[i, :])\n")
    tree, shapes = array_expr.transform(loop_ir.build(src), dict(A=A, B=A.copy(), x=x, out=out, k=np.zeros(4, np.int64), n=4, np=np))
    text = ast.unparse(tree)
    assert "B[i, __c1] = A[i, __c1] * 2" in text                       # the row, element by element
    assert "__r2 = __r2 + A[i, __c3]" in text and "/ A_shape_1" in text     # mean = sum / extent
    assert "A[i, __c5] * x[__c5]" in text                               # np.dot of two 1-D operands
    assert "max(__r" in text and "if A[i, __c" in text and "== __r" in text      # argmax: the maximum, then its first position
    assert ("A", 1) in shapes
    # and the whole nest compiles
    f, _ = compiled(src, A=A, B=A.copy(), x=x, out=out, k=np.zeros(4, np.int64), n=4)
    assert f.analysis.kind == "team"


def test_two_phase_shapes_need_set_up_statements_that_can_be_repeated():
    """Statements in front of a split loop run once per part and again in the finishing kernel;
    a nest whose set-up reads what the loop stores keeps to one kernel."""
    A = np.zeros((4, 100000))
    rows = "#pragma parallel for\nfor i in range(n):\n    f = {first}\n    #pragma simd\n    for j in range(m):\n        C[i, j] = A[i, j] * f\n"
    f, _ = compiled(rows.format(first="A[i, 0]"), A=A, C=A.copy(), n=4, m=100000)
    assert f.analysis.team_split is not None
    f, _ = compiled(rows.format(first="C[i, 0]"), A=A, C=A.copy(), n=4, m=100000)
    assert f.analysis.team_split is None
    cols = "#pragma parallel for\nfor j in range(m):\n    f = {first}\n    for i in range(n):\n        C[i, j] = A[i, j] * f\n"
    f, _ = compiled(cols.format(first="A[0, j]"), A=A, C=A.copy(), n=4, m=100000)
    assert f.analysis.strip_split is not None
    f, _ = compiled(cols.format(first="C[0, j]"), A=A, C=A.copy(), n=4, m=100000)
    assert f.analysis.strip is not None and f.analysis.strip_split is None


def test_store_loops_of_multi_wavefront_teams_wait_for_the_set_up_reads():
    from appy_amd.backends.hip.kernelgen import Spec

    A = np.zeros((100, 256))
    cols = "#pragma parallel for\nfor j in range(m):\n    f = {first}\n    for i in range(n):\n        C[i, j] = A[i, j] * f\n"
    f, _ = compiled(cols.format(first="C[0, j]"), A=A, C=A.copy(), n=100, m=256)
    k = body_of(f.kernel_for(Spec("strip", block=256, vec=1, unroll=8)).src.text)
    assert k.index("f = C[") < k.index("__syncthreads();   // every wavefront has read") < k.index("C[i * C_stride_0 + j] =")
    f, _ = compiled(cols.format(first="A[0, j]"), A=A, C=A.copy(), n=100, m=256)
    assert "every wavefront has read" not in f.kernel_for(Spec("strip", block=256, vec=1, unroll=8)).src.text
    rows = "#pragma parallel for\nfor i in range(n):\n    f = C[i, 0]\n    #pragma simd\n    for j in range(m):\n        C[i, j] = A[i, j] * f\n"
    g, _ = compiled(rows, A=A, C=A.copy(), n=100, m=256)
    assert "every wavefront has read" in g.kernel_for(Spec("team", block=256, vec=2, width=256)).src.text
    assert "every wavefront has read" not in g.kernel_for(Spec("team", block=256, vec=2, width=64)).src.text


def test_rows_that_several_simd_loops_read_stay_in_registers():
    """Soft-max and layer-norm nests: when a row is a whole, small number of vector steps per
    lane, the first simd loop loads it into registers and the later ones read it from there."""
    x = np.zeros((64, 1024), np.float32)
    g = np.zeros(1024, np.float32)
    src = ("#pragma parallel for\nfor i in range(n):\n    s = 0.0\n    #pragma simd\n    for j in range(d):\n        s += x[i, j]\n"
           "    mu = s / d\n    v = 0.0\n    #pragma simd\n    for j in range(d):\n        v += (x[i, j] - mu) * (x[i, j] - mu)\n"
           "    r = 1.0 / np.sqrt(v / d + 1e-5)\n    #pragma simd\n    for k in range(x_shape_1):\n"
           "        out[i, k] = (x[i, k] - mu) * r * g[k]\n")
    env = dict(n=64, d=1024, x_shape_1=1024)
    f, _ = compiled(src, x=x, g=g, out=x.copy(), **env)
    assert f.analysis.row_cache is not None and f.analysis.row_cache[1] == {"x"}
    assert len(f.analysis.row_cache[2]) == 2            # two spellings of the bounds, compared at the launch
    spec = f.choose_spec(64, dict(env), dict(x=x, g=g, out=x))
    assert spec.kind == "team" and spec.width == 64 and spec.row_steps == 4 and spec.tag().endswith("_rc4")
    k = body_of(f.kernel_for(spec).src.text)
    assert k.count("appy::vload<float, 4>(x +") == 1 and k.count("__rc0[__k] = ") == 1
    assert k.count(" = __rc0[__k];") == 3 and "appy::vload<float, 4>(g +" in k
    assert "for (int __k = 0; __k < 4; ++__k)" in k
    # a row that is not a whole number of steps, or too many of them: the loops as before
    assert f.choose_spec(64, dict(env, d=1000, x_shape_1=1000), dict(x=x, g=g, out=x)).row_steps == 0
    assert f.choose_spec(64, dict(env, d=1024, x_shape_1=512), dict(x=x, g=g, out=x)).row_steps == 0
    # rows too long for a wavefront's registers go to a workgroup each
    long = f.choose_spec(4096, dict(env, n=4096, d=8192, x_shape_1=8192), dict(x=np.zeros((4096, 8192), np.float32), g=g, out=x))
    assert long.row_steps == 8 and long.width == long.block == 256
    # a row that the nest stores to is read from memory every time
    upd = ("#pragma parallel for\nfor i in range(n):\n    s = 0.0\n    #pragma simd\n    for j in range(d):\n        s += x[i, j]\n"
           "    #pragma simd\n    for j in range(d):\n        x[i, j] = x[i, j] / s\n")
    h, _ = compiled(upd, x=x, n=64, d=1024)
    assert h.analysis.row_cache is None


def test_simd_loops_of_a_wavefront_team_are_fenced_when_they_touch_stored_arrays():
    """Two simd loops of an iteration may touch the same elements from different lanes (slices
    that overlap): the compiler sees only each lane's own, distinct addresses and could reorder
    them across the loops, so a wavefront-scope fence separates the loops."""
    from appy_amd.backends.hip.kernelgen import Spec

    A = np.zeros((23, 61))
    src = ("#pragma parallel for\nfor i in range(n):\n    #pragma simd\n    for j in range(16):\n        A[i, 18 + j] = B[i, 24 + j] - alpha\n"
           "    #pragma simd\n    for j in range(16):\n        A[i, 12 + j] = B[i, 44 + j] * alpha\n")
    f, _ = compiled(src, A=A, B=A.copy(), n=23, alpha=1.25)
    k = body_of(f.kernel_for(Spec("team", block=256, vec=2, width=4)).src.text)
    assert k.count("appy::wave_fence();") == 2
    assert k.index("A + (i * A_stride_0 + (18LL") < k.index("appy::wave_fence();") < k.index("A + (i * A_stride_0 + (12LL")
    # one lane per iteration: program order; several wavefronts: a workgroup barrier
    assert "wave_fence" not in f.kernel_for(Spec("team", block=256, vec=2, width=1)).src.text.split('extern "C"')[1]
    wide = body_of(f.kernel_for(Spec("team", block=256, vec=2, width=256)).src.text)
    assert "wave_fence" not in wide and "__syncthreads();" in wide
    # loops that only read arrays nothing stores to need none
    src = ("#pragma parallel for\nfor i in range(n):\n    s = 0.0\n    #pragma simd\n    for j in range(m):\n        s += B[i, j]\n"
           "    t = 0.0\n    #pragma simd\n    for j in range(m):\n        t += B[i, j] * B[i, j]\n    y[i] = s * t\n")
    g, _ = compiled(src, B=A, y=np.zeros(23), n=23, m=61)
    assert "wave_fence();" not in body_of(g.kernel_for(Spec("team", block=256, vec=2, width=16)).src.text)


def test_rows_whose_bounds_read_what_the_body_stores_are_not_sorted_by_length():
    """`for j in range(ln[i]): ...; ln[i] = 0` is a legal loop, but the kernels over sorted rows evaluate the bounds
    of a row more than once: such a nest keeps one team width for all rows."""
    ln = np.zeros(8, np.int32)
    v = np.zeros(64, np.float32)
    y = np.zeros(8, np.float32)
    src = ("#pragma parallel for\nfor i in range(m):\n    s = 0.0\n    #pragma simd\n    for j in range(ln[i]):\n"
           "        s += v[i * 8 + j]\n    y[i] = s\n")
    f, _ = compiled(src, ln=ln, v=v, y=y, m=8)
    assert f.analysis.ragged is not None
    g, _ = compiled(src + "    ln[i] = 0\n", ln=ln, v=v, y=y, m=8)
    assert g.analysis.team_split is not None and g.analysis.ragged is None
    assert g.choose_spec(1 << 20, {"m": 1 << 20}, {"v": v}).rows == ""


def test_row_plans_kernel_that_writes_the_pairs_and_kernel_that_runs_a_plan():
    """The two generated kernels of the kept order of elements: one (key, value) pair per element with the
    checks that make an inspector refuse its input; tiles of products dropped into row-sorted slots in LDS and
    added to per-row sums without atomics, every load issued from a scalar base plus a fixed lane offset."""
    f, _ = selfcheck_loop("spmv")
    keys = body_of(f.kernel_for(Spec("team", block=256, vec=1, width=64, aux="rkeys", block_rows=256)).src.text)
    assert "__lp[__r + 1] == __hq[__r]" in keys and "__flag[0] = 1" in keys
    assert "const bool __in = __cq >= 0 && __cq < __nx;" in keys and "if (__j + __q < __end && !__in) __inside = false;" in keys
    assert "appy::vstore<unsigned, 4>(__keys + __j, __kq);" in keys         # four pairs of a lane leave as vectors
    assert "__kq[__q] = ((__rel >> 15) << __lbits) | ((unsigned)__cq >> 5);" in keys
    assert "x[" not in keys.split("{", 1)[1]                                  # the gathered operand is not read here
    for unroll, tile in ((6, 6144), (4, 4096)):
        run = body_of(f.kernel_for(Spec("team", block=1024, vec=1, width=1024, unroll=unroll, parts=8, aux="xcells")).src.text)
        assert f"__shared__ float __sum[32768];" in run and f"__prod[{tile}];" in run
        assert "atomicAdd" not in run and run.count("__syncthreads();") >= 3
        assert "(__cv * __cx)" in run and "A_indptr[" not in run.split("{", 1)[1] and "A_indices[" not in run.split("{", 1)[1]
        assert "__builtin_amdgcn_readfirstlane" in run
        # one sequence of tiles over all the runs of a workgroup: the next run is entered where the loads are issued, and
        # the sums of a run that is through go out inside the loop over the tiles
        assert "while (__any0) {" in run and "__vi += gridDim.x; __vc = __vi < __norder ? __order[__vi] : 0xffffffffu; __tt = 0;" in run
        assert "if (__end0) {" in run
        assert "const unsigned* __restrict__ __cstart" in run.split("{", 1)[0] or "__restrict__ __cstart" in f.kernel_for(
            Spec("team", block=1024, vec=1, width=1024, unroll=unroll, parts=8, aux="xcells")).src.text
    with pytest.raises(ValueError):
        Spec("team", block=1024, vec=1, width=1024, unroll=8, parts=8, aux="xcells")
    # the shape of a plan for the benchmark's matrices: 128 blocks of rows x 8 column ranges, 19 bits of column, tiles of 6144
    arrays = {"A_data": np.broadcast_to(np.float32(0), (16 << 22,)), "A_indices": np.broadcast_to(np.int32(0), (16 << 22,)),
              "A_indptr": np.broadcast_to(np.int32(0), ((1 << 22) + 1,)), "x": np.broadcast_to(np.float32(0), (1 << 22,))}
    shape = f.plan_shape(1 << 22, {"M": 1 << 22}, arrays)
    assert (shape.row_blocks, shape.groups, shape.group_width, shape.col_bits, shape.tile, shape.line_bits) == (128, 8, 1 << 19, 19, 6144, 17)
    assert f.plan_arrays() == ["A_indptr", "A_indices", "A_data"]
    arrays["x"] = np.broadcast_to(np.float32(0), (7 << 20,))
    shape = f.plan_shape(1 << 22, {"M": 1 << 22}, arrays)
    assert (shape.col_bits, shape.tile) == (20, 4096)
    arrays["x"] = np.broadcast_to(np.float32(0), (1 << 19,))                  # an operand that every L2 holds anyway
    assert f.plan_shape(1 << 22, {"M": 1 << 22}, arrays) is None


def test_runs_of_a_row_plan_are_dealt_by_size():
    """How many workgroups share a cell follows from the sizes of the cells, and the runs are dealt to the workgroups
    of their column range largest first, back and forth: every run exactly once, every workgroup its own range only,
    about the same number of tiles each."""
    rng = np.random.default_rng(0)
    # the uniform matrix of the benchmark: 1024 cells of 11 tiles, four per workgroup as they come
    tiles = np.full(1024, 11)
    assert cg.plan_split(tiles, 256, 6144, 16 << 22) == 1
    order = cg.deal_runs(tiles, 1, 256)
    assert len(order) == 1024 and sorted(order.tolist()) == list(range(1024))
    assert all((int(order[w + 256 * i]) & 7) == (w & 7) for w in range(256) for i in range(4))
    # a banded matrix: one cell of each block of rows holds all of its 86 tiles - two workgroups share a cell
    tiles = np.zeros(1024, dtype=np.int64)
    blocks = np.arange(128)
    tiles[blocks * 8 + blocks * 8 // 128] = 86
    assert cg.plan_split(tiles, 256, 6144, 16 << 22) == 2
    assert cg.plan_split(tiles, 256, 6144, 16 << 22, forced=4) == 4
    order = cg.deal_runs(tiles, 2, 256)
    runs = order[order != 0xFFFFFFFF]
    assert sorted(runs.tolist()) == list(range(2048))                      # runs without tiles are dealt too
    size = lambda vc: (lambda b, part, g: ((part + 1) * tiles[b * 8 + g]) // 2 - (part * tiles[b * 8 + g]) // 2)((vc >> 3) // 2, (vc >> 3) % 2, vc & 7)
    load = np.zeros(256, dtype=np.int64)
    for p, vc in enumerate(order.tolist()):
        if vc != 0xFFFFFFFF:
            assert (vc & 7) == (p % 256) & 7
            load[p % 256] += size(vc)
    assert load.sum() == tiles.sum() and load.max() == 43 and load.min() == 43
    # cells of random sizes: no workgroup far above the mean, lists without holes
    tiles = rng.integers(0, 200, 1024)
    split = cg.plan_split(tiles, 256, 6144, int(tiles.sum()) * 6144)
    order = cg.deal_runs(tiles, split, 256)
    load = np.zeros(256, dtype=np.int64)
    for p, vc in enumerate(order.tolist()):
        if vc != 0xFFFFFFFF:
            b, part, g = (vc >> 3) // split, (vc >> 3) % split, vc & 7
            load[p % 256] += ((part + 1) * tiles[b * 8 + g]) // split - (part * tiles[b * 8 + g]) // split
            assert p < 256 or order[p - 256] != 0xFFFFFFFF
    assert load.sum() == tiles.sum() and load.max() <= 1.15 * load.mean()
    # few cells: several workgroups per cell, a workgroup per run
    tiles = np.full(16, 40)
    split = cg.plan_split(tiles, 256, 6144, 16 * 40 * 6144)
    assert split == 20                                                     # until a run is down to two tiles
    order = cg.deal_runs(tiles, split, min(16 * split, 256) // 8 * 8)
    assert sorted(order[order != 0xFFFFFFFF].tolist()) == list(range(16 * split))


def test_launch_shapes_follow_the_device_they_are_for():
    """Grids and the forms that pin stripes of a gathered operand to XCDs are sized from what the runtime reports of
    the device (compute units, XCDs, L2 per XCD), not from literals: another device, other shapes."""
    small = cg.Hardware(cus=64, xcds=4, l2_bytes=2 << 20, mall_bytes=32 << 20)
    assert cg.MI355X == cg.Hardware(cus=256, xcds=8, l2_bytes=4 << 20, mall_bytes=256 << 20)
    assert (cg.MI355X.stripe_bytes, cg.MI355X.stripe_min_bytes, small.stripe_bytes) == (2 << 20, 3 << 20, 1 << 20)
    # a streaming reduction: non-temporal loads from the size of the memory-side cache on
    f, _ = compiled("#pragma parallel for simd shared(s)\nfor i in range(n):\n    s[0] += a[i]", s=np.zeros(1), a=np.zeros(8, np.float32), n=8)
    arrays = {"s": np.zeros(1), "a": np.broadcast_to(np.float32(0), (1 << 24,))}
    assert not f.choose_spec(1 << 24, {}, arrays).stream_loads and f.choose_spec(1 << 24, {}, arrays, hw=small).stream_loads
    # few, very long rows: a workgroup per row up to as many rows as there are compute units
    g, _ = selfcheck_loop("gemv")
    rows = {"A": np.broadcast_to(np.float32(0), (128, 1 << 20)), "x": np.broadcast_to(np.float32(0), (1 << 20,)),
            "y": np.broadcast_to(np.float32(0), (128,))}
    env = {"A_shape_0": 128, "A_shape_1": 1 << 20}
    big, little = g.choose_spec(128, env, rows), g.choose_spec(128, env, rows, hw=small)
    assert (big.block, big.phase) == (1024, 1) and (little.block, little.phase) == (256, 0)
    assert g.team_parts(big, 128, env, rows) == 4 and g.team_parts(big, 128, env, rows, hw=small) == 1
    assert g.grid_for(f.default_spec, 1 << 30, cus=64) < g.grid_for(f.default_spec, 1 << 30)
    # stripes per XCD: only where the kernels' mapping of workgroups to XCDs holds (eight of them)
    sp, _ = selfcheck_loop("spmv")
    csr = {"A_data": np.broadcast_to(np.float32(0), (16 << 20,)), "A_indices": np.broadcast_to(np.int32(0), (16 << 20,)),
           "A_indptr": np.broadcast_to(np.int32(0), ((1 << 20) + 1,)), "x": np.broadcast_to(np.float32(0), (1 << 20,))}
    assert sp.grouped_shape(1 << 20, {"M": 1 << 20}, csr)[0] == 8
    assert sp.grouped_shape(1 << 20, {"M": 1 << 20}, csr, hw=small) is None and sp.plan_shape(1 << 20, {"M": 1 << 20}, csr, hw=small) is None
    double = cg.Hardware(cus=256, xcds=8, l2_bytes=8 << 20)
    assert sp.grouped_shape(1 << 20, {"M": 1 << 20}, csr, hw=double) is None       # 4 MiB stay in an 8 MiB L2 as a whole
    csr["x"] = np.broadcast_to(np.float32(0), (4 << 20,))
    assert sp.grouped_shape(1 << 20, {"M": 1 << 20}, csr, hw=double)[0] == 8
