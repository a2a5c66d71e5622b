"""CPU tests of the @kernel translator: typing rules, generated source, error
reporting, and that the generated HIP compiles for gfx950 (no GPU needed)."""

import math
import os
import re
import subprocess

import numpy as np
import pytest

from numba_mlir_amd.mlir import kernel_compiler as kc


@pytest.fixture(scope="module")
def K(native_libs):
    from numba_mlir_amd.mlir import kernel_impl
    return kernel_impl


F32_1D = kc.Array(kc.FLOAT32, 1)
F64_1D = kc.Array(kc.FLOAT64, 1)
I32_1D = kc.Array(kc.INT32, 1)
I64_1D = kc.Array(kc.INT64, 1)


def source_of(K, func, types, ndim=1, **kw):
    return kc.translate(func, types, ndim, K, **kw).source


def declared_type(src, name):
    m = re.search(r"^\s*([\w:<>, ]+?) v_%s = " % name, src, re.M)
    assert m, f"{name} is not declared in\n{src}"
    return m.group(1).strip()


def test_argument_types():
    class Dev:
        dtype, ndim, elem_strides = np.dtype(np.float32), 2, (4, 1)

    assert kc.type_of_argument(Dev()) == kc.Array(kc.FLOAT32, 2)
    assert kc.type_of_argument(3) is kc.INT64
    assert kc.type_of_argument(3.0) is kc.FLOAT64
    assert kc.type_of_argument(True) is kc.BOOL
    assert kc.type_of_argument(np.int32(3)) is kc.INT32
    assert kc.type_of_argument(np.float32(3)) is kc.FLOAT32
    assert isinstance(kc.type_of_argument(slice(1, 2)), kc.SliceArg)
    with pytest.raises(kc.KernelCompileError):
        kc.type_of_argument("text")


def test_promotion_follows_numpy():
    assert kc.promote(kc.INT32, kc.FLOAT32) is kc.FLOAT64
    assert kc.promote(kc.INT32, kc.INT64) is kc.INT64
    assert kc.promote(kc.FLOAT32, kc.FLOAT32) is kc.FLOAT32
    assert kc.promote(kc.INT16, kc.FLOAT32) is kc.FLOAT32
    assert kc.promote(kc.BOOL, kc.INT8) is kc.INT8


def test_variable_types(K):
    get_global_id = K.get_global_id

    def func(a, f, out):
        i = get_global_id(0)
        lit_i = 7                  # int64
        lit_f = 0.5                # float64
        x = a[i] + lit_i           # int32 + int64 -> int64
        y = f[i] * f[i]            # float32
        z = f[i] + lit_f           # float32 + float64 -> float64
        q = a[i] / a[i]            # true division -> float64
        r = a[i] // 2              # int64 (literal)
        acc = 0                    # int64, then widened by the float32 store
        acc = acc + y
        b = a[i] > 2 and not y < 1.0
        out[i] = x + y + z + q + r + acc + b

    src = source_of(K, func, [I32_1D, F32_1D, F64_1D])
    assert declared_type(src, "i") == "int64_t"
    assert declared_type(src, "x") == "int64_t"
    assert declared_type(src, "y") == "float"
    assert declared_type(src, "z") == "double"
    assert declared_type(src, "q") == "double"
    assert declared_type(src, "r") == "int64_t"
    assert declared_type(src, "acc") == "double"      # int64 joined with float32
    assert declared_type(src, "b") == "bool"
    # a name bound once, at the top level, to a constant is used as that constant
    assert "+ ((int64_t)7ll))" in src and "+ v_lit_i" not in src


def test_known_non_negative_indices_need_no_wrap(K):
    get_global_id, get_local_id = K.get_global_id, K.get_local_id

    def func(a, out):
        i = get_global_id(0)
        j = i + get_local_id(0) * 2
        k = i - 1
        out[i] = a[j] + a[k] + a[-1] + a[i % 4]

    src = source_of(K, func, [F32_1D, F32_1D])
    body = src.split("if (nmk_active)")[1]
    assert body.count("nmkjit::wrap(") == 1            # only a[k]
    assert "v_a.shape[0] + ((int64_t)-1ll)" in body     # a[-1]


def test_kernel_signature_matches_the_launch_abi(K):
    get_global_id, local, barrier = K.get_global_id, K.local, K.barrier

    def func(a, n, s, b):
        lm = local.array((4, 8), np.float64)
        i = get_global_id(0)
        lm[0, 0] = a[i, 0]
        barrier()
        b[s][i] = lm[0, 0] + n

    ck = kc.translate(func, [kc.Array(kc.FLOAT32, 2), kc.INT64, kc.SliceArg(), F64_1D], 1, K)
    sig = ck.source[ck.source.index("void " + ck.name):ck.source.index(") {")]
    params = [p.strip() for p in sig.split("(", 1)[1].split(",")]
    assert params == [
        "float *v_a_p", "int64_t v_a_s0", "int64_t v_a_s1", "int64_t v_a_t0", "int64_t v_a_t1",
        "int64_t v_n", "int64_t v_s_start", "int64_t v_s_stop", "int64_t v_s_step",
        "double *v_b_p", "int64_t v_b_s0", "int64_t v_b_t0",
        "uint64_t nmk_lds0", "int64_t nmk_gsz0", "int64_t nmk_gsz1", "int64_t nmk_gsz2"]
    assert ck.local_bytes == [4 * 8 * 8]
    assert ck.name.startswith("nmkjit_func_")
    # same body, same name; another signature, another name
    assert kc.translate(func, [kc.Array(kc.FLOAT32, 2), kc.INT64, kc.SliceArg(), F64_1D],
                        1, K).name == ck.name
    assert kc.translate(func, [kc.Array(kc.FLOAT64, 2), kc.INT64, kc.SliceArg(), F64_1D],
                        1, K).name != ck.name


def test_bounds_checked_build_adds_the_flag(K):
    get_global_id = K.get_global_id

    def helper(a, i):
        return a[i]

    def func(a, b):
        i = get_global_id(0)
        b[i] = helper(a, i + 1)

    plain = source_of(K, func, [F32_1D, F32_1D])
    checked = source_of(K, func, [F32_1D, F32_1D], boundscheck=True)
    assert "nmk_oob" not in plain and "checked(" not in plain
    assert checked.count("nmkjit::checked(") == 2
    assert "int64_t nmk_gsz2, int *nmk_oob)" in checked
    assert re.search(r"nmk_dev_helper_\d+\(v_a, \(v_i \+ \(\(int64_t\)1ll\)\), nmk_oob\)", checked)


def test_device_functions_are_specialised_per_signature(K):
    get_global_id = K.get_global_id
    square = K.kernel_func(lambda v: v * v)

    def func(a, b, c):
        i = get_global_id(0)
        c[i] = square(a[i]) + square(b[i]) + square(a[i])

    src = source_of(K, func, [F32_1D, I32_1D, F64_1D])
    devs = re.findall(r"__device__ __forceinline__ (\w+) (nmk_dev__lambda__\d+)\((\w+) v_v\)", src)
    assert sorted((r, p) for r, _, p in devs) == [("float", "float"), ("int32_t", "int32_t")]


@pytest.mark.parametrize("body,message", [
    ("x = [1, 2]", "Unsupported expression: List"),
    ("x = a[i]\n    x = a", "both as a scalar and as an array"),
    ("for v in a:\n        pass", "Only 'for x in range"),
    ("x = undefined_name + 1", "Unknown name 'undefined_name'"),
    ("lm = local.array(i, np.float32)", "must be constant"),
    ("return 3", "A kernel cannot return a value"),
    ("x = 'text'", "Unsupported constant"),
    ("a[i, 0] = 1", "Too many indices"),
    ("import os", "Unsupported statement: Import"),
    ("x = y + 1\n    y = 2", None),          # used before assignment in a straight line
])
def test_errors_name_the_line(K, body, message, tmp_path):
    src = ("import numpy as np\n"
           "from numba_mlir_amd.mlir.kernel_impl import get_global_id, local\n"
           "def func(a):\n    i = get_global_id(0)\n    " + body + "\n")
    path = tmp_path / "kern_mod.py"
    path.write_text(src)
    import importlib.util
    spec = importlib.util.spec_from_file_location("kern_mod", path)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    if message is None:
        kc.translate(mod.func, [F32_1D], 1, K)       # legal for the translator: y is typed later
        return
    with pytest.raises(kc.KernelCompileError) as err:
        kc.translate(mod.func, [F32_1D], 1, K)
    assert message in str(err.value)
    assert "func" in str(err.value)


def test_lambdas_are_found_in_their_source_line(K):
    table = {
        "add": lambda a, b: a + b,
        "hyp": lambda a, b: math.sqrt(a * a + b * b),
    }
    get_global_id = K.get_global_id
    for name, expect in (("add", "(v_a + v_b)"), ("hyp", "sqrtF64(")):
        f = table[name]

        def func(x, y, out):
            i = get_global_id(0)
            out[i] = f(x[i], y[i])

        assert expect in source_of(K, func, [F64_1D, F64_1D, F64_1D])


def test_generated_source_compiles_for_gfx950(K, tmp_path, monkeypatch):
    """hipcc cross-compiles without a GPU; the cache is keyed on the source."""
    monkeypatch.setattr(kc, "CACHE_DIR", str(tmp_path))
    get_global_id, atomic, group, private = K.get_global_id, K.atomic, K.group, K.private
    barrier = K.barrier

    def func(a, s, out, hist):
        i = get_global_id(0)
        scratch = private.array(4, np.float64)
        for k in range(4):
            scratch[k] = a[i] ** k
        total = group.reduce_add(scratch[3] % 7.0)
        barrier()
        view = out[s]
        view[i] = total + max(scratch[0], scratch[1]) + abs(a[i]) // 2
        atomic.add(hist, (i % 2, 0), 1)

    ck = kc.translate(func, [F64_1D, kc.SliceArg(), F64_1D, kc.Array(kc.INT32, 2)], 1, K)
    blob = kc.build_code_object(ck)
    assert blob[:4] == b"\x7fELF"
    files = sorted(os.listdir(tmp_path))
    assert len(files) == 2 and files[0].endswith(".hip") and files[1].endswith(".hsaco")
    stamp = os.path.getmtime(tmp_path / files[1])
    assert kc.build_code_object(ck) == blob                       # from the cache
    assert os.path.getmtime(tmp_path / files[1]) == stamp
    # the code object exports exactly the kernel
    rocm = os.environ.get("ROCM_PATH", "/opt/rocm")
    nm = os.path.join(rocm, "llvm", "bin", "llvm-nm")
    if os.path.exists(nm):
        out = subprocess.run([nm, str(tmp_path / files[1])], capture_output=True, text=True).stdout
        assert re.search(r" T %s\b" % ck.name, out)


def test_compile_failure_shows_the_compiler_output(K, tmp_path, monkeypatch):
    monkeypatch.setattr(kc, "CACHE_DIR", str(tmp_path))
    bad = kc.CompiledKernel("nmkjit_bad", "this is not HIP\n", [])
    with pytest.raises(kc.KernelCompileError) as err:
        kc.build_code_object(bad)
    assert "hipcc failed" in str(err.value) and "this is not HIP" in str(err.value)
    assert not [f for f in os.listdir(tmp_path) if f.endswith(".hsaco")]


# ---- njit: whole-array functions and prange loops ---------------------------

def _njit_types(case):
    f32 = lambda n: kc.Array(kc.FLOAT32, n, layout="C")      # noqa: E731
    f64 = lambda n: kc.Array(kc.FLOAT64, n, layout="C")      # noqa: E731
    return {
        "black_scholes_arrays": ("elementwise", 1, [f32(1)] * 3 + [kc.FLOAT32] * 2 + [f32(1)] * 2),
        "black_scholes_loop": ("parallel", 1, [kc.INT64] + [f32(1)] * 3 + [kc.FLOAT32] * 2 + [f32(1)] * 2),
        "fused_map": ("elementwise", 2, [kc.Array(kc.FLOAT64, 2)] * 3 + [kc.FLOAT64]),
        "fused_store": ("elementwise", 1, [kc.Array(kc.INT32, 1, layout="C")] * 2 +
                        [f64(1), kc.Array(kc.INT64, 1, layout="C")]),
        "saxpy_loop": ("parallel", 1, [kc.FLOAT32, f32(1), f32(1), f32(1)]),
        "strided_loop": ("parallel", 1, [kc.Array(kc.FLOAT64, 2), f64(1)]),
    }[case]


@pytest.mark.parametrize("case", ["black_scholes_arrays", "black_scholes_loop", "fused_map",
                                  "fused_store", "saxpy_loop", "strided_loop"])
def test_njit_functions_translate_and_compile(K, case, tmp_path, monkeypatch):
    import njit_cases
    monkeypatch.setattr(kc, "CACHE_DIR", str(tmp_path))
    mode, ndim, types = _njit_types(case)
    ck = kc.translate(getattr(njit_cases, case), types, ndim, K, mode=mode)
    assert kc.build_code_object(ck)[:4] == b"\x7fELF"
    if case == "black_scholes_arrays":
        # the reference's typing falls out of the rules: literal-bearing
        # intermediates are float64, log(P / S), T * mr and exp(b) * S float32
        for name, ctype in (("a", "float"), ("b", "float"), ("Se", "float"),
                            ("sig_sig_two", "double"), ("z", "double"), ("c", "double"),
                            ("y", "double"), ("w1", "double"), ("d1", "double"),
                            ("r", "double")):
            assert declared_type(ck.source, name) == ctype, name
        assert ck.written == ["v_call", "v_put"] and ck.ret_dtype is None
    if case == "fused_map":
        assert ck.ret_dtype == np.float64 and "nmk_ret_p" in ck.source
    if case == "strided_loop":
        assert ck.range_source == ["1", "x.shape[0] - 1", "2"]
    if case == "saxpy_loop":
        assert ck.range_source == ["n"] or ck.range_source == ["len(x)"]


def test_njit_rejects_what_it_cannot_offload(K):
    import njit_cases
    f64 = kc.Array(kc.FLOAT64, 1, layout="C")
    with pytest.raises(kc.KernelCompileError, match="after the parallel loop"):
        kc.translate(njit_cases.statements_after_loop, [f64, f64], 1, K, mode="parallel")
    with pytest.raises(kc.KernelCompileError, match="returns at its end only"):
        kc.translate(njit_cases.two_returns, [f64], 1, K, mode="elementwise")
    with pytest.raises(kc.KernelCompileError, match="no top-level prange loop"):
        kc.translate(njit_cases.no_loop, [f64], 1, K, mode="parallel")


def test_fused_maps_take_several_elements_per_lane(K, tmp_path, monkeypatch):
    import njit_cases
    monkeypatch.setattr(kc, "CACHE_DIR", str(tmp_path))
    mode, ndim, types = _njit_types("black_scholes_arrays")
    ck = kc.translate(njit_cases.black_scholes_arrays, types, ndim, K, mode=mode,
                      noalias=True, elements_per_thread=4)
    assert ck.elements_per_thread == 4
    assert "float *__restrict__ v_price_p" in ck.source
    # Dense arrays that do not overlap: a lane takes four ADJACENT options,
    # one 128-bit streaming load per operand, one 128-bit streaming store per
    # result, the operands handed to the body as values.
    assert "__launch_bounds__(256)" in ck.source
    assert ("const nmk_in_t_price nmk_in_price = __builtin_nontemporal_load("
            "reinterpret_cast<const nmk_in_t_price *>(v_price_p) + nmk_i);") in ck.source
    assert ("__builtin_nontemporal_store(nmk_vec_v_call, "
            "reinterpret_cast<nmk_out_t_v_call *>(v_call_p) + nmk_i);") in ck.source
    assert "NMK_STORE_ALONG0(&" not in ck.source and "v_P.p[" not in ck.source
    # words need 16-byte aligned arrays; single elements otherwise and at the end
    assert "const int64_t nmk_nvec = nmk_words ? nmk_gsz0 / 4 : 0;" in ck.source
    assert "for (int64_t g = nmk_nvec * 4 + nmk_lane; g < nmk_gsz0; g += nmk_lanes)" in ck.source
    # log(P / S), 1.0 / sqrt(z), exp: the plain forms first, the careful ones
    # (out of line) for a wave with an operand out of range
    assert ("v_a = nmkjit::logQuotientF32m<decltype(nmk_careful)::value>(nmk_pf_price, "
            "nmk_pf_strike, nmk_ok);") in ck.source
    assert "v_y = nmkjit::rsqrtF64m<decltype(nmk_careful)::value>(v_z, nmk_ok);" in ck.source
    assert "if (__builtin_amdgcn_ballot_w64(!nmk_ok) != 0) {" in ck.source
    assert "__attribute__((noinline)) -> nmk_results {" in ck.source
    # 0.5 + 0.5 * erf(w) with float32 results only: one table term, its own table
    assert ("v_d1 = nmkjit::cdfTermF64m<decltype(nmk_careful)::value>(v_w1, nmk_ok);"
            in ck.source)
    assert "nmkjit::cdfTableLoad();" in ck.source and "erfTableLoad" not in ck.source
    assert kc.build_code_object(ck)[:4] == b"\x7fELF"
    small = kc.translate(njit_cases.black_scholes_arrays, types, ndim, K, mode=mode,
                         noalias=True, elements_per_thread=4, stream=False)
    assert "nontemporal" not in small.source and "NMK_STORE_ALONG0(&" not in small.source
    assert ("const nmk_in_t_price nmk_in_price = *(reinterpret_cast<const nmk_in_t_price *>"
            "(v_price_p) + nmk_i);") in small.source
    # arrays with a stride: elements a block apart, loaded ahead of the body
    strided = [kc.Array(t.elem, 1) if isinstance(t, kc.Array) else t for t in types]
    ck = kc.translate(njit_cases.black_scholes_arrays, strided, ndim, K, mode=mode,
                      noalias=True, elements_per_thread=4)
    assert "for (int nmk_rep = 0; nmk_rep < 4; ++nmk_rep)" in ck.source
    assert ck.source.count("NMK_STORE_ALONG0(&") == 2
    assert "#define NMK_STORE_ALONG0(p, v, unit) nmkjit::streamStore(p, v, unit)" in ck.source
    assert ("nmk_ahead_price[nmk_rep] = __builtin_nontemporal_load(&v_price_p[g * v_price_t0]);"
            in ck.source)
    assert 'asm volatile("" : "+v"(nmk_ahead_t[nmk_rep]));' in ck.source
    assert ("nmk_item(nmk_base + nmk_rep * nmk_lsz0, nmkjit::No(), nmk_ahead_price[nmk_rep], "
            "nmk_ahead_strike[nmk_rep], nmk_ahead_t[nmk_rep]);") in ck.source
    assert "v_a = nmk::logQuotientF32(nmk_pf_price, nmk_pf_strike);" in ck.source
    assert "nmkjit::cdfTableLoad();" in ck.source and "__launch_bounds__(1024)" in ck.source
    assert kc.build_code_object(ck)[:4] == b"\x7fELF"
    # the loop form of the same body: prange(n), reads p[i], stores call[i], put[i]
    mode2, ndim2, types2 = _njit_types("black_scholes_loop")
    ck = kc.translate(njit_cases.black_scholes_loop, types2, ndim2, K, mode=mode2,
                      noalias=True, elements_per_thread=4)
    assert "nmk_out.v_call = (float)" in ck.source and "nmk_words" in ck.source
    assert ("v_a = nmkjit::logQuotientF32m<decltype(nmk_careful)::value>(v_P, v_S, nmk_ok);"
            in ck.source)
    assert ("v_d2 = nmkjit::cdfTermF64m<decltype(nmk_careful)::value>(v_w2, nmk_ok);"
            in ck.source)
    assert ("__builtin_nontemporal_store(nmk_vec_v_put, "
            "reinterpret_cast<nmk_out_t_v_put *>(v_put_p) + nmk_i);") in ck.source
    assert kc.build_code_object(ck)[:4] == b"\x7fELF"
    # ... but not when a store sits under a condition, or at another index
    def guarded(n, a, out):
        for i in njit_cases.prange(n):
            if a[i] > 0:
                out[i] = a[i]

    def shifted(n, a, out):
        for i in njit_cases.prange(n):
            out[i + 1] = a[i]

    f32c1 = kc.Array(kc.FLOAT32, 1, layout="C")
    for body in (guarded, shifted):
        ck = kc.translate(body, [kc.INT64, f32c1, f32c1], 1, K, mode="parallel", noalias=True,
                          elements_per_thread=4)
        assert "nmk_words" not in ck.source
    # a body that stores single elements keeps one element per lane and trip
    def by_index(a, b, c):
        for i in range(len(a)):
            c[i] = a[i] + b[i]

    f32c = kc.Array(kc.FLOAT32, 1, layout="C")
    ck = kc.translate(by_index, [f32c, f32c, f32c], 1, K, mode="elementwise", noalias=True,
                      elements_per_thread=4)
    assert "nmk_words" not in ck.source and "__launch_bounds__(1024)" in ck.source
    # overlapping arguments: plain pointers and stores, every load where it is used
    ck = kc.translate(njit_cases.black_scholes_arrays, types, ndim, K, mode=mode,
                      noalias=False, elements_per_thread=4)
    assert "__restrict__" not in ck.source and "nontemporal" not in ck.source
    assert "nmk_ahead" not in ck.source and "v_P.p[" in ck.source
    assert "nmk_item(nmk_base + nmk_rep * nmk_lsz0, nmkjit::No());" in ck.source
    # an argument the body also assigns is not loaded ahead; the others are
    ck = kc.translate(njit_cases.scale_in_place, [kc.Array(kc.FLOAT64, 1), kc.Array(kc.FLOAT64, 1)],
                      1, K, mode="elementwise", noalias=True, elements_per_thread=4)
    assert "nmk_ahead_b" in ck.source and "nmk_ahead_a" not in ck.source
    # more than one dimension, or an @kernel body: one element per lane
    mode, ndim, types = _njit_types("fused_map")
    ck = kc.translate(njit_cases.fused_map, types, ndim, K, mode=mode, noalias=True,
                      elements_per_thread=4)
    assert ck.elements_per_thread == 1 and "nmk_rep" not in ck.source


def test_prange_loops_load_what_every_iteration_reads_ahead(K):
    import njit_cases
    f64, i64 = kc.Array(kc.FLOAT64, 1), kc.INT64
    mode, ndim, types = _njit_types("black_scholes_loop")
    ck = kc.translate(njit_cases.black_scholes_loop, types, ndim, K, mode=mode, noalias=True,
                      elements_per_thread=4)
    # (dense float32 arrays stored at the loop's own index: four adjacent
    # iterations a lane, the loads in one 128-bit word per array)
    assert "nmk_in_price = __builtin_nontemporal_load(" in ck.source
    assert "v_P = nmk_pf_price;" in ck.source and "v_T = nmk_pf_t;" in ck.source
    # arrays with a stride: a lane's iterations a block apart
    strided = [kc.Array(t.elem, 1) if isinstance(t, kc.Array) else t for t in types]
    ck = kc.translate(njit_cases.black_scholes_loop, strided, ndim, K, mode=mode, noalias=True,
                      elements_per_thread=4)
    assert "nmk_ahead_price[nmk_rep] = *(&v_price_p[g * v_price_t0]);" in ck.source
    assert "v_P = nmk_pf_price;" in ck.source and "v_T = nmk_pf_t;" in ck.source
    # overlapping arguments, or one element per lane: every load where it is written
    for kw in ({"noalias": False, "elements_per_thread": 4},
               {"noalias": True, "elements_per_thread": 1}):
        ck = kc.translate(njit_cases.black_scholes_loop, types, ndim, K, mode=mode, **kw)
        assert "nmk_ahead" not in ck.source and "v_P = v_price.p[" in ck.source
    # Only reads that every iteration performs: not behind a condition, not
    # in a loop that leaves early, not of an array the function also writes.
    ck = kc.translate(njit_cases.loop_reads, [i64, f64, f64, f64, f64], 1, K, mode="parallel",
                      noalias=True, elements_per_thread=4)
    assert "nmk_ahead_a" in ck.source                  # x = a[i] + ...
    assert "nmk_ahead_b" not in ck.source              # b[i] if x > 0 else 0.0
    assert "nmk_ahead_c" not in ck.source              # c[i] inside an if statement
    assert "nmk_ahead_out" not in ck.source            # written
    ck = kc.translate(njit_cases.loop_leaves_early, [i64, f64, f64], 1, K, mode="parallel",
                      noalias=True, elements_per_thread=4)
    assert "nmk_ahead" not in ck.source
    # (continue ends the iteration: the work-item body returns)
    assert "return;" in ck.source and "continue;" not in ck.source


def test_prange_reductions(K, tmp_path, monkeypatch):
    import njit_cases
    monkeypatch.setattr(kc, "CACHE_DIR", str(tmp_path))
    f32 = kc.Array(kc.FLOAT32, 1, layout="C")
    ck = kc.translate(njit_cases.mean_and_count, [f32, kc.FLOAT64], 1, K, mode="parallel",
                      noalias=True, elements_per_thread=4)
    assert ck.reductions == [("above", np.dtype(np.int64), "add"),
                             ("total", np.dtype(np.float64), "add")]
    assert ck.return_source == "(total / n, above)"
    assert "int64_t *nmk_part_above, double *nmk_part_total" in ck.source
    assert ck.source.count("nmkjit::blockReduceStore<") == 2
    # the launch's last block adds the blocks' results up: nothing is summed on the host
    assert "uint32_t *nmk_ticket" in ck.source
    assert "if (nmkjit::drewLastTicket(nmk_ticket)) {" in ck.source
    assert ck.source.count("nmkjit::foldPartials<") == 2
    # dense float32 operands read at the loop's own index: a 128-bit word of
    # four adjacent iterations a lane, the sums kept where they are (one
    # inlined form of the body, closures by reference)
    assert ("const nmk_in_t_x nmk_in_x = __builtin_nontemporal_load("
            "reinterpret_cast<const nmk_in_t_x *>(v_x_p) + nmk_i);") in ck.source
    assert "auto nmk_item = [&](const int64_t nmk_gid0, auto nmk_careful" in ck.source
    assert "noinline" not in ck.source and "ballot" not in ck.source
    assert kc.build_code_object(ck)[:4] == b"\x7fELF"
    # (float64 operands: a lane's elements a block apart, as before)
    f64 = kc.Array(kc.FLOAT64, 1, layout="C")
    ck64 = kc.translate(njit_cases.sum_of_squares, [f64], 1, K, mode="parallel",
                        noalias=True, elements_per_thread=4)
    assert "nmk_in_t_x" not in ck64.source and "nmk_ahead_x[4]" in ck64.source
    ck = kc.translate(njit_cases.product, [f32], 1, K, mode="parallel")
    assert ck.reductions == [("p", np.dtype(np.float64), "mul")]
    assert "double v_p = (double)1;" in ck.source
    with pytest.raises(kc.KernelCompileError, match="cannot be read inside the loop"):
        kc.translate(njit_cases.reduction_read_in_loop, [f32], 1, K, mode="parallel")


def test_kernels_stream_stores_nobody_reads_back(K):
    """With arguments the host found disjoint, an array the body only stores
    into is written past the caches -- where the innermost index runs along
    the grid dimension that lies on x."""
    get_global_id = K.get_global_id
    f64_2d = kc.Array(kc.FLOAT64, 2, layout="C")

    def pairwise(X1, X2, D):
        i = get_global_id(0)
        j = get_global_id(1)
        d = 0.0
        for k in range(X1.shape[1]):
            tmp = X1[i, k] - X2[j, k]
            d += tmp * tmp
        D[i, j] = np.sqrt(d)

    def stream(src):
        return [k for k in range(3)
                if f"#define NMK_STORE_ALONG{k}(p, v, unit) nmkjit::streamStore" in src]

    src = source_of(K, pairwise, [f64_2d] * 3, ndim=2, remap=True, noalias=True)
    assert "NMK_STORE_ALONG1(&v_D.p[" in src and stream(src) == [1]
    assert "double *__restrict__ v_D_p" in src
    # as written (dimension 0 on x) lanes write a column apart: plain stores
    src = source_of(K, pairwise, [f64_2d] * 3, ndim=2, remap=False, noalias=True)
    assert "NMK_STORE_ALONG1(&v_D.p[" in src and stream(src) == [0]
    # arrays small enough to stay cached between launches: ordinary stores
    src = source_of(K, pairwise, [f64_2d] * 3, ndim=2, remap=True, noalias=True,
                    stream=False)
    assert "NMK_STORE_ALONG1(&" not in src and "double *__restrict__ v_D_p" in src
    # arguments that may overlap: nothing changes
    src = source_of(K, pairwise, [f64_2d] * 3, ndim=2, remap=True)
    assert "NMK_STORE_ALONG1(&" not in src and "__restrict__" not in src

    def reads_back(a, out):
        i = get_global_id(0)
        out[i] = a[i]
        out[i] += 1.0

    def shifted(a, out):
        i = get_global_id(0)
        out[i + 1] = a[i]

    def scattered(a, idx, out):
        i = get_global_id(0)
        out[idx[i]] = a[i]

    def handed_on(a, out):
        i = get_global_id(0)
        view = out[1:]
        view[i] = a[i]
        out[i] = 0.0

    assert "NMK_STORE_ALONG0(&" not in source_of(K, reads_back, [F64_1D] * 2, noalias=True)
    assert "NMK_STORE_ALONG0(&" in source_of(K, shifted, [F64_1D] * 2, noalias=True)
    assert "NMK_STORE_ALONG0(&" not in source_of(K, scattered, [F64_1D, I64_1D, F64_1D],
                                                  noalias=True)
    assert "NMK_STORE_ALONG0(&" not in source_of(K, handed_on, [F64_1D] * 2, noalias=True)

    # work-items that exchange data through memory keep plain pointers
    barrier = K.barrier

    def exchanging(a, out):
        i = get_global_id(0)
        out[i] = a[i]
        barrier()
        a[i] = 1.0

    assert "__restrict__" not in source_of(K, exchanging, [F64_1D] * 2, noalias=True)


def test_bodies_are_split_at_reductions_and_contractions():
    """A straight-line body becomes map stages (one fused kernel each) around
    library stages (the reductions and matrix products)."""
    import ast
    import njit_cases
    from numba_mlir_amd.mlir import staging

    def plan(func):
        node = kc._function_ast(func)
        return staging.plan_of(node, lambda name: name == "np")

    p = plan(njit_cases.l2_norm_rows)
    assert [s.kind for s in p.stages] == ["map", "lib", "return"]
    assert ast.unparse(p.stages[0].expr) == "np.square(a)"
    assert (p.stages[1].op, p.stages[1].kwargs) == ("sum", {"axis": 1})
    assert ast.unparse(p.stages[2].expr) == "np.sqrt(_nmk_t2)"

    p = plan(njit_cases.softmax)
    assert [repr(s) for s in p.stages] == [
        "_nmk_t1 = max(x, {})", "map e np.exp(x - _nmk_t1)",
        "_nmk_t2 = sum(e, {})", "return e / _nmk_t2"]
    assert p.stages[1].inputs == ["x", "_nmk_t1"]

    p = plan(njit_cases.chain)
    assert [(s.kind, s.op, s.operands) for s in p.stages[:2]] == [
        ("lib", "dot", ["a", "b"]), ("lib", "dot", ["_nmk_t1", "c"])]

    p = plan(njit_cases.weighted_rows)
    assert [s.kind for s in p.stages] == ["map", "lib", "map", "map", "store"]
    assert p.stages[3].target == "s" and ast.unparse(p.stages[3].expr) == "s + 1.0"

    def affine(a, b, c, out):
        np.add(np.dot(a, b), c, out)

    p = plan(affine)
    assert [repr(s) for s in p.stages] == ["_nmk_t1 = dot(a, b, {})",
                                           "store out np.add(_nmk_t1, c)"]

    # nothing to split at, or not straight-line: left to the other paths
    assert plan(njit_cases.fused_map) is None
    assert plan(njit_cases.saxpy_loop) is None
    assert plan(njit_cases.sum_of_squares) is None

    # a stage's function carries its own tree for the kernel compiler
    func, params = staging.stage_function(plan(njit_cases.softmax).stages[1],
                                          "softmax_stage1", {"np": np})
    assert params == ["x", "_nmk_t1"]
    assert kc._function_ast(func).name == "softmax_stage1"
    np.testing.assert_allclose(func(np.array([0.0, 1.0]), 1.0), np.exp([-1.0, 0.0]))


def test_array_operands_follow_the_array_typing_rule(K):
    """Between values computed from array elements a float meeting an integer
    keeps its width (the reference's _select_float_type, numpy/funcs.py:
    402-418); scalar arithmetic keeps Numba's scalar rules."""
    f32 = kc.Array(kc.FLOAT32, 1, layout="C")
    i32 = kc.Array(kc.INT32, 1, layout="C")

    def ret(func, types):
        return np.dtype(kc.translate(func, types, 1, K, mode="elementwise").ret_dtype)

    assert ret(lambda a: a ** 2, [f32]) == np.float32
    assert ret(lambda a: a * 2 + 1, [f32]) == np.float32
    assert ret(lambda a, i: a + i, [f32, i32]) == np.float32
    assert ret(lambda a, i: np.where(i > 0, a, i), [f32, i32]) == np.float32
    assert ret(lambda a, i: np.maximum(a, i), [f32, i32]) == np.float32
    assert ret(lambda a: a * 2.0, [f32]) == np.float64          # two floats promote
    assert ret(lambda a: a / 3, [f32]) == np.float32
    assert ret(lambda i: i / 3, [i32]) == np.float64
    assert ret(lambda i: i * 2, [i32]) == np.int64
    # a scalar argument times a literal is scalar arithmetic: float64
    assert ret(lambda a, s: a + s * 2, [f32, kc.FLOAT32]) == np.float64

    def through_names(a, i):
        t = a - 1
        u = t * i
        return u ** 2

    assert ret(through_names, [f32, i32]) == np.float32


def test_which_arguments_fit_a_prepared_launch():
    """A stored launch accepts the arrays it was prepared with, or dense
    arrays of the same type and size (launches are prepared on arrays with
    their dimensions merged); anything else could be addressed out of bounds."""
    from numba_mlir_amd.mlir import kernel_impl as ki
    f8, f4 = np.dtype("f8"), np.dtype("f4")
    assert ki._dense_size((4096, 4096), (32768, 8), 8) == 4096 * 4096
    assert ki._dense_size((3, 1, 5), (40, 8, 8), 8) == 15          # a stride of a 1-extent is free
    assert ki._dense_size((4, 4), (64, 8), 8) is None              # rows with gaps
    assert ki._dense_size((4, 4), (8, 32), 8) is None              # column-major
    merged = (f8, (16777216,), (8,))
    assert ki._fits(merged, (f8, (4096, 4096), (32768, 8)))
    assert ki._fits(merged, merged)
    assert not ki._fits(merged, (f4, (4096, 4096), (16384, 4)))
    assert not ki._fits(merged, (f8, (4096, 4095), (32760, 8)))
    assert not ki._fits((f8, (16,), (8,)), (f8, (4, 4), (64, 8)))
    assert ki._fits((f8, (4, 4), (64, 8)), (f8, (4, 4), (64, 8)))   # the same strided layout
    assert ki._fits(float, float) and not ki._fits(float, int)
    assert not ki._fits(np.dtype("f4"), merged)
