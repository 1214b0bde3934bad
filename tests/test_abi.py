"""CPU-side checks of the boundary: the shared library loads, exports every
symbol include/tlhip.h declares, fails loudly without a GPU, and its host-side
functions (f16 codec, quantizer) match the oracle bit for bit."""
import ctypes
import json
import os
import re

import numpy as np
import pytest

import torchlette_amd as T
from oracle import quant_oracle as O
from torchlette_amd import _lib as L

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "tlhip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(tlhip_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = L.load()
    names = declared_symbols()
    assert len(names) >= 40
    for name in names:
        assert hasattr(lib, name), name
    # and the binding declares a signature for each of them
    assert sorted(L.SIGNATURES) == names


def test_struct_sizes_match_the_header_layout():
    assert ctypes.sizeof(L.EpilogueOp) == 24
    assert ctypes.sizeof(L.Epilogue) == 8 + 4 * 24
    assert ctypes.sizeof(L.QWeight) == 40
    assert ctypes.sizeof(L.KernelConfig) == 32
    assert ctypes.sizeof(L.DeviceInfo) == 64 + 32 + 6 * 4 + 2 * 8


@pytest.mark.skipif(os.path.exists("/dev/kfd"), reason="GPU present")
def test_compute_fails_loudly_without_a_gpu():
    with pytest.raises(L.TlhipError, match="no HIP device|no CPU fallback"):
        T.HipBackend(0)
    qw = L.QWeight(L.FMT_INT4_GROUPED, 32, 4, 32, 16, 16)
    rc = L.load().tlhip_dequant(ctypes.byref(qw), 16, None)
    assert rc == 3 and "not initialised" in L.last_error()
    rc = L.load().tlhip_matmul_quantized(ctypes.byref(qw), 16, L.F16, 1, 16, L.F16, 1.0, None, None)
    assert rc == 3


def test_host_f16_codec_matches_oracle_everywhere_it_matters():
    lib = L.load()
    bits = np.arange(65536, dtype=np.uint16)
    ref = O.f16_bits_to_f32(bits)
    got = np.array([lib.tlhip_f16_bits_to_f32(int(b)) for b in bits], np.float32)
    nan = np.isnan(ref)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got[~nan].view(np.uint32), ref[~nan].view(np.uint32))
    rng = np.random.default_rng(1)
    u = np.concatenate([
        rng.integers(0, 2 ** 32, 20000, dtype=np.uint64).astype(np.uint32),
        np.arange(102 << 23, 114 << 23, 40009, dtype=np.uint32),          # subnormal range + first normal
        (np.arange(113 << 23, 143 << 23, 1 << 13, dtype=np.uint32) | 0x1000)[::7],  # exact ties
        np.array([0, 0x80000000, 0x7F800000, 0xFF800000, 0x7FC00000, 0x33000000, 0x32FFFFFF,
                  0x477FE000, 0x477FEFFF, 0x477FF000], np.uint32),
    ])
    x = u.view(np.float32)
    want = O.f32_to_f16_bits(x)
    got = np.array([lib.tlhip_f32_to_f16_bits(float(v)) if not np.isnan(v) else
                    lib.tlhip_f32_to_f16_bits(float("nan")) for v in x], np.uint16)
    ok = ~np.isnan(x)
    assert np.array_equal(got[ok], want[ok])
    assert all((g & 0x7FFF) == 0x7C00 for g in got[~ok])


@pytest.mark.parametrize("n,k,g", [(1, 4, 4), (3, 64, 64), (64, 256, 64), (17, 384, 128), (300, 1024, 64)])
def test_host_quantizer_matches_oracle(n, k, g):
    rng = np.random.default_rng(n * 1000 + k)
    w = (rng.standard_normal((n, k)) * np.exp(rng.uniform(-8, 3, (n, 1)))).astype(np.float32)
    if n > 2:
        w[1, : g] = 0.0                      # all-zero group
        w[2, 0] = np.float32(1.0004)         # scale rounds below abs-max -> clamp
    p, s = T.quantizeLinearWeight(w, n, k, g)
    p2, s2 = O.quantize_int8_grouped(w, n, k, g)
    assert np.array_equal(s, s2) and np.array_equal(p, p2)


def test_host_quantizer_half_integers_nan_inf_and_threads():
    w = np.array([127.0, 2.5, -2.5, -0.5, 0.5, 1.5, -1.5, -126.5], np.float32)
    p, s = T.quantizeLinearWeight(w, 1, 8, 8)
    assert O.np_unpack_int8(p, 1, 8).ravel().tolist() == [127, 3, -2, 0, 1, 2, -1, -126]
    w = np.zeros(12, np.float32)
    w[4:8] = [np.nan, 1.0, -0.25, np.nan]
    w[8:12] = [np.inf, 1.0, -1.0, 0.0]
    p, s = T.quantizeLinearWeight(w, 1, 12, 4)
    p2, s2 = O.quantize_int8_grouped(w, 1, 12, 4)
    assert np.array_equal(p, p2) and np.array_equal(s, s2)
    # large enough to take the multi-threaded path
    rng = np.random.default_rng(9)
    w = rng.standard_normal((2048, 2048)).astype(np.float32)
    p, s = T.quantizeLinearWeight(w, 2048, 2048, 64)
    p2, s2 = O.quantize_int8_grouped(w, 2048, 2048, 64)
    assert np.array_equal(p, p2) and np.array_equal(s, s2)


def test_host_quantizer_errors_carry_the_reference_messages():
    w = np.zeros(16, np.float32)
    with pytest.raises(L.TlhipError, match="expected 32 elements, got 16"):
        T.quantizeLinearWeight(w, 4, 8, 4)
    with pytest.raises(L.TlhipError, match="K=6 must be divisible by 4"):
        T.quantizeLinearWeight(np.zeros(12, np.float32), 2, 6, 2)
    with pytest.raises(L.TlhipError, match="K=8 must be divisible by groupSize=3"):
        T.quantizeLinearWeight(w, 2, 8, 3)


def test_tuning_cache_json_round_trip_and_autotune_toggle():
    T.resetMatmulState()
    assert not T.isAutotuneEnabled()
    T.setAutotuneEnabled(True)
    T.setAutotuneEnabled(True)
    assert T.isAutotuneEnabled()
    T.setAutotuneEnabled(False)  # resets the nesting counter (dispatch.ts:128-134)
    assert not T.isAutotuneEnabled()
    text = '{"version":1,"entries":{"1_4096_4096_int4-grouped_g32_f16_f16":[0,64,1,4,1,0,0,0],' \
           '"512_12288_4096_int4-grouped_g32_f16_f16":[2,128,128,64,2,2,0,0]}}'
    T.importTuningCache(text)
    out = T.exportTuningCache()
    assert out.startswith(text[:-1] + ',"model":{')      # the entries as imported, then the routing model
    assert json.loads(out)["entries"] == json.loads(text)["entries"]
    T.clearTuningCache()
    assert json.loads(T.exportTuningCache())["entries"] == {}
    with pytest.raises(L.TlhipError, match="entries"):
        T.importTuningCache("{}")


def test_tuning_cache_import_survives_malformed_text():
    """Every prefix of a valid cache text, pretty-printed text and junk: an error or a
    clean import, never a crash, and a failed import leaves the cache as it was."""
    import json
    T.clearTuningCache()
    entries = {"1_4096_4096_int4-grouped_g32_f16_f16": [0, 64, 1, 4, 1, 0, 0, 0],
               "16_4096_12288_int4-grouped_g32_f16_f16": [1, 8, 4, 4, 2, 0, 1, 0]}
    model = {"rows_break_even": 0.5, "pass_base_us": 4.0}
    text = json.dumps({"version": 1, "entries": entries, "model": model}, separators=(",", ":"))
    whole_entries = text.index(',"model"')
    empty = T.exportTuningCache()
    for cut in range(len(text)):
        try:
            T.importTuningCache(text[:cut])
            # only a text whose entries object is whole is taken, and a model object only whole
            assert cut >= len(text) - 1 or whole_entries <= cut <= whole_entries + len(',"model'), cut
            T.clearTuningCache()
        except L.TlhipError:
            assert T.exportTuningCache() == empty, cut   # neither entries nor model numbers were taken
    T.importTuningCache(json.dumps({"version": 1, "entries": entries}, indent=2))   # as json.dump writes it
    assert json.loads(T.exportTuningCache())["entries"] == entries
    T.clearTuningCache()
    for junk in ('{"entries":', '{"entries":{"k":[1,2,3]}}', '{"entries":{"k":"v"}}', '{"entries":{k:[0]}}',
                 '{"entries":{"a_b":[0,0,0,0,0,0,0,0]}}'):
        try:
            T.importTuningCache(junk)
        except L.TlhipError:
            pass
    T.clearTuningCache()


def test_format_names_resolve_like_the_reference():
    f = T.resolveWeightFormat("int8-64")
    assert f.elementType == "f16" and f.packing == T.QuantPacking("int8-grouped", 64, "f16")
    assert T.resolveWeightFormat("int8-128", "f32").packing.groupSize == 128
    assert T.resolveWeightFormat("int4-32").packing == T.QuantPacking("int4-grouped", 32, "f16")
    assert T.resolveWeightFormat("int8-row").packing.scheme == "int8-row"


def test_enum_values_of_the_header_match_both_bindings():
    """The ctypes mirror and the JavaScript files carry the header's enum values as plain
    numbers: every one of them is checked against include/tlhip.h."""
    import re
    here = os.path.dirname(os.path.abspath(__file__))
    header = open(os.path.join(here, "..", "include", "tlhip.h")).read()
    enums = {name: int(value) for name, value in re.findall(r"\b(TLHIP_[A-Z0-9_]+)\s*=\s*(-?\d+)", header)}
    assert enums["TLHIP_EPI_BINARY"] == 3 and enums["TLHIP_BINARY_MUL"] == 2   # the regex sees them
    from torchlette_amd import _lib as L
    assert (L.EPI_NONE, L.EPI_BIAS, L.EPI_UNARY, L.EPI_BINARY, L.EPI_CAST_F16) == tuple(
        enums[n] for n in ("TLHIP_EPI_NONE", "TLHIP_EPI_BIAS", "TLHIP_EPI_UNARY", "TLHIP_EPI_BINARY", "TLHIP_EPI_CAST_F16"))
    assert L.BINARY == {"add": enums["TLHIP_BINARY_ADD"], "sub": enums["TLHIP_BINARY_SUB"], "mul": enums["TLHIP_BINARY_MUL"]}
    unary = {"none": "NONE", "relu": "RELU", "silu": "SILU", "gelu": "GELU_TANH", "gelu_tanh": "GELU_TANH",
             "gelu_erf": "GELU_ERF", "sigmoid": "SIGMOID", "tanh": "TANH"}
    assert L.UNARY == {k: enums["TLHIP_UNARY_" + v] for k, v in unary.items()}
    assert (L.FMT_INT8_GROUPED, L.FMT_INT8_ROW, L.FMT_INT4_GROUPED) == (
        enums["TLHIP_FMT_INT8_GROUPED"], enums["TLHIP_FMT_INT8_ROW"], enums["TLHIP_FMT_INT4_GROUPED"])
    assert (L.F32, L.F16, L.I32) == (enums["TLHIP_F32"], enums["TLHIP_F16"], enums["TLHIP_I32"])
    # the side door's constants (a JavaScript file: read as text)
    js = open(os.path.join(here, "..", "torchlette_amd", "addon", "hip_matmul_dispatch.js")).read()
    m = re.search(r"const EPI_BIAS = (\d+), EPI_UNARY = (\d+), EPI_BINARY = (\d+), EPI_CAST_F16 = (\d+);", js)
    assert m and tuple(int(v) for v in m.groups()) == (L.EPI_BIAS, L.EPI_UNARY, L.EPI_BINARY, L.EPI_CAST_F16)
    m = re.search(r"const BINARY = \{ add: (\d+), sub: (\d+), mul: (\d+) \};", js)
    assert m and tuple(int(v) for v in m.groups()) == (L.BINARY["add"], L.BINARY["sub"], L.BINARY["mul"])
    m = re.search(r"const UNARY = \{([^}]*)\};", js)
    js_unary = {k.strip(): int(v) for k, v in (item.split(":") for item in m.group(1).split(","))}
    assert js_unary == {k: v for k, v in L.UNARY.items() if k != "none"}


def test_an_epilogue_input_of_the_wrong_shape_is_refused_before_any_launch():
    """EpilogueOp names a typed tensor in the reference (matmul/types.ts:13-24); the C ABI
    sees a pointer, so each step states its input's rows and the library checks them against
    the call: a BINARY step indexes its input by output element, and an [N] tensor handed to
    it at M > 1 would be read past its end.  The check needs no device."""
    lib = L.load()
    w = L.QWeight(L.FMT_INT4_GROUPED, 32, 64, 256, None, None)
    buf = ctypes.create_string_buffer(64)  # never dereferenced: the check looks at shapes only
    ptr = ctypes.cast(buf, ctypes.c_void_p).value

    def check(m, *ops):
        ep = L.Epilogue()
        ep.n_ops = len(ops)
        for i, op in enumerate(ops):
            ep.ops[i] = L.EpilogueOp(*op)
        return lib.tlhip_epilogue_check(ctypes.byref(w), m, ctypes.byref(ep)), L.last_error()

    assert check(8, (L.EPI_BIAS, 0, ptr, L.F32, 1), (L.EPI_UNARY, L.UNARY["silu"], None, 0, 0), (L.EPI_BINARY, 0, ptr, L.F32, 8))[0] == 0
    rc, msg = check(8, (L.EPI_BINARY, 0, ptr, L.F32, 1))       # an [N] tensor as a residual at 8 rows
    assert rc == L.ERR_INVALID and "binary epilogue input must be [M,N] = [8,64]" in msg
    rc, msg = check(8, (L.EPI_BINARY, 0, ptr, L.F32, 0))       # the field left at zero
    assert rc == L.ERR_INVALID and "rows field says 0" in msg
    rc, msg = check(1, (L.EPI_BINARY, 0, ptr, L.F32, 1))       # one row: [N] is [M,N]
    assert rc == 0
    rc, msg = check(8, (L.EPI_BIAS, 0, ptr, L.F32, 8))         # an [M,N] tensor as a bias
    assert rc == L.ERR_INVALID and "bias epilogue input must be [N] = [64]" in msg
    rc, msg = check(8, (L.EPI_BIAS, 0, ptr, L.F32, 0))
    assert rc == L.ERR_INVALID


def _routes(lib):
    """The default route of a grid of problems between decode and prefill sizes."""
    out = []
    buf = ctypes.create_string_buffer(64)
    ptr = ctypes.cast(buf, ctypes.c_void_p).value
    for fmt, g in ((L.FMT_INT4_GROUPED, 32), (L.FMT_INT8_GROUPED, 64), (L.FMT_INT8_ROW, 0)):
        for n, k in ((4096, 4096), (12288, 4096), (4096, 12288), (2048, 2048), (28672, 8192), (256000, 2304)):
            for m in (1, 4, 9, 16, 17, 40, 64, 100, 128, 200, 256, 512, 1000, 2048):
                w = L.QWeight(fmt, g, n, k, ptr, ptr)
                chunk, first, last = ctypes.c_int64(), L.KernelConfig(), L.KernelConfig()
                assert lib.tlhip_selected_route(ctypes.byref(w), L.F16, m, L.F16, ctypes.byref(chunk), ctypes.byref(first),
                                                ctypes.byref(last)) == 0, L.last_error()
                out.append((fmt, n, k, m, chunk.value, first.as_tuple(), last.as_tuple()))
    return out


def test_the_routing_model_travels_with_the_tuning_cache():
    """The fitted numbers of the default routing are data, not code: without any tuning file
    and with only the shipped file's model the routes agree (the file carries the built-in
    values), the export writes the model back, and a changed number changes routes."""
    lib = L.load()
    shipped = json.load(open(os.path.join(os.path.dirname(T.__file__), "tuning", "mi355x.json")))
    before = T.exportTuningCache()
    try:
        T.clearTuningCache()                       # what TLHIP_TUNING_FILE=none leaves: built-in model, no entries
        builtin = _routes(lib)
        T.importTuningCache(json.dumps({"version": 1, "entries": {}, "model": shipped["model"]}))
        assert _routes(lib) == builtin
        exported = json.loads(T.exportTuningCache())["model"]
        assert exported == {k: float(v) for k, v in shipped["model"].items()}
        assert any(chunk == 64 for (_, _, _, _, chunk, _, _) in builtin)      # some rows go 64 at a time ...
        T.importTuningCache(json.dumps({"version": 1, "entries": {}, "model": {"rows_break_even": 1e-6, "passes_break_even": 1e-6}}))
        changed = _routes(lib)
        assert changed != builtin and not any(chunk == 64 for (_, _, _, _, chunk, _, _) in changed)  # ... until the model says no
        with pytest.raises(L.TlhipError, match="unknown model field"):
            T.importTuningCache('{"version":1,"entries":{},"model":{"no_such_number":1}}')
        T.clearTuningCache()
        assert _routes(lib) == builtin
    finally:
        T.clearTuningCache()
        T.importTuningCache(before)
