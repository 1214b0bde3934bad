"""GPU parity through the reference's own host language: the N-API addon
(torchlette_amd/addon/tlhip_napi.c) and the JavaScript `hip` backend object above it
(hip_backend.js), driven by Node in one child process over inputs written here, and
checked here against the oracle.  The scenario is tests/js/addon_scenario.js.

Tolerances as in the ctypes tests: dequant and quantize bit-exact; f32 GEMV rel-L2
<= 2e-6; f16 outputs and prefill rel-L2 <= 1e-3."""
import json
import os
import shutil
import subprocess
import zlib

import numpy as np
import pytest

from oracle import quant_oracle as O
from helpers import f16_round, fmt_name, make_weight, make_x, rel_l2

pytestmark = pytest.mark.gpu
HERE = os.path.dirname(os.path.abspath(__file__))
ADDON = os.path.join(HERE, "..", "torchlette_amd", "addon", "tlhip_napi.node")


def seeded(*key):
    return np.random.default_rng(zlib.crc32(repr(key).encode()))


LINEAR = [
    # name, format, n, k, g, m, xdtype, element, bias, act, fused
    ("int8g_m1_f32", "int8-grouped", 512, 1024, 64, 1, "f32", "f32", False, "none", False),
    ("int8g_m1_bias_silu", "int8-grouped", 512, 1024, 128, 1, "f32", "f32", True, "silu", False),
    ("int4_m1_f16", "int4-grouped", 1024, 2048, 32, 1, "f16", "f16", False, "none", False),
    ("int4_m8_fused", "int4-grouped", 1024, 2048, 32, 8, "f16", "f16", True, "gelu", True),
    ("int4_m96_prefill", "int4-grouped", 512, 1024, 32, 96, "f16", "f16", True, "silu", True),
    ("int8row_m3", "int8-row", 640, 1024, 0, 3, "f16", "f32", False, "relu", True),
]


@pytest.fixture(scope="module")
def run(tmp_path_factory):
    node = shutil.which("node")
    if node is None:
        pytest.skip("no node binary on this machine")
    if not os.path.exists(ADDON):
        pytest.fail("torchlette_amd/addon/tlhip_napi.node is not built (run __graft_entry__.build())")
    d = str(tmp_path_factory.mktemp("addon"))
    cases, want = [], {}

    def put(name, arr):
        np.ascontiguousarray(arr).tofile(os.path.join(d, name))
        return name

    for (name, fmt, n, k, g, m, xdt, element, has_bias, act, fused) in LINEAR:
        rng = seeded("addon", name)
        packed, scales, deq = make_weight(fmt, n, k, g, rng)
        x = make_x(m, k, xdt, rng)
        bias = rng.standard_normal(n).astype(np.float32) if has_bias else None
        cases.append({"kind": "linear", "name": name, "format": fmt_name(fmt, g), "element": element, "n": n, "k": k,
                      "m": m, "xdtype": xdt, "act": act, "fused": fused,
                      "packed": put(name + ".packed", packed), "scales": put(name + ".scales", scales),
                      "x": put(name + ".x", x.astype(np.float32)),
                      "bias": put(name + ".bias", bias) if has_bias else None, "out": name + ".y"})
        want[name] = (O.linear(x.astype(np.float32), deq, bias, "gelu_tanh" if act == "gelu" else act),
                      "f16" if (xdt == "f16" and element == "f16") else "f32", (m, n))

    rng = seeded("addon", "quantize")
    n, k, g = 96, 512, 64
    w = (rng.random((n, k)) * 2 - 1).astype(np.float32)
    w[3, :64] = 0.0
    w[5, 70] = 1e-7
    cases.append({"kind": "quantize", "name": "quantize", "n": n, "k": k, "g": g, "weight": put("q.w", w),
                  "out_packed": "q.packed", "out_scales": "q.scales", "out_dequant": "q.deq",
                  "out_dequant_device": "q.deqdev"})
    want["quantize"] = O.quantize_int8_grouped(w, n, k, g)

    for kind in ("rmsnorm_linear", "gated_linear"):
        rng = seeded("addon", kind)
        n, k, g, m = 768, 1024, 32, 2
        packed, scales, deq = make_weight("int4-grouped", n, k, g, rng)
        x = make_x(m, k, "f16", rng, std=2.0)
        c = {"kind": kind, "name": kind, "format": "int4-32", "element": "f16", "n": n, "k": k, "m": m,
             "xdtype": "f16", "packed": put(kind + ".packed", packed), "scales": put(kind + ".scales", scales),
             "x": put(kind + ".x", x.astype(np.float32)), "out": kind + ".y", "out_apart": kind + ".yapart"}
        if kind == "rmsnorm_linear":
            nw = (1 + 0.2 * rng.standard_normal(k)).astype(np.float32)
            c.update(norm_weight=put(kind + ".nw", nw), eps=1e-6, out_norm=kind + ".norm")
            fx = O.rmsnorm(x.astype(np.float32), nw, 1e-6)
        else:
            up = make_x(m, k, "f16", rng)
            c.update(up=put(kind + ".up", up.astype(np.float32)), out_prod=kind + ".prod")
            fx = O.gated(x.astype(np.float32), up.astype(np.float32), "silu")
        cases.append(c)
        want[kind] = (fx, O.linear(f16_round(fx).astype(np.float32), deq), (m, n))

    rng = seeded("addon", "grouped")
    k = 1024
    x = make_x(1, k, "f16", rng)
    gw = []
    for i, n in enumerate((1024, 256, 256)):
        packed, scales, deq = make_weight("int4-grouped", n, k, 32, rng)
        gw.append({"n": n, "packed": put(f"g{i}.packed", packed), "scales": put(f"g{i}.scales", scales),
                   "out": f"g{i}.y"})
        want[f"grouped{i}"] = O.linear(x.astype(np.float32), deq)
    cases.append({"kind": "grouped", "name": "grouped", "format": "int4-32", "k": k, "m": 1,
                  "x": put("g.x", x.astype(np.float32)), "weights": gw})
    # the same group for a batched decode step (8 rows), and one Linear through the entry point
    # that allocates nothing
    x8 = make_x(8, k, "f16", rng)
    gw8 = []
    for i in range(3):
        gw8.append(dict(gw[i], out=f"g8_{i}.y"))
        n = gw[i]["n"]
        deq = O.dequant_int4_grouped(np.fromfile(os.path.join(d, gw[i]["packed"]), np.uint32),
                                     np.fromfile(os.path.join(d, gw[i]["scales"]), np.uint16), n, k, 32)
        want[f"grouped8_{i}"] = O.linear(x8.astype(np.float32), deq)
    cases.append({"kind": "grouped", "name": "grouped8", "format": "int4-32", "k": k, "m": 8,
                  "x": put("g8.x", x8.astype(np.float32)), "weights": gw8, "out_noalloc": "g8.noalloc"})

    # the MLP block of a decode step through its one-call entry point
    rng = seeded("addon", "mlp")
    k, ff, m = 512, 1536, 4
    x = make_x(m, k, "f16", rng)
    mw, deqs = [], []
    for i, (n_, k_) in enumerate(((ff, k), (ff, k), (k, ff))):
        packed, scales, deq = make_weight("int4-grouped", n_, k_, 32, rng)
        mw.append({"n": n_, "k": k_, "packed": put(f"mlp{i}.packed", packed), "scales": put(f"mlp{i}.scales", scales)})
        deqs.append(deq)
    cases.append({"kind": "mlp", "name": "mlp", "format": "int4-32", "k": k, "m": m, "act": "silu",
                  "x": put("mlp.x", x.astype(np.float32)), "weights": mw, "out": "mlp.y"})
    xf = x.astype(np.float32)
    hidden = O.gated(O.linear(xf, deqs[0]), O.linear(xf, deqs[1]), "silu")
    want["mlp"] = (O.linear(f16_round(hidden).astype(np.float32), deqs[2]), (m, k))

    for name, m, xdt, out_dtype in (("door_m1", 1, "f32", "f32"), ("door_m64", 64, "f16", "f16")):
        rng = seeded("addon", name)
        n, k, g = 768, 1024, 32
        packed, scales, deq = make_weight("int4-grouped", n, k, g, rng)
        x = make_x(m, k, xdt, rng)
        bias = rng.standard_normal(n).astype(np.float32)
        residual = rng.standard_normal((m, n)).astype(np.float32)
        cases.append({"kind": "side_door", "name": name, "format": "int4-32", "element": "f16", "n": n, "k": k, "m": m,
                      "xdtype": xdt, "act": "silu", "out_dtype": out_dtype, "packed": put(name + ".packed", packed),
                      "scales": put(name + ".scales", scales), "x": put(name + ".x", x.astype(np.float32)),
                      "bias": put(name + ".bias", bias), "residual": put(name + ".residual", residual), "out": name + ".y"})
        lin = O.linear(x.astype(np.float32), deq, bias, "silu")
        want[name] = (lin, out_dtype, (m, n))
        want[name + "_residual"] = (lin + residual).astype(np.float32)

    rng = seeded("addon", "topk")
    logits = rng.standard_normal(50000).astype(np.float32)
    logits[[7, 49999]] = logits.max() + 1.0  # a tie at the top: the smaller index first
    cases.append({"kind": "topk", "name": "topk", "length": logits.size, "k": 40, "logits": put("t.logits", logits),
                  "out_values": "t.values", "out_indices": "t.indices", "out_packed": "t.packed"})
    want["topk"] = logits

    with open(os.path.join(d, "manifest.json"), "w") as f:
        json.dump({"cases": cases}, f)
    print("running node scenario in", d, flush=True)
    proc = subprocess.run([node, os.path.join(HERE, "js", "addon_scenario.js"), d], capture_output=True, text=True,
                          timeout=300)
    assert proc.returncode == 0, proc.stdout[-2000:] + proc.stderr[-4000:]
    with open(os.path.join(d, "results.json")) as f:
        results = json.load(f)

    def get(name, dtype=np.float32):
        return np.fromfile(os.path.join(d, name), dtype=dtype)

    return {"results": results, "want": want, "get": get}


def test_device_is_the_mi355x(run):
    assert run["results"]["device"]["arch"].startswith("gfx950")
    assert run["results"]["device"]["computeUnits"] == 256


@pytest.mark.parametrize("case", LINEAR, ids=[c[0] for c in LINEAR])
def test_linear_through_the_js_backend(run, case):
    name, m = case[0], case[5]
    want, dtype, shape = run["want"][name]
    r = run["results"]["cases"][name]
    assert tuple(r["shape"]) == shape and r["dtype"] == dtype
    # routing: M <= 16 counts as a GEMV dispatch, larger M as a GEMM dispatch
    assert (r["gemv"], r["gemm"]) == ((1, 0) if m <= 16 else (0, 1))
    got = run["get"](name + ".y").reshape(shape)
    assert rel_l2(got, want) <= (2e-6 if dtype == "f32" and case[6] == "f32" else 1e-3)


def test_quantize_and_dequant_bits(run):
    packed, scales = run["want"]["quantize"]
    assert np.array_equal(run["get"]("q.packed", np.uint32), packed.ravel())
    assert np.array_equal(run["get"]("q.scales", np.uint16), scales.ravel())
    deq = O.dequant_int8_grouped(packed, scales, 96, 512, 64)
    assert np.array_equal(run["get"]("q.deq").view(np.uint32), deq.ravel().view(np.uint32))
    assert np.array_equal(run["get"]("q.deqdev").view(np.uint32), deq.ravel().view(np.uint32))
    assert run["results"]["cases"]["quantize"]["dequant"] == 1


@pytest.mark.parametrize("kind,first", [("rmsnorm_linear", ".norm"), ("gated_linear", ".prod")])
def test_producers_and_their_fused_form(run, kind, first):
    fx, want, shape = run["want"][kind]
    assert rel_l2(run["get"](kind + first).reshape(fx.shape), fx) <= 1e-3   # f16 tensors
    assert rel_l2(run["get"](kind + ".y").reshape(shape), want) <= 1e-3
    assert rel_l2(run["get"](kind + ".yapart").reshape(shape), want) <= 1e-3


@pytest.mark.parametrize("name", ["door_m1", "door_m64"])
def test_fused_side_door(run, name):
    """matmul -> bias -> silu -> cast handed over as one EpilogueConfig: one launch, and the
    four ways in (transposed view, transB, donated buffer, cached geometry) agree."""
    want, dtype, shape = run["want"][name]
    r = run["results"]["cases"][name]
    assert r["launches"] == 1 and r["dtype"] == dtype and r["donated_reused"] is True
    assert r["plan"] == "quantized-operand"           # planBareMatmul: webgpu/dispatch.ts:826
    if shape[0] > 1:
        assert "[M,N]" in r["binary_error"]              # an [N] tensor as a binary step's input is refused
    else:
        assert r["binary_error"] is None                 # one row: [N] is [M,N]
    assert "Unsupported binary epilogue: div" in r["binary_op_error"]   # matmul-skeleton.ts:953
    yr = run["get"](f"{name}.y_residual").reshape(shape)
    assert rel_l2(yr, run["want"][name + "_residual"]) <= (1e-5 if dtype == "f32" else 1e-3)
    ys = [run["get"](f"{name}.y{i}").reshape(shape) for i in range(4)]
    for y in ys:
        assert rel_l2(y, want) <= (1e-5 if dtype == "f32" else 1e-3)
        assert np.array_equal(y, ys[0])


def test_grouped_launch(run):
    for i in range(3):
        want = run["want"][f"grouped{i}"]
        assert rel_l2(run["get"](f"g{i}.y").reshape(want.shape), want) <= 1e-3


def test_grouped_launch_of_a_batched_step_and_the_no_alloc_entry_point(run):
    for i in range(3):
        want = run["want"][f"grouped8_{i}"]
        assert rel_l2(run["get"](f"g8_{i}.y").reshape(want.shape), want) <= 1e-3
    want = run["want"]["grouped8_0"]
    assert rel_l2(run["get"]("g8.noalloc").reshape(want.shape), want) <= 1e-3
    # linearInto writes a buffer of the caller's: one that is too short, or a bias that is,
    # is refused before anything is launched
    errors = run["results"]["cases"]["grouped8"]["into_errors"]
    assert len(errors) == 2 and "out must be a contiguous tensor of at least" in errors[0] and "bias must hold N" in errors[1]


def test_mlp_block_in_one_call(run):
    """mlpDecode: gate, up, silu(gate) * up and down from one call into the addon."""
    want, shape = run["want"]["mlp"]
    r = run["results"]["cases"]["mlp"]
    assert tuple(r["shape"]) == shape and r["dtype"] == "f16" and r["dispatches"] >= 2 and r["status"] == 0
    assert rel_l2(run["get"]("mlp.y").reshape(shape), want) <= 1e-3


def test_topk(run):
    logits = run["want"]["topk"]
    order = np.argsort(-logits, kind="stable")[:40]
    assert np.array_equal(run["get"]("t.indices", np.int32), order.astype(np.int32))
    assert np.array_equal(run["get"]("t.values"), logits[order])
    packed = run["get"]("t.packed")
    assert np.array_equal(packed[:40], logits[order]) and np.array_equal(packed[40:], order.astype(np.float32))


def test_errors_are_thrown_with_the_library_message(run):
    e = run["results"]["errors"]
    assert e["dimension_mismatch"]["message"] == "matmul dimension mismatch"
    assert "dense matmul" in e["dense_matmul"]["message"]
    assert "divisible by 4" in e["quantize_bad_k"]["message"] and e["quantize_bad_k"]["code"] == "TLHIP_1"
    assert e["bad_config"] is not None and e["bad_config"]["code"] == "TLHIP_1"
    assert "unknown weight format" in e["unknown_format"]["message"]


def test_tuning_cache_and_autotune_hooks(run):
    t = run["results"]["tuning"]
    assert t["exported_entries"] >= 1 and t["text_has_key"]
    assert t["selected_after_import"] == t["seeded"]
    assert run["results"]["autotune_enabled"] is True
    assert run["results"]["autotune_runs"] == 1


def test_backend_object_conforms_to_the_required_ops(run):
    """The Backend contract (src/backend/types.ts:340-696): every op the smallest conforming
    backend has (src/backend/mock/index.ts:150-176) is a function, `read` is a Promise of
    numbers (types.ts:666), and the ops outside the path are declared cpu delegates."""
    c = run["results"]["conformance"]
    mock_ops = ["tensorFromArray", "add", "sub", "div", "mul", "matmul", "sqrt", "relu", "expand", "reshape", "transpose",
                "permute", "contiguous", "max", "where", "stridedScatterCopy", "stridedScatterAdd", "gather", "scatterAdd",
                "sum", "mean", "read"]
    assert sorted(c["required"]) == sorted(mock_ops)
    assert c["missing"] == [] and c["name"] == "hip"
    assert c["read_is_promise"] and c["read_is_array"] and c["read_value"] == [1, 2, 3, 4, 5, 6]
    e = run["results"]["errors"]
    assert "sub is outside the quantized-weight linear path" in e["delegated_without_cpu"]["message"]
    assert "setCpuDelegate" in e["delegated_without_cpu"]["message"]
    assert "gather is outside" in e["delegated_unknown_to_cpu"]["message"]
    assert c["sub"] == [-5, -3, -1, 1, 3, 5] and c["sub_shape"] == [2, 3]
    assert c["sum"] == [21]
    assert c["transposed_contiguous"] is False
    assert c["transposed"] == [1, 4, 2, 5, 3, 6] and c["transposed_to_array"] == [1, 4, 2, 5, 3, 6]
