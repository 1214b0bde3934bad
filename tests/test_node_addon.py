"""The N-API addon without a GPU: it is built, loads under the image's Node, exports
what hip_backend.js calls, runs the host-side routines, and reports a missing device
(or a call before init) as a thrown Error with the library's message and code."""
import json
import os
import re
import shutil
import subprocess

import numpy as np
import pytest

from oracle import quant_oracle as O

HERE = os.path.dirname(os.path.abspath(__file__))
ADDON_DIR = os.path.join(HERE, "..", "torchlette_amd", "addon")

node = shutil.which("node")
pytestmark = pytest.mark.skipif(node is None, reason="no node binary on this machine")


def run_js(code: str) -> dict:
    proc = subprocess.run([node, "-e", code], capture_output=True, text=True, timeout=120, cwd=ADDON_DIR)
    assert proc.returncode == 0, proc.stderr[-3000:]
    return json.loads(proc.stdout.strip().splitlines()[-1])


def test_addon_is_built_and_exports_what_the_backend_calls():
    assert os.path.exists(os.path.join(ADDON_DIR, "tlhip_napi.node")), "run __graft_entry__.build()"
    exported = set(run_js('console.log(JSON.stringify(Object.keys(require("./tlhip_napi.node"))))'))
    with open(os.path.join(ADDON_DIR, "hip_backend.js")) as f:
        used = set(re.findall(r"\btl\.([A-Za-z0-9_]+)", f.read()))
    assert used and used <= exported, sorted(used - exported)


def test_host_routines_match_the_oracle():
    rng = np.random.default_rng(0)
    w = (rng.random((4, 128)) * 2 - 1).astype(np.float32)
    out = run_js(f'''
      const tl = require("./tlhip_napi.node");
      const q = tl.quantizeInt8Grouped(new Float32Array({json.dumps([float(v) for v in w.ravel()])}), 4, 128, 64);
      console.log(JSON.stringify({{packed: Array.from(q.packed), scales: Array.from(q.scales),
        bits: [1.0, -2.5, 65504, 1e-8, 6.1e-5].map((v) => tl.f32ToF16Bits(v)),
        back: [0x3c00, 0xc100, 0x7bff, 0x0001].map((b) => tl.f16BitsToF32(b))}}));''')
    packed, scales = O.quantize_int8_grouped(w, 4, 128, 64)
    assert out["packed"] == [int(v) for v in packed.ravel()]
    assert out["scales"] == [int(v) for v in scales.ravel()]
    assert out["bits"] == [int(v) for v in O.f32_to_f16_bits(np.array([1.0, -2.5, 65504, 1e-8, 6.1e-5], np.float32))]
    assert out["back"] == [1.0, -2.5, 65504.0, 2.0 ** -24]


def test_failures_are_thrown_errors():
    out = run_js('''
      const tl = require("./tlhip_napi.node");
      const r = {};
      try { tl.quantizeInt8Grouped(new Float32Array(6), 2, 3, 64); } catch (e) { r.k = [e.code, e.message]; }
      try { tl.malloc("16"); } catch (e) { r.type = [e.name, e.message]; }
      let inited = true;
      try { tl.init(0); } catch (e) { inited = false; r.init = [e.code, e.message]; }
      if (!inited) { try { tl.malloc(16); } catch (e) { r.state = [e.code, e.message]; } }
      r.inited = inited;
      console.log(JSON.stringify(r));''')
    assert out["k"][0] == "TLHIP_1" and "divisible by 4" in out["k"][1]
    assert out["type"][0] == "TypeError"
    if not out["inited"]:  # no GPU here: no silent CPU path
        assert out["init"][0] == "TLHIP_2" and "no CPU fallback" in out["init"][1]
        assert out["state"][0] == "TLHIP_3"
