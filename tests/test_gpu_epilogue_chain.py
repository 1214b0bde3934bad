"""GPU parity: the whole EpilogueConfig op set (matmul/types.ts:13-24) on every kernel
family: bias, unary, binary add / sub / mul with an [M,N] input (a residual, a gate), and a
cast to f16 inside the chain (matmul-skeleton.ts:916-966).

The oracle is the reference's unfused sequence: the CPU matmul (f64 accumulate, f32 store),
then each op as its own f32 elementwise pass.  Tolerances as for the plain epilogues:
rel-L2 <= 2e-6 for f32 outputs of the decode kernels on f16 activations, <= 1e-3 wherever
the prefill kernels' f16 rounding of a weight or an f16 store takes part."""
import numpy as np
import pytest

import torchlette_amd as T
from oracle import quant_oracle as O
from torchlette_amd import _lib as L
from helpers import f16_round, fmt_name, make_weight, make_x, rel_l2

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def be():
    return T.getBackend()


def f32(a):
    return np.asarray(a, np.float32)


def chain_oracle(lin, ops):
    """lin: the matmul's f32 output; ops as the test names them, host arrays inside."""
    v = f32(lin)
    for op in ops:
        if op[0] == "bias":
            v = f32(v + f32(op[1])[None, :])
        elif op[0] == "unary":
            v = O.unary(op[1], v)
        elif op[0] == "binary":
            b = f32(op[2])
            v = f32(v + b) if op[1] == "add" else (f32(v - b) if op[1] == "sub" else f32(v * b))
        elif op[0] == "cast":
            v = f32(v.astype(np.float16))
    return v


def run_chain(be, fmt, g, m, n, k, ops, xdt="f16", ydt="f32", config=None, seed=0):
    rng = np.random.default_rng(seed)
    packed, scales, deq = make_weight(fmt, n, k, g, rng)
    x = make_x(m, k, xdt, rng, std=0.5)
    host_ops, dev_ops, keep = [], [], []
    for op in ops:
        if op[0] == "bias":
            h = f16_round(rng.standard_normal(n) * 0.1)
            t = be.ops.tensorFromArray(h.astype(np.float16 if op[1] == "f16" else np.float32), [n], op[1])
            host_ops.append(("bias", h)); dev_ops.append(("bias", t)); keep.append(t)
        elif op[0] == "binary":
            h = f16_round(rng.standard_normal((m, n)))
            t = be.ops.tensorFromArray(h.astype(np.float16 if op[2] == "f16" else np.float32), [m, n], op[2])
            host_ops.append(("binary", op[1], h)); dev_ops.append(("binary", op[1], t)); keep.append(t)
        else:
            host_ops.append(op); dev_ops.append(op)
    w = be.createQuantizedWeight(packed, scales, n, k, T.resolveWeightFormat(fmt_name(fmt, g), ydt))
    xt = be.ops.tensorFromArray(x, [m, k], xdt)
    ep = be.makeEpilogueChain(dev_ops)
    y = be._matmulQuantizedB(xt, be.ops.transpose(w), ep, L.KernelConfig.of(*config) if config else None)
    got = y.numpy()
    lin = O.linear(x.astype(np.float32), deq, None, "none", threads=8)
    want = chain_oracle(lin, host_ops)
    for t in keep + [y, xt, w]:
        t.destroy()
    return got, want


CHAINS = [
    [("bias", "f16"), ("unary", "silu"), ("binary", "add", "f32")],                  # Linear + activation + residual
    [("binary", "mul", "f16")],                                                       # a gate
    [("bias", "f32"), ("binary", "sub", "f32"), ("unary", "gelu"), ("binary", "mul", "f32")],
    [("unary", "relu"), ("cast", "f16"), ("binary", "add", "f32")],
]


@pytest.mark.parametrize("chain", range(len(CHAINS)))
@pytest.mark.parametrize("fmt,g,m,n,k,config", [
    ("int4-grouped", 32, 1, 300, 512, None),                          # VALU decode kernel
    ("int4-grouped", 32, 3, 300, 512, (0, 16, 1, 4, 1, 2)),           # VALU kernel, several rows per pass
    ("int8-row", 0, 7, 515, 1024, None),                              # VALU passes of four rows / skinny matrix-core kernel
    ("int8-grouped", 64, 16, 1000, 2048, None),                       # skinny matrix-core kernel
    ("int4-grouped", 32, 16, 512, 4096, (1, 8, 2, 4, 4)),             # ... with K slices across workgroups
    ("int4-grouped", 32, 40, 256, 1024, (1, 8, 2, 8, 1)),             # ... 17..64 rows in one launch
    ("int4-grouped", 32, 12, 256, 1024, (4, 8, 1, 1, 1)),             # activations in registers
    ("int4-grouped", 128, 130, 333, 1024, (3, 128, 128, 128, 2, 2)),  # direct GEMM
    ("int8-row", 0, 300, 520, 512, (3, 256, 128, 128, 2, 4, 2)),      # direct GEMM, K slices (second launch runs the chain)
    ("int8-grouped", 64, 100, 384, 1024, (2, 128, 128, 64, 2, 2)),    # staged GEMM
    ("int8-grouped", 128, 70, 256, 2048, (2, 64, 128, 64, 2, 2, 4)),  # staged GEMM, K slices
    ("int4-grouped", 32, 100, 1000, 4096, None),                      # routing: rows in chunks of 64 through the decode kernel
])
def test_epilogue_chain_on_every_kernel(be, fmt, g, m, n, k, config, chain):
    got, want = run_chain(be, fmt, g, m, n, k, CHAINS[chain], config=config, seed=chain + m)
    assert got.shape == (m, n)
    tiled = config is not None and config[0] in (2, 3) or (config is None and m > 16)
    tol = 1e-3 if tiled or any(op[0] == "cast" for op in CHAINS[chain]) else 5e-6
    assert rel_l2(got, want) <= tol, rel_l2(got, want)


@pytest.mark.parametrize("m", [20, 150])
def test_epilogue_chain_on_f32_activations_in_chunks(be, m):
    """f32 activations above 16 rows are cast and run in chunks of rows: the [M,N] input of
    a binary step has to move with the chunk."""
    got, want = run_chain(be, "int4-grouped", 32, m, 777, 256, CHAINS[0], xdt="f32", seed=m)
    assert rel_l2(got, want) <= 1e-3, rel_l2(got, want)


def test_epilogue_chain_f16_output(be):
    got, want = run_chain(be, "int4-grouped", 32, 64, 512, 512, CHAINS[0], ydt="f16", config=(3, 128, 128, 128, 2, 2))
    assert got.dtype == np.float16 and rel_l2(got, want) <= 1e-3


@pytest.mark.parametrize("chain", range(len(CHAINS)))
@pytest.mark.parametrize("ydt", ["f32", "f16"])
def test_a_binary_step_on_a_large_output_runs_behind_the_gemm(be, chain, ydt):
    """From 4 M output elements on the chain is cut at its first binary step: the GEMM runs
    the steps before it, one elementwise launch the rest, in place.  Same results as the
    unfused sequence (an f16 output is rounded once more in between), and as the chain
    inside the GEMM, which an explicit kernel config still runs."""
    m, n, k = 1024, 4096, 256
    got, want = run_chain(be, "int4-grouped", 32, m, n, k, CHAINS[chain], ydt=ydt, seed=40 + chain)
    assert got.shape == (m, n) and got.dtype == (np.float16 if ydt == "f16" else np.float32)
    assert rel_l2(got, want) <= 1e-3, rel_l2(got, want)
    fused, _ = run_chain(be, "int4-grouped", 32, m, n, k, CHAINS[chain], ydt=ydt, seed=40 + chain, config=(3, 128, 128, 128, 2, 2))
    assert rel_l2(got, fused) <= (1e-3 if ydt == "f16" else 2e-6), rel_l2(got, fused)


def test_a_binary_step_stays_in_the_gemm_where_the_tail_cannot_run(be):
    """N not a multiple of 8: no 16-byte pieces of a row, the chain stays in the GEMM."""
    got, want = run_chain(be, "int4-grouped", 32, 1100, 4004, 256, CHAINS[0], seed=7)
    assert rel_l2(got, want) <= 1e-3, rel_l2(got, want)


def test_epilogue_chain_rejects(be):
    rng = np.random.default_rng(1)
    packed, scales, _ = make_weight("int4-grouped", 64, 256, 32, rng)
    w = be.createQuantizedWeight(packed, scales, 64, 256, T.resolveWeightFormat("int4-32", "f32"))
    xt = be.ops.tensorFromArray(make_x(2, 256, "f16", rng), [2, 256], "f16")
    ep = L.Epilogue()
    ep.n_ops = 1
    ep.ops[0] = L.EpilogueOp(L.EPI_BINARY, 0, None, L.F32, 2)
    with pytest.raises(L.TlhipError, match="binary epilogue without input"):
        be._matmulQuantizedB(xt, be.ops.transpose(w), ep, None)
    r = be.ops.tensorFromArray(np.zeros((2, 64), np.float32), [2, 64], "f32")
    ep.ops[0] = L.EpilogueOp(L.EPI_BINARY, 7, r.ptr, L.F32, 2)
    with pytest.raises(L.TlhipError, match="unknown binary epilogue op"):
        be._matmulQuantizedB(xt, be.ops.transpose(w), ep, None)
    ep.ops[0] = L.EpilogueOp(9, 0, None, 0, 0)
    with pytest.raises(L.TlhipError, match="unknown epilogue op kind"):
        be._matmulQuantizedB(xt, be.ops.transpose(w), ep, None)
    with pytest.raises(ValueError, match="Unsupported binary epilogue"):
        be.makeEpilogueChain([("binary", "div", r)])
    # an [N] tensor where the [M,N] one belongs would be read out of bounds: refused on the host
    b = be.ops.tensorFromArray(np.zeros(64, np.float32), [64], "f32")
    with pytest.raises(ValueError, match=r"must be an \[M,N\]"):
        be._matmulQuantizedB(xt, be.ops.transpose(w), be.makeEpilogueChain([("binary", "mul", b)]), None)
