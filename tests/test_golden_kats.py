"""The known-answer vectors the reference's own tests hold for this path
(tests/golden/reference_kats.json: inputs and expected outputs, each with the
reference test it comes from), run against the oracle on the CPU and against
the HIP path on the GPU."""
import json
import os

import numpy as np
import pytest
import torch

import oracle

HERE = os.path.dirname(os.path.abspath(__file__))
KATS = json.load(open(os.path.join(HERE, "golden", "reference_kats.json")))
OPS = {"sum": oracle.OP_SUM, "avg": oracle.OP_AVG, "min": oracle.OP_MIN, "max": oracle.OP_MAX,
       "product": oracle.OP_PRODUCT}
DT = {"float32": (oracle.F32, np.float32, torch.float32), "float16": (oracle.F16, np.float16, torch.float16),
      "int64": (oracle.I64, np.int64, torch.int64), "int32": (oracle.I32, np.int32, torch.int32),
      "bool": (oracle.BOOL, np.uint8, torch.bool)}


def _np(vals, dtype):
    code, npdt, _ = DT[dtype]
    a = np.array(vals, dtype=npdt)
    return a.view(np.uint16) if dtype == "float16" else a


def _back(a, dtype):
    return a.view(np.float16).astype(np.float64) if dtype == "float16" else a.astype(np.float64)


# ---- oracle (CPU) --------------------------------------------------------------
@pytest.mark.parametrize("kat", KATS["binary"], ids=lambda k: f"{k['op']}-{k['dtype']}")
def test_oracle_binary(kat):
    a, b = _np(kat["a"], kat["dtype"]).copy(), _np(kat["b"], kat["dtype"])
    assert oracle.fold2(a, b, DT[kat["dtype"]][0], OPS[kat["op"]]) == oracle.OK
    assert np.array_equal(_back(a, kat["dtype"]), np.array(kat["expect"], dtype=np.float64))


@pytest.mark.parametrize("kat", KATS["uniform_binary"], ids=lambda k: f"{k['dtype']}-{k['sizes'][-1]}")
def test_oracle_uniform_binary(kat):
    for n in kat["sizes"]:
        a, b = _np([kat["a"]] * n, kat["dtype"]).copy(), _np([kat["b"]] * n, kat["dtype"])
        oracle.fold2(a, b, DT[kat["dtype"]][0], OPS[kat["op"]])
        assert np.all(_back(a, kat["dtype"]) == kat["expect"]), n


@pytest.mark.parametrize("kat", KATS["scale"], ids=lambda k: k["dtype"])
def test_oracle_scale(kat):
    a = _np(kat["a"], kat["dtype"]).copy()
    oracle.scale(a, DT[kat["dtype"]][0], float(np.float32(kat["scale"])), round_i32=True)
    assert np.array_equal(_back(a, kat["dtype"]), np.array(kat["expect"], dtype=np.float64))


def test_oracle_scale_world_sizes():
    k = KATS["scale_world_size"]
    for ws in k["world_sizes"]:
        a = np.full(k["n"], float(ws), dtype=np.float32)
        oracle.scale(a, oracle.F32, float(np.float32(1.0 / ws)))
        assert np.allclose(a, 1.0, rtol=k["rtol"], atol=k["rtol"]), ws


@pytest.mark.parametrize("kat", KATS["accumulate_and_scale"], ids=lambda k: k["dtype"])
def test_oracle_accumulate_and_scale(kat):
    code = DT[kat["dtype"]][0]
    a, b = _np(kat["a"], kat["dtype"]).copy(), _np(kat["b"], kat["dtype"])
    if kat["dtype"] in ("float32", "float16"):
        oracle.fold2_scale(a, b, code, kat["scale"])
    else:  # integral types: wrap-around add, then the integral scale rule
        oracle.fold2(a, b, code, oracle.OP_SUM)
        oracle.scale(a, code, kat["scale"], round_i32=True)
    assert np.array_equal(_back(a, kat["dtype"]), np.array(kat["expect"], dtype=np.float64))


@pytest.mark.parametrize("kat", KATS["allreduce_constants"], ids=lambda k: f"ws{k['world_size']}-{k['op']}")
def test_oracle_ring_constants(kat):
    ws, add = kat["world_size"], int(kat["rank_value"].split("+")[1])
    for n in kat.get("sizes", [100]):
        ins = [np.full(n, float(r + add), dtype=np.float32) for r in range(ws)]
        for schedule in (oracle.RING_BASIC, oracle.RING_CHUNKED):
            scale = float(np.float32(1.0 / ws)) if kat["op"] == "avg" else None
            out = oracle.ring_fold(ins, oracle.F32, OPS[kat["op"]], schedule, scale_by=scale)
            assert np.all(out == np.float32(kat["expect"])), (n, schedule)   # zero tolerance


def test_oracle_topk_wire_format():
    k = KATS["topk_wire"]
    n = 64
    g = np.zeros(n, dtype=np.float32)
    for idx, val in k["pairs"]:
        g[idx] = val
    wire, rc = oracle.topk_compress(g, np.zeros(n, np.float32), k["k"] / n)
    assert rc == 4 + 8 * k["k"] and wire.tobytes().hex() == k["bytes_hex"]
    dense, rc = oracle.topk_decompress(wire, n)
    assert rc == 0 and np.array_equal(dense, g)


# ---- HIP path (GPU) --------------------------------------------------------------
@pytest.fixture(scope="module")
def C():
    import torch.distributed  # noqa: F401
    from mccl_amd import _C
    return _C


def _t(vals, dtype):
    return torch.tensor(vals, dtype=DT[dtype][2], device="cuda:0")


@pytest.mark.gpu
def test_gpu_known_answers(C):
    fn = {"sum": C._metal_accumulate_chunk, "min": C._metal_elementwise_min, "max": C._metal_elementwise_max,
          "product": C._metal_elementwise_product}
    for kat in KATS["binary"]:
        got = fn[kat["op"]](_t(kat["a"], kat["dtype"]), _t(kat["b"], kat["dtype"]))
        assert torch.equal(got, _t(kat["expect"], kat["dtype"])), kat["ref"]
    for kat in KATS["uniform_binary"]:
        for n in kat["sizes"]:
            got = fn[kat["op"]](_t([kat["a"]] * n, kat["dtype"]), _t([kat["b"]] * n, kat["dtype"]))
            assert torch.equal(got, _t([kat["expect"]] * n, kat["dtype"])), (kat["ref"], n)
    for kat in KATS["scale"]:
        got = C._metal_scale_inplace(_t(kat["a"], kat["dtype"]), kat["scale"])
        assert torch.equal(got, _t(kat["expect"], kat["dtype"])), kat["ref"]
    for kat in KATS["accumulate_and_scale"]:
        got = C._metal_accumulate_and_scale(_t(kat["a"], kat["dtype"]), _t(kat["b"], kat["dtype"]), kat["scale"])
        assert torch.equal(got, _t(kat["expect"], kat["dtype"])), kat["ref"]
    k = KATS["scale_world_size"]
    for ws in k["world_sizes"]:
        got = C._metal_scale_inplace(torch.full((k["n"],), float(ws), device="cuda:0"), 1.0 / ws)
        assert torch.allclose(got, torch.ones_like(got), rtol=k["rtol"], atol=k["rtol"])


@pytest.mark.gpu
def test_gpu_allreduce_constants_and_wire(C):
    for kat in KATS["allreduce_constants"]:
        ws, add = kat["world_size"], int(kat["rank_value"].split("+")[1])
        g = C.LoopbackGroup(ws)
        for n in kat.get("sizes", [100]):
            ts = [torch.full((n,), float(r + add), device="cuda:0") for r in range(ws)]
            g.allreduce(ts, OPS[kat["op"]])
            for t in ts:
                assert float((t - kat["expect"]).abs().max()) == 0.0, kat["ref"]
    k = KATS["topk_wire"]
    n = 64
    gt = torch.zeros(n, device="cuda:0")
    for idx, val in k["pairs"]:
        gt[idx] = val
    comp = C.TopKCompressor(k["k"] / n)
    wire = comp.compress(gt)
    assert bytes(wire.cpu().numpy()).hex() == k["bytes_hex"]
    assert torch.equal(comp.decompress(wire, n), gt)
    e = KATS["fp16_e2e"]
    h = C.FP16Compressor()
    for n in e["sizes"]:
        total = torch.zeros(n, device="cuda:0")
        for r in range(3):
            total += h.decompress(h.compress(torch.full((n,), (r + 1) * 0.5, device="cuda:0")), n)
        assert int((total != 3.0).sum()) == 0
