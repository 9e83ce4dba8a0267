"""The `.rbw` snapshot reader: byte layout and parameter order as the reference writes them
(src/transformer.rs:1806-1932), the Q8 rule (`quantize`, :512-519), and — on the GPU — a sparse block
loaded from a Q8 file running on the int8 path."""
import json
import struct

import numpy as np
import pytest

from rustingbrain_amd import rbw, synth
from rustingbrain_amd.moe import InvalidConfig

CONFIG = dict(vocab_size=32, d_model=64, n_layers=3, n_heads=2, n_kv_heads=1, head_dim=16, d_ff=96, moe_d_ff=64,
              num_experts=4, experts_per_token=2, moe_layers=[1, 2], shared_expert=True, max_seq_len=16,
              rope_base=10000.0, rmsnorm_eps=1e-5, tie_embeddings=False, causal=True, aux_loss_weight=0.01,
              router_z_loss_weight=0.001, lora=None)


def model_params(c, seed=3):
    """f32 matrices in `params_mut()` order, plus the indices of the sparse blocks' parameters."""
    d, hd = c["d_model"], c["head_dim"]
    stream = [0]

    def m(rows, cols, std=0.05):
        stream[0] += 1
        return synth.normal((rows, cols), std, seed, stream[0])

    params, moe = [m(c["vocab_size"], d)], {}
    for b in range(c["n_layers"]):
        params += [np.ones((1, d), np.float32), m(c["n_heads"] * hd, d), m(c["n_kv_heads"] * hd, d),
                   m(c["n_kv_heads"] * hd, d), m(d, c["n_heads"] * hd),
                   (np.float32(1.0) + m(1, d, 0.1)).astype(np.float32)]  # feed_forward_norm: not all ones
        if b in c["moe_layers"]:
            start = len(params)
            params.append(m(c["num_experts"], d, 0.5))
            for _ in range(c["num_experts"] + (1 if c["shared_expert"] else 0)):
                params += [m(c["moe_d_ff"], d), m(c["moe_d_ff"], d), m(d, c["moe_d_ff"])]
            moe[b] = (start, len(params))
        else:
            params += [m(c["d_ff"], d), m(c["d_ff"], d), m(d, c["d_ff"])]
    params.append(np.ones((1, d), np.float32))
    if not c["tie_embeddings"]:
        params.append(m(c["vocab_size"], d))
    return params, moe


def test_byte_layout_is_the_reference_writers(tmp_path):
    p = tmp_path / "m.rbw"
    w = np.array([[1.0, -2.0, 0.5], [0.0, 0.0, 0.0]], np.float32)
    rbw.write(str(p), {"x": 1}, [w], "Q8")
    data = p.read_bytes()
    assert data[:8] == b"RBWTS001"
    (hlen,) = struct.unpack_from("<Q", data, 8)
    header = json.loads(data[16:16 + hlen])
    assert header["precision"] == "Q8" and header["config"] == {"x": 1}
    pos = 16 + hlen
    assert struct.unpack_from("<QQQ", data, pos) == (1, 2, 3)  # one parameter, 2 x 3
    pos += 24
    (scale,) = struct.unpack_from("<f", data, pos)
    assert scale == np.float32(2.0) / np.float32(127.0)
    assert list(np.frombuffer(data, np.int8, 3, pos + 4)) == [64, -127, 32]   # 63.5 rounds away from zero
    assert struct.unpack_from("<f", data, pos + 7) == (0.0,) and data[pos + 11:pos + 14] == b"\0\0\0"  # zero row
    assert len(data) == pos + 14


@pytest.mark.parametrize("precision", ["F32", "Q8"])
@pytest.mark.parametrize("tie", [False, True])
def test_round_trip_and_parameter_order(tmp_path, precision, tie):
    c = dict(CONFIG, tie_embeddings=tie)
    params, moe = model_params(c)
    path = str(tmp_path / "model.rbw")
    rbw.write(path, c, params, precision, optimizer_step=7)
    snap = rbw.read(path)
    assert snap.precision == precision and snap.optimizer_step == 7 and len(snap.params) == len(params)
    for got, want in zip(snap.params, params):
        if precision == "F32":
            assert np.array_equal(got.values, want)
        else:
            q, s = synth.quantize_rows(want)   # the same rule, written independently
            assert np.array_equal(got.q, q) and np.array_equal(got.scales, s)
            assert np.max(np.abs(got.dequantized() - want)) <= np.max(np.abs(want)) / 127 * 0.5 + 1e-7
    blocks = rbw.moe_blocks(snap)
    assert [b.block for b in blocks] == c["moe_layers"]
    for b in blocks:
        start, end = moe[b.block]
        assert b.router is snap.params[start]
        assert b.experts[0]["gate"] is snap.params[start + 1] and b.experts[0]["down"] is snap.params[start + 3]
        assert b.experts[3]["up"] is snap.params[start + 1 + 9 + 1]
        assert b.shared["down"] is snap.params[end - 1]


def test_rejects_what_the_reference_rejects(tmp_path):
    c = dict(CONFIG)
    params, _ = model_params(c)
    path = str(tmp_path / "model.rbw")
    rbw.write(path, c, params, "F32")
    blob = open(path, "rb").read()
    bad = str(tmp_path / "bad.rbw")
    open(bad, "wb").write(b"RBOPT001" + blob[8:])
    with pytest.raises(rbw.InvalidSnapshot, match="not a RustingBrain weight file"):
        rbw.read(bad)
    open(bad, "wb").write(blob[:-5])
    with pytest.raises(rbw.InvalidSnapshot, match="truncated"):
        rbw.read(bad)
    rbw.write(bad, c, params[:-1], "F32")
    with pytest.raises(rbw.InvalidSnapshot, match="parameters"):
        rbw.moe_blocks(rbw.read(bad))
    wrong = list(params)
    wrong[1 + 6] = np.zeros((5, 5), np.float32)  # block 0's gate matrix
    rbw.write(bad, c, wrong, "F32")
    with pytest.raises(rbw.InvalidSnapshot, match="5x5 parameter where the model has 96x64"):
        rbw.moe_blocks(rbw.read(bad))
    rbw.write(bad, dict(c, lora={"rank": 4, "alpha": 8.0, "seed": 1}), params, "F32")
    with pytest.raises(InvalidConfig, match="LoRA"):
        rbw.moe_blocks(rbw.read(bad))


@pytest.mark.gpu
@pytest.mark.parametrize("precision", ["Q8", "F32"])
def test_sparse_blocks_of_a_snapshot_run_on_the_device(tmp_path, device, precision):
    from conftest import rel_l2
    from helpers import assert_routing_identical
    from oracle import rb_oracle as orc
    c = dict(CONFIG)
    params, moe = model_params(c)
    path = str(tmp_path / "model.rbw")
    rbw.write(path, c, params, precision)
    layers = rbw.load_moe_layers(path, device, max_tokens=40)
    assert len(layers) == 2
    snap = rbw.read(path)
    x = synth.round_bf16(synth.normal((40, c["d_model"]), 1.0, 9, 1))
    for layer, blk in zip(layers, rbw.moe_blocks(snap)):
        def ew(ex):
            if precision == "Q8":
                return orc.ExpertWeights(gate_q=ex["gate"].q, gate_s=ex["gate"].scales, up_q=ex["up"].q,
                                         up_s=ex["up"].scales, down_q=ex["down"].q, down_s=ex["down"].scales)
            r = synth.round_bf16
            return orc.ExpertWeights(gate=r(ex["gate"].values), up=r(ex["up"].values), down=r(ex["down"].values))
        ref_layer = orc.OracleLayer(c["d_model"], c["num_experts"], c["experts_per_token"], c["moe_d_ff"],
                                    blk.router.dequantized(), [ew(e) for e in blk.experts], ew(blk.shared),
                                    c["moe_d_ff"], c["aux_loss_weight"], c["router_z_loss_weight"])
        ref = ref_layer.forward(x)
        out, cache = layer.forward_train(x)
        assert layer.kernel_name().startswith("mfma_bf16")
        assert_routing_identical(cache, ref)
        assert rel_l2(out, ref.out) <= 2e-2
        # the block step with the snapshot's own feed_forward_norm and rmsnorm_eps
        nw = blk.norm.dequantized().reshape(-1)
        want, _, ref_b = ref_layer.forward_block(x, nw, c["rmsnorm_eps"], round_normed=synth.round_bf16)
        out_b, cache_b = layer.forward_block(x)
        assert_routing_identical(cache_b, ref_b)
        assert rel_l2(out_b, want) <= 2e-2
        layer.close()


# ------------------------------------------------------------------ the C++ host mirror's reader (host/rbw.hpp)
def _cpp(*args):
    import os
    import subprocess
    from conftest import ROOT
    exe = os.path.join(ROOT, "rustingbrain_amd", "host", "moe_tutorial")
    if not os.path.exists(exe):
        from rustingbrain_amd import build
        build.build_host()
    return subprocess.run([exe, "--rbw", *args], capture_output=True, text=True, timeout=120)


def _checksum(p):
    return float(p.dequantized().astype(np.float64).sum())


@pytest.mark.parametrize("precision", ["F32", "Q8"])
def test_cpp_reader_sees_what_the_python_reader_sees(tmp_path, precision):
    c = dict(CONFIG)
    params, _ = model_params(c)
    path = str(tmp_path / "model.rbw")
    rbw.write(path, c, params, precision, optimizer_step=11)
    res = _cpp(path)
    assert res.returncode == 0, res.stdout + res.stderr
    lines = res.stdout.strip().splitlines()
    assert lines[0] == f"precision {precision} parameters {len(params)} optimizer_step 11"
    blocks = rbw.moe_blocks(rbw.read(path))
    assert len(lines) == 1 + len(blocks)
    for line, b in zip(lines[1:], blocks):
        f = line.split()
        assert f[:6] == ["block", str(b.block), "experts", str(len(b.experts)), "shared", "1"]
        got = dict(zip(f[6::2], (float(v) for v in f[7::2])))
        want = {"norm": _checksum(b.norm), "router": _checksum(b.router), "gate0": _checksum(b.experts[0]["gate"]),
                "down_last": _checksum(b.shared["down"])}
        for name, v in want.items():
            assert abs(got[name] - v) <= 1e-7 * max(1.0, abs(v)), (name, got[name], v)


def test_cpp_reader_rejects_what_the_reference_rejects(tmp_path):
    c = dict(CONFIG)
    params, _ = model_params(c)
    good = str(tmp_path / "model.rbw")
    rbw.write(good, c, params, "F32")
    blob = open(good, "rb").read()
    bad = str(tmp_path / "bad.rbw")
    for data, message in ((b"RBOPT001" + blob[8:], "not a RustingBrain weight file"), (blob[:-5], "truncated"),
                          (blob + b"\0\0", "bytes follow the last parameter")):
        open(bad, "wb").write(data)
        res = _cpp(bad)
        assert res.returncode == 2 and message in res.stdout, res.stdout
    rbw.write(bad, c, params[:-1], "F32")
    res = _cpp(bad)
    assert res.returncode == 2 and "parameters" in res.stdout
    wrong = list(params)
    wrong[1 + 6] = np.zeros((5, 5), np.float32)
    rbw.write(bad, c, wrong, "F32")
    res = _cpp(bad)
    assert res.returncode == 2 and "5x5 parameter where the model has 96x64" in res.stdout
    rbw.write(bad, dict(c, lora={"rank": 4, "alpha": 8.0, "seed": 1}), params, "F32")
    res = _cpp(bad)
    assert res.returncode == 2 and "LoRA" in res.stdout


@pytest.mark.gpu
@pytest.mark.parametrize("precision", ["Q8", "F32"])
def test_cpp_host_loads_a_snapshot_and_runs_the_block_step(tmp_path, device, precision):
    """Both hosts load the same file onto the device and run the same block step: identical bits."""
    c = dict(CONFIG)
    params, _ = model_params(c)
    path = str(tmp_path / "model.rbw")
    rbw.write(path, c, params, precision)
    x = synth.round_bf16(synth.normal((40, c["d_model"]), 1.0, 9, 1))
    rows = str(tmp_path / "rows.f32")
    x.astype("<f4").tofile(rows)
    out = str(tmp_path / "out")
    res = _cpp(path, rows, "40", out)
    assert res.returncode == 0, res.stdout + res.stderr
    layers = rbw.load_moe_layers(path, device, max_tokens=40)
    for layer, blk in zip(layers, rbw.moe_blocks(rbw.read(path))):
        want, _ = layer.forward_block(x)
        got = np.fromfile(f"{out}.{blk.block}", dtype="<f4").reshape(40, c["d_model"])
        assert np.array_equal(got, want)
        assert f"block {blk.block} ran on mfma_bf16" in res.stdout
        layer.close()
