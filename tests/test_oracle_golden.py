"""The oracle against the reference's own known-answer vectors (CPU only)."""
import json
import os

import numpy as np


def _load(golden_dir, name):
    with open(os.path.join(golden_dir, name)) as f:
        return json.load(f)


def test_linear_forward_kat(oracle, golden_dir):
    k = _load(golden_dir, "linear_kat.json")
    y = oracle.linear_forward(np.array(k["input"]), np.array(k["projection"]), np.array(k["bias"]))
    assert np.array_equal(y, np.array(k["output"], dtype=np.float32))


def test_linear_backward_kat(oracle, golden_dir):
    k = _load(golden_dir, "linear_kat.json")
    dx, dw, db = oracle.linear_backward(np.array(k["output"]), np.array(k["output_grad"]),
                                        np.array(k["input"]), np.array(k["projection"]))
    assert np.array_equal(dx, np.array(k["input_grad"], dtype=np.float32))
    assert np.array_equal(dw, np.array(k["projection_grad"], dtype=np.float32))
    assert np.array_equal(db, np.array(k["bias_grad"], dtype=np.float32))


def test_tensor_accessor_kats(oracle, golden_dir):
    k = _load(golden_dir, "tensor_accessor_kat.json")
    s = k["scale"]
    assert np.array_equal(oracle.scale(np.array(s["input"]), s["constant"]),
                          np.array(s["output"], dtype=np.float32))
    r = k["relu"]
    assert np.array_equal(oracle.relu(np.array(r["input"])), np.array(r["output"], dtype=np.float32))
    t = k["transpose"]
    assert np.array_equal(oracle.transpose(np.array(t["input"])),
                          np.array(t["output"], dtype=np.float32))
    b = k["broadcast"]
    out = oracle.broadcast(np.array(b["input"]), b["output_dims"])
    want = np.tile(np.array(b["output_block"], dtype=np.float32), (4, 1, 1, 1))
    assert out.shape == tuple(b["output_dims"])
    assert np.array_equal(out, want)
    rd = k["reduce"]
    assert np.array_equal(oracle.reduce_dim(np.array(rd["input"]), 1),
                          np.array(rd["inner"], dtype=np.float32))
    assert np.array_equal(oracle.reduce_dim(np.array(rd["input"]), 0),
                          np.array(rd["outer"], dtype=np.float32))
    for case in k["offset"]:
        assert oracle.offset(case["dims"], case["coord"]) == case["offset"]


def test_philox_kat(oracle, golden_dir):
    k = _load(golden_dir, "philox_kat.json")
    for v in k["vectors"]:
        ctr = [int(x, 16) for x in v["ctr"]]
        key = [int(x, 16) for x in v["key"]]
        want = [int(x, 16) for x in v["out"]]
        got = oracle.philox4x32_10(ctr, key)
        assert [int(x) for x in got] == want, (v, [hex(int(x)) for x in got])
