"""The C++ host layer (include/autograph_hip.hpp), through its test program tests/cpp/host_mirror_test:
built by __graft_entry__.build() (and here on the CPU side when missing), run without a GPU for the
host-only logic and on the GPU for a LeNet5 forward pass, a transposed dot, an im2col/col2im round
trip and a pool backward, whose outputs are compared with the CPU oracle."""
import os
import subprocess

import numpy as np
import pytest

import oracle as orc

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BIN = os.path.join(ROOT, "tests", "cpp", "host_mirror_test")


def test_cpp_host_layer_cpu_checks():
    if not os.path.exists(BIN):
        subprocess.check_call(["make", "-s", "-C", os.path.dirname(BIN)])
    out = subprocess.run([BIN, "cpu"], capture_output=True, text=True, timeout=120)
    assert out.returncode == 0, out.stderr
    assert "cpu ok" in out.stdout


def he(rng, shape, fan_in):
    a = np.sqrt(2.0 / fan_in)
    return rng.uniform(-a, a, shape).astype(np.float32)


@pytest.mark.gpu
def test_cpp_host_layer_on_gpu(tmp_path):
    assert os.path.exists(BIN), "tests/cpp/host_mirror_test has not been built (run __graft_entry__.build())"
    from test_gpu_layers import oracle_lenet_bf16
    rng = np.random.default_rng(51)
    bs = 64
    x = rng.uniform(0, 1, (bs, 1, 28, 28)).astype(np.float32)
    params = [he(rng, (6, 1, 5, 5), 25), he(rng, (16, 6, 5, 5), 150), he(rng, (256, 128), 256), he(rng, (128, 84), 128),
              he(rng, (84, 10), 84), he(rng, (10,), 84)]
    a, b = rng.standard_normal((37, 53)).astype(np.float32), rng.standard_normal((41, 53)).astype(np.float32)
    fin, fout = tmp_path / "in.bin", tmp_path / "out.bin"
    with open(fin, "wb") as f:
        np.float32(bs).tofile(f)
        for arr in [x] + params + [a, b]:
            arr.tofile(f)
    run = subprocess.run([BIN, "gpu", str(fin), str(fout)], capture_output=True, text=True, timeout=300)
    assert run.returncode == 0, run.stderr + run.stdout
    out = np.fromfile(fout, dtype=np.float32)
    pos = 0

    def take(*shape):
        nonlocal pos
        n = int(np.prod(shape))
        v = out[pos:pos + n].reshape(shape)
        pos += n
        return v

    want = orc.lenet5_forward_f32(x, *params)
    tol = 2e-4 * max(1.0, np.abs(want).max())
    assert np.abs(take(bs, 10) - want).max() <= tol       # layer by layer
    assert np.abs(take(bs, 10) - want).max() <= tol       # single launch
    p16 = [orc.f32_to_bf16(p) for p in params]
    want16 = orc.bf16_to_f32(oracle_lenet_bf16(orc.f32_to_bf16(x), p16)).astype(np.float64)
    assert np.abs(take(bs, 10) - want16).max() <= 0.05 * max(1.0, np.abs(want16).max())
    dot = take(37, 41)
    exact = a.astype(np.float64) @ b.T.astype(np.float64)
    assert np.all(np.abs(dot - exact) <= 1e-5 * np.sqrt(53) * (np.abs(a).astype(np.float64) @ np.abs(b.T).astype(np.float64)))
    assert np.array_equal(take(bs, 1, 28, 28), orc.col2im_conv2(orc.im2col_conv2(x, (5, 5)), (24, 24), (5, 5)))
    act = take(bs, 6, 24, 24)
    grad = take(bs, 6, 24, 24)
    assert pos == out.size
    assert np.array_equal(grad, orc.max_pool2_backward(act, np.ones((bs, 6, 12, 12), dtype=np.float32), (2, 2)))
