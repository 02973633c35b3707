"""CPU checks for the fused-epilogue / gated-projection slice: the oracle's
activation formulas against torch's library routines, closed forms, and the host
logic that decides which regions the gfx950 candidate accepts."""
import numpy as np
import pytest
import torch

import standin_host as host
import tessera_oracle as orc
from tessera_amd import candidates as cand
from tessera_amd import ops


def test_epilogue_vocabulary_matches_torch():
    x = np.linspace(-12, 12, 4001)
    t = torch.from_numpy(x)
    F = torch.nn.functional
    lib = {"relu": F.relu(t), "gelu": F.gelu(t, approximate="tanh"), "silu": F.silu(t),
           "sigmoid": torch.sigmoid(t), "tanh": torch.tanh(t)}
    for name, want in lib.items():
        assert np.allclose(orc.EPILOGUE_REFS[name](x), want.numpy(), atol=1e-12), name
        assert np.allclose(host.POINTWISE[name](x), want.numpy(), atol=1e-12), name


def test_fused_epilogue_order_and_closed_forms():
    A = np.array([[1.0, -2.0]])
    B = np.array([[3.0], [1.0]])                       # A @ B = 1
    bias = np.array([-4.0])
    # order matters: relu(1 - 4) = 0 but relu(1) - 4 = -3
    assert orc.fused_epilogue(A, B, bias, ("bias", "relu"))[0, 0] == 0.0
    assert orc.fused_epilogue(A, B, bias, ("relu", "bias"))[0, 0] == -3.0
    assert orc.fused_epilogue(A, B, None, ())[0, 0] == 1.0
    with pytest.raises(ValueError):
        orc.fused_epilogue(A, B, None, ("bias",))
    # gated: act on the gate branch only
    Wg, Wu = np.array([[0.0], [0.0]]), np.array([[5.0], [0.0]])
    assert orc.gated_matmul(A, Wg, Wu, "sigmoid")[0, 0] == pytest.approx(0.5 * 5.0)
    assert orc.gated_matmul(A, Wg, Wu, "silu")[0, 0] == 0.0
    # the oracle agrees with the region classes' own numpy definitions
    rng = np.random.default_rng(0)
    a, b = rng.standard_normal((8, 12)), rng.standard_normal((12, 16))
    bi = rng.standard_normal(16)
    r = host.FusedRegion(epilogue=("bias", "gelu"))
    assert np.allclose(r.reference(a, b, bi), orc.fused_epilogue(a, b, bi, ("bias", "gelu")), atol=1e-5)
    g = host.GatedMatmulRegion("silu")
    assert np.allclose(g.reference(a, b, b[:, ::-1]), orc.gated_matmul(a, b, b[:, ::-1], "silu"), atol=1e-5)


def test_mfma_epilogue_representability():
    R = host.FusedRegion
    assert cand.fused_epilogue_plan(R(epilogue=("bias",))) == (True, "none")
    assert cand.fused_epilogue_plan(R(epilogue=("bias", "silu"))) == (True, "silu")
    assert cand.fused_epilogue_plan(R(epilogue=("tanh",))) == (False, "tanh")
    assert cand.fused_epilogue_plan(R(epilogue=("relu", "bias"))) is None          # bias after activation
    assert cand.fused_epilogue_plan(R(epilogue=("relu", "gelu"))) is None          # two activations
    assert cand.fused_epilogue_plan(R(epilogue=("relu",), residual=True)) is None
    assert cand.fused_epilogue_plan(R(epilogue=("relu",), reduction="softmax")) is None
    assert cand.fused_epilogue_plan(R(epilogue=("relu",), prologue=("gelu",))) is None
    assert cand.fused_epilogue_plan(host.MatmulRegion()) is None
    with pytest.raises(ValueError):
        R(epilogue=("swish",))
    with pytest.raises(ValueError):
        R(epilogue=("bias", "bias"))
    with pytest.raises(ValueError):
        host.GatedMatmulRegion("bias")


def test_host_argument_checks_need_no_device():
    a = np.zeros((4, 8), np.float16)
    with pytest.raises(ValueError):
        ops.fused_gemm(a, np.zeros((8, 4), np.float16), None, "softmax")
    with pytest.raises(ValueError):
        ops.fused_gemm(a, np.zeros((8, 4), np.float16), np.zeros(5, np.float32), "relu")
    with pytest.raises(ValueError):
        ops.fused_gemm(a, np.zeros((7, 4), np.float16))
    with pytest.raises(ValueError):
        ops.gated_gemm(a, np.zeros((8, 4), np.float16), np.zeros((8, 5), np.float16))
    with pytest.raises(ValueError):
        ops.gated_gemm(a, np.zeros((8, 4), np.float16), np.zeros((8, 4), np.float16), "none")
