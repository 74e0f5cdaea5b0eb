"""`torch.ops.llmopt.w4a16_linear` (python/llmopt_backend/quantization.py:174-185) on ROCm tensors."""
import numpy as np
import pytest

import oracle
from tests.gpu_util import assert_close_to_oracle, w4_case

pytestmark = pytest.mark.gpu
torch = pytest.importorskip("torch")


@pytest.fixture(scope="module")
def op():
    import llmopt_amd.torch_ops  # noqa: F401  (registers the operator)
    return torch.ops.llmopt.w4a16_linear


@pytest.mark.parametrize("shape,n,k,bias", [((1, 576), 1536, 576, False), ((2, 3, 576), 192, 576, True),
                                            ((40, 1024), 1000, 1024, True)])
def test_matches_oracle(op, shape, n, k, bias):
    rng = np.random.default_rng(n)
    x, packed, scale, b = w4_case(rng, int(np.prod(shape[:-1])), n, k, bias=bias)
    device = torch.device("cuda:0")
    tx = torch.from_numpy(x.reshape(shape)).to(device)
    out = op(tx, torch.from_numpy(packed).to(device), torch.from_numpy(scale).to(device),
             torch.from_numpy(b).to(device) if bias else None)
    assert out.shape == (*shape[:-1], n) and out.dtype == torch.float16
    expected = oracle.w4a16_linear(x, packed, scale, b)
    assert_close_to_oracle(out.cpu().numpy().reshape(-1, n), expected, "torch op")


def test_reference_golden_fixture(op, golden):
    """python/tests/test_quantization.py:43-55 / python/examples/w4a16_linear_fx.json."""
    case = golden["w4a16_linear_fixture"]
    device = torch.device("cuda:0")
    packed = np.arange(96, dtype=np.uint8).reshape(3, 32)
    packed[0, 0] = 0x78
    scale = np.array(case["scale"], dtype=np.float16).reshape(3, 1)
    bias = np.array(case["bias"], dtype=np.float16)
    x = torch.ones((2, 64), dtype=torch.float16, device=device)
    out = op(x, torch.from_numpy(packed).to(device), torch.from_numpy(scale).to(device),
             torch.from_numpy(bias).to(device))
    assert out.cpu().numpy().view(np.uint16).reshape(-1).tolist() == case["expected_output_bits"]


def test_argument_checks(op):
    device = torch.device("cuda:0")
    packed = torch.zeros((8, 32), dtype=torch.uint8, device=device)
    scale = torch.ones((8, 1), dtype=torch.float16, device=device)
    with pytest.raises(TypeError, match="activations must be torch.float16"):
        op(torch.zeros((1, 64), dtype=torch.float32, device=device), packed, scale, None)
    with pytest.raises(TypeError, match="storage must be torch.uint8"):
        op(torch.zeros((1, 64), dtype=torch.float16, device=device), packed.to(torch.int8), scale, None)
    with pytest.raises(ValueError, match="scales must have shape"):
        op(torch.zeros((1, 64), dtype=torch.float16, device=device), packed, scale.reshape(1, 8), None)


def test_meta_kernel(op):
    out = op(torch.empty((5, 64), dtype=torch.float16, device="meta"),
             torch.empty((8, 32), dtype=torch.uint8, device="meta"),
             torch.empty((8, 1), dtype=torch.float16, device="meta"), None)
    assert out.shape == (5, 8) and out.dtype == torch.float16
