"""The layer-level callers of the path (python/mlx/nn/layers/quantized.py)."""
import pytest
import torch

import mlx_amd
from mlx_amd import nn as qnn

pytestmark = pytest.mark.gpu


def _model(gpu, bias=True):
    return torch.nn.Sequential(
        torch.nn.Embedding(5, 256), torch.nn.ReLU(), torch.nn.Linear(256, 256, bias=bias)
    ).to(gpu)


def test_quantize_swaps_linear_and_embedding(gpu):
    # python/tests/test_nn.py:229-243
    m = qnn.quantize(_model(gpu))
    assert isinstance(m[0], qnn.QuantizedEmbedding)
    assert isinstance(m[1], torch.nn.ReLU)
    assert isinstance(m[2], qnn.QuantizedLinear)
    m = qnn.quantize(_model(gpu), class_predicate=lambda _, mod: isinstance(mod, torch.nn.Linear))
    assert isinstance(m[0], torch.nn.Embedding)
    assert isinstance(m[2], qnn.QuantizedLinear)
    m = qnn.quantize(_model(gpu), class_predicate=lambda p, mod: {"group_size": 32, "bits": 8}
                     if p == "2" else False)
    assert isinstance(m[0], torch.nn.Embedding)
    assert (m[2].group_size, m[2].bits) == (32, 8)
    with pytest.raises(ValueError):
        qnn.quantize(_model(gpu), group_size=32, mode="mxfp4")
    with pytest.raises(ValueError):
        qnn.quantize(_model(gpu), quantize_input=True)


def test_quantized_model_matches_dequantized_dense_model(gpu):
    torch.manual_seed(0)
    dense = _model(gpu)
    q = qnn.quantize(_model(gpu))
    q[0] = qnn.QuantizedEmbedding.from_embedding(dense[0])
    q[2] = qnn.QuantizedLinear.from_linear(dense[2])
    tokens = torch.tensor([[0, 3, 4], [1, 1, 2]], device=gpu)
    got = q(tokens)
    assert got.shape == (2, 3, 256)
    emb = mlx_amd.dequantize(q[0].weight, q[0].scales, q[0].biases)
    w = mlx_amd.dequantize(q[2].weight, q[2].scales, q[2].biases)
    ref = torch.relu(emb[tokens]).double() @ w.double().T + dense[2].bias.detach().double()
    assert float((got.double() - ref).abs().max()) < 1e-4
    # tied output projection
    h = torch.randn(4, 256, device=gpu)
    logits = q[0].as_linear(h)
    assert logits.shape == (4, 5)
    assert float((logits.double() - h.double() @ emb.double().T).abs().max()) < 1e-4


@pytest.mark.parametrize("bits", (2, 3, 4, 5, 6, 8))
def test_quantized_linear_shapes(gpu, bits):
    # python/tests/test_nn.py:268-281: packed width for every code width
    lin = torch.nn.Linear(1536, 1024).to(gpu)
    ql = qnn.QuantizedLinear.from_linear(lin, bits=bits)
    assert ql.weight.shape == (1024, 1536 * bits // 32)
    assert ql.scales.shape == ql.biases.shape == (1024, 1536 // 64)
    assert ql(torch.randn(3, 1536, device=gpu)).shape == (3, 1024)
    assert "bits=%d" % bits in repr(ql)
    fresh = qnn.QuantizedLinear(512, 64, bias=False, group_size=128, bits=bits, device=gpu,
                                dtype=torch.bfloat16)
    y = fresh(torch.randn(2, 7, 512, device=gpu, dtype=torch.bfloat16))
    assert y.shape == (2, 7, 64) and y.dtype == torch.bfloat16
