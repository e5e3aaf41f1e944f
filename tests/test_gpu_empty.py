"""Empty inputs (zero batch / zero rows) through every op: shapes and dtypes of outputs and
gradients are those of the non-empty case, nothing is launched, nothing faults."""
import pytest
import torch

from slapo_amd import op

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_empty_inputs(dtype):
    dev = "cuda"
    q = torch.zeros(0, 16, 2, 64, dtype=dtype, device=dev, requires_grad=True)
    out = op.hip_attention(q, q, q, None, causal=True, p=0.1)
    assert out.shape == q.shape and out.dtype == dtype
    out.sum().backward()
    assert q.grad.shape == q.shape

    x = torch.zeros(0, 128, dtype=dtype, device=dev, requires_grad=True)
    b = torch.zeros(128, dtype=dtype, device=dev, requires_grad=True)
    w = torch.ones(128, dtype=dtype, device=dev, requires_grad=True)
    for y in (op.bias_gelu(x, b), op.bias_dropout_residual(x, b, x, 0.1, True),
              op.bias_dropout_residual_layer_norm(x, b, x, w, b, 0.1)):
        assert y.shape == x.shape and y.dtype == dtype
        y.sum().backward()
    assert x.grad.shape == x.shape
    assert torch.equal(b.grad, torch.zeros_like(b)) and torch.equal(w.grad, torch.zeros_like(w))

    logits = torch.zeros(0, 50, dtype=dtype, device=dev, requires_grad=True)
    loss = op.vocab_parallel_cross_entropy(logits, torch.zeros(0, dtype=torch.long, device=dev))
    assert loss.shape == (0,) and loss.dtype == torch.float32
    loss.sum().backward()
    assert logits.grad.shape == logits.shape
