"""Host-side mirror of the reference's operator interface (CPU only): constructor signatures,
attribute / child names, error behaviour, class-name contract, RNG tracker state machine.
Assertions restate what the reference's callers rely on (slapo/model_schedule/gpt2.py:212-239,
:452-520; slapo/tracer.py:626-635; tests/test_random.py:23-63)."""
import inspect

import pytest
import torch
from torch import nn

import slapo_amd
from slapo_amd import op
from slapo_amd.random import CudaRNGStatesTracker


def _params(fn):
    return [(p.name, p.default) for p in inspect.signature(fn).parameters.values()
            if p.name != "self"]


def test_constructor_and_forward_signatures():
    E = inspect.Parameter.empty
    assert _params(op.FlashAttentionOp.__init__)[:3] == [
        ("attn_op_name", E), ("apply_causal_mask", E), ("scale", None)]
    assert _params(op.FlashAttentionOp.forward) == [
        ("query_layer", E), ("key_layer", E), ("value_layer", E), ("attention_mask", E), ("p", E)]
    assert _params(op.FlashAttention.__init__)[:8] == [
        ("hidden_size", E), ("num_attention_heads", E), ("attn_pdrop", 0.0), ("resid_pdrop", 0.0),
        ("attn_op_name", "auto"), ("bias", True), ("output_proj", True), ("fused_qkv", False)]
    assert _params(op.FlashAttention.forward) == [
        ("hidden_states", E), ("attention_mask", None), ("layer_past", None), ("head_mask", None),
        ("encoder_hidden_states", None), ("encoder_attention_mask", None), ("use_cache", False),
        ("output_attentions", False)]
    assert _params(op.FusedMLP.__init__) == [
        ("hidden_size", E), ("intermediate_size", E), ("orig_act", E), ("resid_pdrop", E),
        ("use_torchscript", False)]
    assert _params(op.LinearWithAct.__init__) == [
        ("in_features", E), ("out_features", E), ("bias", True), ("act_fn", "gelu"),
        ("device", None), ("dtype", None), ("sync_fn", None)]
    assert _params(op.LinearWithDropout.__init__) == [
        ("in_features", E), ("out_features", E), ("bias", True), ("p", 0.5), ("inplace", False),
        ("device", None), ("dtype", None), ("sync_fn", None), ("use_torchscript", False)]
    assert _params(op.bias_dropout) == [
        ("x", E), ("bias", E), ("p", 0.5), ("training", True), ("inplace", False)]


def test_attention_module_children_and_attributes():
    # kwargs exactly as the GPT-2 schedule passes them (model_schedule/gpt2.py:212-220)
    m = op.FlashAttention(hidden_size=64, num_attention_heads=4, output_proj=True, attn_pdrop=0.1,
                          resid_pdrop=0.1, attn_op_name="hip_cdna4", fused_qkv=True)
    assert set(dict(m.named_children())) == {"qkv", "out_proj", "resid_dropout", "attn_op"}
    assert m.qkv.out_features == 192 and m.attn_op.apply_causal_mask is True
    assert m.bias_layout == m.attn_op.bias_layout == "b11k"
    assert m.attn_op.pkg == "hip" and callable(m.attn_op.attn_fn)
    # BERT style (model_schedule/bert.py:165-174): no projection -> bidirectional, separate q/k/v
    e = op.FlashAttention(64, 4, output_proj=False, fused_qkv=False)
    assert set(dict(e.named_children())) == {"query", "key", "value", "attn_op"}
    assert e.attn_op.apply_causal_mask is False
    mlp = op.FusedMLP(16, 64, "gelu_new", 0.1)
    assert set(dict(mlp.named_children())) == {"fc_in", "fc_out"}
    assert mlp.fc_in.act_fn == "gelu" and mlp.fc_out.p == 0.1
    assert mlp.fc_in.sync_fn is None and mlp.fc_out.sync_fn is None
    mlp.fc_out.sync_fn = lambda x: x  # schedules assign it after construction
    assert "sync_fn=<lambda>" in repr(mlp.fc_out)


def test_class_name_contract_for_leaf_matching():
    # the reference's tracer matches substrings of type(m).__name__
    assert "FlashAttentionOp" in type(op.FlashAttentionOp("hip_cdna4", True)).__name__
    assert "LinearWithAct" in type(op.LinearWithAct(4, 4)).__name__
    assert "LinearWithDropout" in type(op.LinearWithDropout(4, 4)).__name__
    assert op.LinearWithSyncFunc(4, 4).traceable is False


def test_error_behaviour():
    with pytest.raises(ValueError):
        op.FlashAttention(30, 4)
    with pytest.raises(ValueError):
        op.FlashAttentionOp("no_such_kernel", True)
    with pytest.raises(ValueError):
        op.FlashAttentionOp("native_xformers", True)
    with pytest.raises(ValueError):
        op.LinearWithAct(4, 4, bias=False)
    with pytest.raises(ValueError):
        op.LinearWithDropout(4, 4, bias=False)
    with pytest.raises(NotImplementedError):
        op.LinearWithAct(4, 4, act_fn="relu")
    m = op.FlashAttention(16, 2, attn_op_name="hip_cdna4")
    x = torch.zeros(1, 4, 16)
    with pytest.raises(NotImplementedError):
        m(x, encoder_hidden_states=x)
    with pytest.raises(NotImplementedError):
        m(x, output_attentions=True)
    with pytest.raises(NotImplementedError):
        m(x, head_mask=torch.ones(2))


def test_third_party_names_are_aliases():
    # schedules fall back to "cutlass" when a constructor raises (gpt2.py:229-239)
    for name in ("cutlass", "flash", "triton", "cuda", "small_k", "auto"):
        assert op.FlashAttentionOp(name, True).pkg == "hip"


def test_no_cpu_fallback():
    """CPU tensors are refused loudly: the package has no eager substitute for its kernels."""
    with pytest.raises(RuntimeError, match="gfx950"):
        op.bias_gelu(torch.zeros(4, 8), torch.zeros(8))
    with pytest.raises(RuntimeError, match="gfx950"):
        op.bias_dropout(torch.zeros(4, 8), torch.zeros(8), 0.0, False)
    with pytest.raises(RuntimeError, match="gfx950"):
        op.hip_attention(*(torch.zeros(1, 8, 1, 8, dtype=torch.float16) for _ in range(3)))
    mlp = op.FusedMLP(8, 32, "gelu", 0.0)
    with pytest.raises(RuntimeError, match="gfx950"):
        mlp(torch.zeros(2, 8))
    with pytest.raises(RuntimeError, match="gfx950"):
        op.bias_dropout_residual_layer_norm(torch.zeros(4, 8), torch.zeros(8), torch.zeros(4, 8),
                                            torch.ones(8), torch.zeros(8), 0.0)
    with pytest.raises(RuntimeError, match="gfx950"):
        op.ParallelCrossEntropy()(torch.zeros(4, 8), torch.zeros(4, dtype=torch.long))


def test_layer_norm_fusion_module_and_cross_entropy_interfaces():
    """The LayerNorm payload carries nn.LayerNorm's parameter names (a state_dict of the module it
    replaces loads into it); ParallelCrossEntropy keeps the reference's constructor and forward
    (slapo/op/cross_entropy.py:153-160) and its helper for the vocabulary range (:11-14)."""
    ln = nn.LayerNorm(16, eps=1e-6)
    fused = op.HipBiasDropoutResidualLayerNorm.from_layer_norm(ln, p=0.25)
    assert fused.weight is ln.weight and fused.bias is ln.bias
    assert (fused.p, fused.eps, fused.normalized_shape) == (0.25, 1e-6, (16,))
    fresh = op.HipBiasDropoutResidualLayerNorm(16, 0.1)
    fresh.load_state_dict(ln.state_dict())
    assert _params(fresh.forward) == [("x", inspect.Parameter.empty),
                                      ("bias", inspect.Parameter.empty),
                                      ("residual", inspect.Parameter.empty)]
    with pytest.raises(ValueError):
        op.HipBiasDropoutResidualLayerNorm(16, 1.5)
    with pytest.raises(NotImplementedError):
        op.HipBiasDropoutResidualLayerNorm((4, 16), 0.1)
    with pytest.raises(NotImplementedError):
        op.HipBiasDropoutResidualLayerNorm.from_layer_norm(
            nn.LayerNorm(16, elementwise_affine=False), 0.1)

    from slapo_amd.op import cross_entropy as CE

    assert _params(op.ParallelCrossEntropy.__init__) == [("group", None)]
    assert [n for n, _ in _params(op.ParallelCrossEntropy.forward)] == ["outputs", "labels"]
    assert _params(op.vocab_parallel_cross_entropy) == [
        ("vocab_parallel_logits", inspect.Parameter.empty), ("target", inspect.Parameter.empty),
        ("label_smoothing", 0.0), ("group", None)]
    assert CE.vocab_range_from_per_partition_vocab_size(100, 3, 8) == (300, 400)


def test_meta_device_construction():
    # schedules build the modules under init_empty_weights (gpt2.py:268-272)
    with torch.device("meta"):
        m = op.FlashAttention(64, 4, attn_op_name="hip_cdna4", fused_qkv=True)
        f = op.FusedMLP(64, 256, "gelu", 0.1)
    assert all(p.is_meta for p in list(m.parameters()) + list(f.parameters()))


def test_separate_bias_linear_and_fused_qkv_on_cpu():
    lin = op.LinearWithSeparateBias(6, 5)
    x = torch.randn(3, 6)
    torch.testing.assert_close(lin(x), nn.functional.linear(x, lin.weight, lin.bias))
    sync = op.LinearWithSyncFunc(6, 5, sync_fn=lambda t: t * 2)
    torch.testing.assert_close(sync(x), nn.functional.linear(x, sync.weight) * 2 + sync.bias)
    qkv = op.FusedQKV(8, 2, 1)
    q, k, v = qkv(torch.randn(2, 3, 8))
    assert q.shape == k.shape == v.shape == (2, 3, 2, 4)


class _FakeBackend:
    """Stands in for the device generator: state = (seed, offset)."""

    def __init__(self):
        self.state = (0, 0)

    def get_state(self):
        return self.state

    def set_state(self, s):
        self.state = s

    def manual_seed(self, seed):
        self.state = (seed, 0)

    def draw(self, n=4):
        s = self.state
        self.state = (s[0], s[1] + n)
        return s


def test_rng_tracker_state_machine():
    be = _FakeBackend()
    tr = CudaRNGStatesTracker(be)
    be.manual_seed(2013)
    be.draw()
    tr.add("model-parallel-rng", 2013 + 2718)
    assert be.state == (2013, 4)  # add() leaves the outer stream untouched
    with pytest.raises(Exception, match="seed 4731 already exists"):
        tr.add("other", 4731)
    with pytest.raises(Exception, match="already exists"):
        tr.add("model-parallel-rng", 1)
    with pytest.raises(RuntimeError, match="is not added"):
        with tr.fork("missing"):
            pass
    with tr.fork():
        assert be.draw() == (4731, 0)
    with tr.fork():
        assert be.draw() == (4731, 4)  # the named stream continues where it stopped
    assert be.state == (2013, 4)       # and the outer one never moved
    try:
        with tr.fork():
            be.draw()
            raise KeyError
    except KeyError:
        pass
    assert be.state == (2013, 4) and tr.get_states()["model-parallel-rng"] == (4731, 12)
    tr.reset()
    assert not tr.get_states()


def test_set_random_seed_arithmetic():
    assert slapo_amd.set_random_seed(2013) == 2013
    assert slapo_amd.set_random_seed(2013, dp_rank=3, pp_rank=2) == 2013 + 200 + 30
    a = torch.rand(3)
    slapo_amd.set_random_seed(2013, dp_rank=3, pp_rank=2)
    torch.testing.assert_close(torch.rand(3), a)


def test_checkpoint_replays_every_random_stream(monkeypatch):
    """The reference's test of its checkpoint with forked streams
    (tests/test_checkpoint.py:138-198), on the host: a block that draws from the outer stream,
    from the forked stream and from the host generator gives the same output and gradients with
    and without the checkpoint, and the recompute moves none of the streams."""
    import importlib
    ckpt = importlib.import_module("slapo_amd.checkpoint")  # the package attribute is the function

    be = _FakeBackend()
    tr = CudaRNGStatesTracker(be)
    monkeypatch.setattr(ckpt, "get_cuda_rng_tracker", lambda: tr)
    monkeypatch.setattr(ckpt, "is_random_seed_set", lambda: bool(tr.get_states()))

    def device_dropout(x):
        seed, off = be.draw()
        g = torch.Generator().manual_seed(seed * 1000 + off)
        return x * (torch.rand(x.shape, generator=g) < 0.5) * 2.0

    w1 = torch.randn(6, 5, requires_grad=True)
    w2 = torch.randn(5, 6, requires_grad=True)
    calls = []

    def block(x, tag):
        calls.append(tag)
        h = x @ w1
        with tr.fork():
            h = device_dropout(h)
        h = device_dropout(h @ w2)
        return nn.functional.dropout(h, 0.5)  # host generator

    def run(use_checkpoint):
        be.manual_seed(123)
        tr.reset()
        tr.add("model-parallel-rng", 123 + 2718)
        torch.manual_seed(5)
        x = torch.arange(36.0).reshape(6, 6).requires_grad_()
        out = ckpt.checkpoint(block, x, "t") if use_checkpoint else block(x, "t")
        before = (be.state, tr.get_states(), torch.get_rng_state())
        out.mean().backward()
        after = (be.state, tr.get_states(), torch.get_rng_state())
        assert before[0] == after[0] and before[1] == after[1] and torch.equal(before[2], after[2])
        grads = [t.grad.clone() for t in (x, w1, w2)]
        w1.grad = w2.grad = None
        return [out.detach()] + grads

    ref = run(False)
    n = len(calls)
    got = run(True)
    assert len(calls) == n + 2 and calls[-1] == "t"   # forward and one recompute
    for a, b in zip(ref, got):
        assert torch.equal(a, b)
    assert be.state == (123, 4) and tr.get_states()["model-parallel-rng"] == (123 + 2718, 4)

    # without tracked streams the call goes to torch's own checkpoint
    tr.reset()
    x = torch.randn(6, 6, requires_grad=True)
    out = ckpt.checkpoint(lambda t: (t @ w1).relu(), x, use_reentrant=False)
    out.sum().backward()
    assert x.grad is not None and w1.grad is not None


def test_flash_attention_is_fx_traceable_with_the_op_as_a_leaf():
    """The GPT-2 schedule traces the replaced attention module with FlashAttentionOp as a leaf and
    these concrete_args (model_schedule/gpt2.py:457-469); the graph must call the `out_proj` and
    `resid_dropout` children as modules, so that `.sync` hooks and `.shard` still find them."""
    from torch import fx

    class _Tracer(fx.Tracer):
        def is_leaf_module(self, m, qualname):
            return "FlashAttentionOp" in type(m).__name__ or super().is_leaf_module(m, qualname)

    m = op.FlashAttention(hidden_size=64, num_attention_heads=4, output_proj=True, attn_pdrop=0.1,
                          resid_pdrop=0.1, attn_op_name="hip_cdna4", fused_qkv=True)
    graph = _Tracer().trace(m, concrete_args={
        "layer_past": None, "head_mask": None, "encoder_hidden_states": None,
        "encoder_attention_mask": None, "use_cache": False, "output_attentions": False})
    targets = [n.target for n in graph.nodes if n.op == "call_module"]
    assert targets == ["qkv", "attn_op", "out_proj", "resid_dropout"]


def test_fused_tail_is_taken_only_for_plain_hook_free_children():
    """`_tail_can_fuse` decides between one fused pass and the two child calls of the reference
    (slapo/op/attention.py:514-516).  Evaluated on the host with a stand-in for a device tensor's
    `is_cuda`: the decision reads only types and hook tables."""
    m = op.FlashAttention(64, 4, resid_pdrop=0.1, fused_qkv=True)
    x = torch.zeros(1, 2, 64)
    assert m._tail_can_fuse(x) is False  # CPU tensor: the children raise the device error
    from slapo_amd.op.attention import _has_hooks
    assert not _has_hooks(m.out_proj) and not _has_hooks(m.resid_dropout)
    h = m.out_proj.register_forward_hook(lambda mod, inp, out: out)
    assert _has_hooks(m.out_proj)
    h.remove()
    assert not _has_hooks(m.out_proj)
    h = m.resid_dropout.register_forward_pre_hook(lambda mod, inp: None)
    assert _has_hooks(m.resid_dropout)
    h.remove()
    h = m.out_proj.register_full_backward_hook(lambda mod, gi, go: None)
    assert _has_hooks(m.out_proj)
    h.remove()
