"""The attention wrappers of the reference's model schedules (restated in tests/adapters.py)
around this package's FlashAttention: constructor arguments, the "cutlass" fall-back, attribute
reads (CPU only; tests/test_gpu_schedule_dropin.py runs them on the device)."""
import pytest

from slapo_amd import op
from tests import adapters as A

FAMILIES = ["gpt2", "gpt_neo", "opt", "bert", "albert"]


@pytest.mark.parametrize("family", FAMILIES)
@pytest.mark.parametrize("name", ["cuda", "triton", "cutlass", "hip_cdna4"])
def test_schedule_kwargs_build_the_module(family, name):
    cfg = A.model_config(attn_pdrop=0.1, attention_dropout=0.1, attention_probs_dropout_prob=0.1,
                         resid_pdrop=0.2, resid_dropout=0.2, dropout=0.2,
                         hidden_dropout_prob=0.2)
    m = A.inner(A.make_adapter(family, op.FlashAttention, cfg, name))
    # what the schedules read back (e.g. gpt2.py:272) and address afterwards (gpt2.py:452-489)
    assert m.attn_op_name == name and m.attn_op.pkg == "hip" and m.bias_layout == "b11k"
    assert m.fused_qkv and hasattr(m, "qkv") and m.attn_pdrop == 0.1
    assert m.attn_op.apply_causal_mask is (family != "bert")
    if family == "bert":
        assert not hasattr(m, "out_proj")
    else:
        assert m.resid_dropout.p == 0.2
        assert (m.out_proj.bias is None) == (family == "gpt_neo")
    assert (m.qkv.bias is None) == (family == "gpt_neo")


@pytest.mark.parametrize("family", FAMILIES)
def test_constructor_failure_falls_back_to_cutlass_and_lands_on_the_hip_op(family):
    """The schedules catch ANY constructor error and retry with "cutlass" (gpt2.py:229-239); a
    name this package rejects must therefore end on the HIP op, and "native_xformers" must surface
    as the RuntimeError the wrappers raise for it."""
    m = A.inner(A.make_adapter(family, op.FlashAttention, A.model_config(), "not_installed_op"))
    assert m.attn_op_name == "cutlass" and m.attn_op.pkg == "hip"
    with pytest.raises(RuntimeError, match="Failed to create native attention"):
        A.make_adapter(family, op.FlashAttention, A.model_config(), "native_xformers")
