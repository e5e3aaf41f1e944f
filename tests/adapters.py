"""Stand-ins for the attention wrappers that the reference's model schedules build around
`FlashAttention` (test infrastructure; nothing here is product code).  Each class restates one
schedule's constructor arguments, its try / except fall-back to "cutlass" and the way it maps the
original HF forward signature onto `FlashAttention.forward` and trims the result:

    GPT-2     slapo/model_schedule/gpt2.py:212-264      -> outputs[:1]
    GPT-Neo   slapo/model_schedule/gpt_neo.py:163-215   -> outputs[:1], bias=False
    OPT       slapo/model_schedule/opt.py:158-201       -> (out, None, None)
    BERT      slapo/model_schedule/bert.py:165-208      -> outputs[:1], output_proj=False
    ALBERT    slapo/model_schedule/albert.py:168-205    -> (context, None), child `self_attn`

They take the `FlashAttention` class as an argument so that the same wrappers can be pointed at
this package's module.
"""
from types import SimpleNamespace

from torch import nn


def _build(flash_cls, kwargs):
    """The constructor pattern shared by all five schedules (e.g. gpt2.py:226-239)."""
    try:
        return flash_cls(**kwargs)
    except Exception as err:  # pylint: disable=broad-except
        if kwargs["attn_op_name"] == "native_xformers":
            raise RuntimeError(f"Failed to create native attention: {err}") from None
        kwargs["attn_op_name"] = "cutlass"
        return flash_cls(**kwargs)


def model_config(**over):
    cfg = dict(hidden_size=256, num_attention_heads=4, attn_pdrop=0.0, resid_pdrop=0.0,
               attention_dropout=0.0, resid_dropout=0.0, dropout=0.0,
               attention_probs_dropout_prob=0.0, hidden_dropout_prob=0.0)
    cfg.update(over)
    return SimpleNamespace(**cfg)


def init_config(family, cfg, attn_op_name):
    common = dict(hidden_size=cfg.hidden_size, num_attention_heads=cfg.num_attention_heads,
                  attn_op_name=attn_op_name, fused_qkv=True)
    if family == "gpt2":
        return dict(common, output_proj=True, attn_pdrop=cfg.attn_pdrop,
                    resid_pdrop=cfg.resid_pdrop)
    if family == "gpt_neo":
        return dict(common, output_proj=True, attn_pdrop=cfg.attention_dropout,
                    resid_pdrop=cfg.resid_dropout, bias=False)
    if family == "opt":
        return dict(common, output_proj=True, attn_pdrop=cfg.attention_dropout,
                    resid_pdrop=cfg.dropout, bias=True)
    if family == "bert":
        return dict(common, output_proj=False, attn_pdrop=cfg.attention_probs_dropout_prob,
                    resid_pdrop=cfg.hidden_dropout_prob, bias=True)
    if family == "albert":
        return dict(common, output_proj=True, attn_pdrop=cfg.attention_probs_dropout_prob,
                    resid_pdrop=cfg.hidden_dropout_prob, bias=True)
    raise KeyError(family)


def make_adapter(family, flash_cls, cfg, attn_op_name="cuda"):
    kwargs = init_config(family, cfg, attn_op_name)

    class GPT2Attention(nn.Module):
        def __init__(self):
            super().__init__()
            self.module = _build(flash_cls, kwargs)

        def forward(self, hidden_states, layer_past=None, attention_mask=None, head_mask=None,
                    encoder_hidden_states=None, encoder_attention_mask=None, use_cache=False,
                    output_attentions=False):
            outputs = self.module(hidden_states, attention_mask, layer_past, head_mask,
                                  encoder_hidden_states, encoder_attention_mask, use_cache,
                                  output_attentions)
            return outputs[:1]

    class GPTNeoAttention(nn.Module):
        def __init__(self):
            super().__init__()
            self.module = _build(flash_cls, kwargs)

        def forward(self, hidden_states, layer_past=None, attention_mask=None, head_mask=None,
                    use_cache=False, output_attentions=False):
            outputs = self.module(hidden_states, attention_mask, layer_past, head_mask, None,
                                  None, use_cache, output_attentions)
            return outputs[:1]

    class OPTAttention(nn.Module):
        def __init__(self):
            super().__init__()
            self.module = _build(flash_cls, kwargs)

        def forward(self, hidden_states, past_key_value=None, attention_mask=None,
                    layer_head_mask=None, output_attentions=False, use_cache=False):
            outputs = self.module(hidden_states, attention_mask, past_key_value)
            return outputs[0], None, None

    class BertSelfAttention(nn.Module):
        def __init__(self):
            super().__init__()
            self.module = _build(flash_cls, kwargs)

        def forward(self, hidden_states, attention_mask=None, head_mask=None,
                    encoder_hidden_states=None, encoder_attention_mask=None,
                    past_key_value=None, output_attentions=False):
            outputs = self.module(hidden_states, attention_mask, past_key_value)
            return outputs[:1]

    class AlbertXFAttention(nn.Module):
        def __init__(self):
            super().__init__()
            self.self_attn = _build(flash_cls, kwargs)

        def forward(self, hidden_states, attention_mask=None, head_mask=None,
                    output_attentions=False):
            outputs = self.self_attn(hidden_states, attention_mask)
            return (outputs[0], None)

    return {"gpt2": GPT2Attention, "gpt_neo": GPTNeoAttention, "opt": OPTAttention,
            "bert": BertSelfAttention, "albert": AlbertXFAttention}[family]()


def inner(adapter):
    """The FlashAttention inside an adapter (ALBERT names the child `self_attn`)."""
    return adapter.self_attn if hasattr(adapter, "self_attn") else adapter.module
