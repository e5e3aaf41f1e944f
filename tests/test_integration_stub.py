"""The reference-side binding shown in the integration guide at the repository root (the code a
maintainer would paste into slapo/op/attention.py) is executed here exactly as documented.

CPU: its ctypes structs are compared, field by field, with what the C compiler makes of
include/slapo_amd.h (offsets and sizes printed by a small program built with gcc), and so is the
package's own binding.  GPU: its forward, backward and dropout traffic are compared with the
package's `hip_attention` on the same inputs and generator state (bitwise: both call the same
entry points)."""
import ctypes
import os
import re
import subprocess
import sys

import pytest
import torch

from slapo_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
DOC = os.path.join(ROOT, "INTEGRATION.md")
HEADER_DIR = os.path.join(ROOT, "include")


def _stub_source():
    text = open(DOC).read()
    m = re.search(r"<!-- stub:begin -->\s*```python\n(.*?)```\s*<!-- stub:end -->", text, re.S)
    assert m, "the integration guide lost its stub markers"
    return m.group(1)


@pytest.fixture(scope="module")
def stub():
    os.environ["SLAPO_AMD_LIB"] = _lib.LIB_PATH
    ns = {"__name__": "integration_stub"}
    exec(compile(_stub_source(), DOC, "exec"), ns)  # pylint: disable=exec-used
    return ns


def _c_layout(tmp_path_factory, struct, fields):
    """{field: (offset, size)} and the struct's size as gcc lays it out from the header."""
    d = tmp_path_factory.mktemp("layout")
    lines = [f'printf("%s %zu %zu\\n", "{f}", offsetof({struct}, {f}), sizeof((({struct}*)0)->{f}));'
             for f in fields]
    src = d / "layout.c"
    src.write_text('#include <stdio.h>\n#include <stddef.h>\n#include "slapo_amd.h"\n'
                   "int main(void) {\n" + "\n".join(lines)
                   + f'\nprintf("sizeof %zu 0\\n", sizeof({struct}));\nreturn 0;\n}}\n')
    exe = d / "layout"
    subprocess.run(["gcc", "-std=c11", "-I", HEADER_DIR, str(src), "-o", str(exe)], check=True)
    out = subprocess.run([str(exe)], check=True, capture_output=True, text=True).stdout
    table = {}
    for line in out.splitlines():
        name, off, size = line.split()
        table[name] = (int(off), int(size))
    return table


def _ctypes_layout(cls):
    table = {name: (getattr(cls, name).offset, getattr(cls, name).size) for name, *_ in cls._fields_}
    table["sizeof"] = (ctypes.sizeof(cls), 0)
    return table


@pytest.mark.parametrize("which", ["documented stub", "package binding"])
def test_struct_layouts_match_the_header(stub, tmp_path_factory, which):
    plan_cls, prm_cls = ((stub["_Plan"], stub["_Params"]) if which == "documented stub"
                         else (_lib.DropoutPlan, _lib.AttnParams))
    header = re.sub(r"/\*.*?\*/", "", open(os.path.join(HEADER_DIR, "slapo_amd.h")).read(),
                    flags=re.S)
    for cls, struct in ((plan_cls, "slapo_dropout_plan"), (prm_cls, "slapo_attn_params")):
        body = re.search(r"typedef struct[^{}]*\{([^{}]*)\}\s*" + struct + r"\s*;", header).group(1)
        declared = re.findall(r"(\w+)\s*(?:\[\d+\])?\s*;", body)
        names = [name for name, *_ in cls._fields_]
        assert names == declared, f"{which}: fields of {struct} differ from the header"
        assert _ctypes_layout(cls) == _c_layout(tmp_path_factory, struct, declared)


def test_stub_prototypes_agree_with_the_package_table(stub):
    lib = stub["_hip"]
    for name in ("slapo_amd_attn_fwd", "slapo_amd_attn_bwd", "slapo_amd_attn_bwd_workspace_bytes",
                 "slapo_amd_dropout_plan"):
        restype, argtypes = _lib.PROTOTYPES[name]
        mine = getattr(lib, name).argtypes
        assert len(mine) == len(argtypes), name
        for a, b in zip(mine, argtypes):
            # pointer-to-struct types differ by class identity; compare their kind and size
            assert ctypes.sizeof(a) == ctypes.sizeof(b), name
            assert issubclass(a, ctypes._Pointer) == issubclass(b, ctypes._Pointer) or \
                ctypes.c_void_p in (a, b), name  # pylint: disable=protected-access


class _Op(torch.nn.Module):
    """FlashAttentionOp reduced to the two edits that the guide asks for: the registry branch sets
    pkg / attn_fn, the forward takes the new first branch."""

    def __init__(self, attn_fn, apply_causal_mask, scale=None):
        super().__init__()
        self.pkg, self.attn_fn = "hip", attn_fn
        self.apply_causal_mask, self.scale = apply_causal_mask, scale
        self.bias_layout = "b11k" if self.pkg in ("flash_attn", "hip") else "bhqk"

    def forward(self, query_layer, key_layer, value_layer, attention_mask, p):
        assert self.pkg == "hip"
        return self.attn_fn(query_layer, key_layer, value_layer, attention_mask,
                            self.apply_causal_mask, p, self.scale)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype,p,causal,masked", [
    (torch.float16, 0.0, True, False), (torch.bfloat16, 0.0, True, True),
    (torch.bfloat16, 0.1, True, True), (torch.float32, 0.0, False, True),
    (torch.float16, 0.1, False, False)])
def test_documented_binding_runs_and_equals_the_package(stub, dtype, p, causal, masked):
    from slapo_amd.op.attention import hip_attention
    import slapo_amd.op.attention as A
    b, s, h, d = 2, 192, 4, 64
    torch.manual_seed(1)
    packed = torch.randn(b, s, h, 3 * d, device="cuda", dtype=dtype)
    dout = torch.randn(b, s, h, d, device="cuda", dtype=dtype)
    mask = None
    if masked:  # HF padding mask [B,1,1,S] in the model's dtype
        mask = torch.zeros(b, 1, 1, s, device="cuda", dtype=dtype)
        mask[1, :, :, 150:] = torch.finfo(dtype).min
    results = []
    for fn in ("stub", "package"):
        leaves = [t.detach().clone().requires_grad_(True) for t in packed.split(d, dim=-1)]
        # strided views of one buffer, as the fused QKV projection hands them over
        buf = torch.cat(leaves, dim=-1)
        q, k, v = buf.split(d, dim=-1)
        torch.cuda.manual_seed(11)
        if fn == "stub":
            out = _Op(stub["_hip_attention"], causal)(q, k, v, mask, p)
        else:
            A.SAVE_DROPOUT_MASK, keep = False, A.SAVE_DROPOUT_MASK
            try:
                out = hip_attention(q, k, v, mask, causal=causal, p=p)
            finally:
                A.SAVE_DROPOUT_MASK = keep
        offset = torch.cuda.default_generators[0].get_offset()
        out.backward(dout)
        results.append((out.detach(), [t.grad for t in leaves], offset))
    (o1, g1, off1), (o2, g2, off2) = results
    assert off1 == off2  # same generator traffic
    assert torch.equal(o1, o2)
    for a, b_ in zip(g1, g2):
        assert torch.equal(a, b_)
    assert torch.isfinite(o1.float()).all()
