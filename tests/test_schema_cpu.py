"""The operator surface: every schema this build registers equals the
reference's (tests/golden/op_schemas.txt), argument by argument.

Allowed differences, each a widening the reference itself relies on (it passes
Python ``None`` for these plain ``Tensor`` arguments and tests ``.defined()``,
fused_moe.py:256-266, modular_experts.py:246): ``Tensor`` -> ``Tensor?`` for
``azp``, ``e_score_correction_bias``, ``expert_map``, ``real_token_num``,
``B_scale`` (absent for unquantised experts) and ``B_zero`` (fused_moe.py:182
passes None).  ``(a!)`` and ``!`` both mean
"written in place" and compare equal.
"""
import os

import pytest
import torch

from vllm_gcu_amd.kernels import _custom_ops  # noqa: F401  (registers the ops)

GOLDEN = os.path.join(os.path.dirname(__file__), "golden", "op_schemas.txt")
WIDENED = {"azp", "e_score_correction_bias", "expert_map", "real_token_num", "B_scale", "B_zero"}


def golden_rows():
    rows = []
    with open(GOLDEN) as f:
        for line in f:
            line = line.strip()
            if not line or line.startswith("#"):
                continue
            ns, lineno, schema = line.split(" ", 2)
            rows.append((ns, int(lineno), schema))
    return rows


def describe(schema):
    args = []
    for a in schema.arguments:
        written = a.alias_info is not None and a.alias_info.is_write
        args.append((a.name, str(a.type), written))
    rets = [str(r.type) for r in schema.returns]
    return args, rets


@pytest.mark.parametrize("ns,lineno,text", golden_rows(), ids=lambda v: v if isinstance(v, str) and "(" not in v else None)
def test_schema_matches_reference(ns, lineno, text):
    want = torch._C.parse_schema(f"{ns}::{text}")
    op = getattr(getattr(torch.ops, ns), want.name.split("::")[-1])
    got = op.default._schema
    wargs, wrets = describe(want)
    gargs, grets = describe(got)
    assert grets == wrets
    assert len(gargs) == len(wargs), (gargs, wargs)
    for (gn, gt, gw), (wn, wt, ww) in zip(gargs, wargs):
        assert gn == wn
        assert gw == ww, f"{gn}: mutability differs"
        if gt != wt:
            assert wn in WIDENED and gt == f"Optional[{wt}]", f"{gn}: {gt} vs {wt}"


def test_cutlass_scaled_mm_is_flexible_layout():
    # csrc/torch_bindings.cpp:1013-1017 tags the op so that w.t() views reach it unchanged
    assert torch.Tag.flexible_layout in torch.ops._C.cutlass_scaled_mm.default.tags


def test_golden_list_covers_every_registered_op():
    have = {(ns, torch._C.parse_schema(f"{ns}::{t}").name.split("::")[-1]) for ns, _, t in golden_rows()}
    registered = {tuple(q.split("::")) for q in _custom_ops.SCHEMAS}
    assert registered == have


def test_moe_wna16_config_parsing_and_compatibility():
    """MoeWNA16GCUConfig.from_config / is_moe_wna16_gcu_compatible / override_quantization_method
    (vllm_gcu/kernels/quantization/moe_wna16.py:67-158): host logic, no GPU work."""
    import pytest
    try:
        from vllm_gcu_amd.kernels.quantization.moe_wna16 import MoeWNA16GCUConfig
    except Exception as e:                                     # library not built in this environment
        pytest.skip(f"package not importable here: {e}")
    c = MoeWNA16GCUConfig.from_config({"quant_method": "gptq", "bits": 4, "group_size": 128, "sym": True})
    assert c.has_zp and c.weight_bits == 4 and int(c.pack_factor) == 8 and c.get_name() == "moe_wna16_gcu"
    c = MoeWNA16GCUConfig.from_config({"quant_method": "gptq", "bits": 8, "group_size": -1, "sym": True})
    assert not c.has_zp and int(c.pack_factor) == 4
    c = MoeWNA16GCUConfig.from_config({"quant_method": "awq", "bits": 4, "group_size": 64, "zero_point": True,
                                       "modules_to_not_convert": ["gate"]})
    assert c.has_zp and c.modules_to_not_convert == ["gate"]
    with pytest.raises(ValueError):
        MoeWNA16GCUConfig.from_config({"quant_method": "fp8", "bits": 8, "group_size": 128})
    ok = MoeWNA16GCUConfig.is_moe_wna16_gcu_compatible
    assert ok({"quant_method": "gptq", "bits": 4, "desc_act": False})
    assert ok({"quant_method": "gptq", "bits": 8, "desc_act": True, "static_groups": True})
    assert not ok({"quant_method": "gptq", "bits": 4, "desc_act": True})
    assert not ok({"quant_method": "gptq", "bits": 3})
    assert ok({"quant_method": "awq", "bits": 4}) and not ok({"quant_method": "awq", "bits": 8})
    over = MoeWNA16GCUConfig.override_quantization_method
    assert over({"quant_method": "gptq", "bits": 4}, "moe_wna16_gcu") == "moe_wna16_gcu"
    assert over({"quant_method": "gptq", "bits": 4}, None) is None
