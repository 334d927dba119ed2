"""Host-side logic of the drop-in MoE block that needs no GPU: tensors made under torch.inference_mode() have no
version counter (reading `_version` raises), so nothing derived from them may be cached against one; an expert list
other than wall-x's own (two silu experts) selects the generic path instead of raising."""

from types import SimpleNamespace

import pytest
import torch

from wallx_mi355 import moe


def _cfg(inters=(96, 32), acts=("silu", "silu"), hidden=64):
    return SimpleNamespace(experts=[dict(hidden_size=hidden, intermediate_size=i, hidden_act=a)
                                    for i, a in zip(inters, acts)])


def test_version_of_inference_tensors_is_none():
    normal = torch.zeros(3)
    assert moe._version_of(normal) == normal._version
    with torch.inference_mode():
        made_inside = torch.zeros(3)
        assert moe._version_of(made_inside) is None
        with pytest.raises(RuntimeError):
            made_inside._version  # what the guard exists for
        assert moe._version_of(normal) == normal._version  # a normal tensor keeps its counter in inference mode


def test_host_row_counts_from_inference_mode_tensors_are_read_on_every_call():
    block = moe.SparseMoeBlock(_cfg(), 2)
    with torch.inference_mode():
        start, end = torch.tensor([0, 5]), torch.tensor([5, 12])
        rows = block._host_rows(start, end, 12)
        assert list(rows) == [5, 7] and block._rows_seen is None  # nothing to check a later call against
        end[1] = 11  # an in-place write no counter records
        assert block._host_rows(start, end, 11) is not None and list(block._host_rows(start, end, 11)) == [5, 6]
    start, end = torch.tensor([0, 5]), torch.tensor([5, 12])
    first = block._host_rows(start, end, 12)
    assert block._host_rows(start, end, 12) is first  # tracked tensors: answered from the cache
    end[1] = 11
    assert list(block._host_rows(start, end, 11)) == [5, 6]  # the version counter moved
    assert block._host_rows(start, end, 12) is None  # counts that do not add up to the token count are not used


def test_expert_lists_other_than_two_silu_experts_select_the_generic_path():
    assert moe.SparseMoeBlock(_cfg(), 2)._fused
    three = moe.SparseMoeBlock(_cfg((96, 32, 48), ("silu",) * 3), 3)
    assert not three._fused and len(three.experts) == 3
    gelu = moe.SparseMoeBlock(_cfg(acts=("gelu", "silu")), 2)
    assert not gelu._fused
    x = torch.linspace(-3, 3, 13)
    assert torch.allclose(gelu.experts[0].act_fn(x), torch.nn.functional.gelu(x))
    assert torch.allclose(gelu.experts[1].act_fn(x), torch.nn.functional.silu(x))
    with pytest.raises(KeyError):
        moe.SparseMoeBlock(_cfg(acts=("no_such_activation", "silu")), 2)
    with pytest.raises(RuntimeError, match="generic ops"):
        gelu.pack_for_inference()
    # the reference's parameter names (act.py:74-76, 101-103), whatever the path
    assert sorted(three.state_dict()) == sorted(f"experts.{e}.{p}_proj.weight" for e in range(3)
                                                for p in ("gate", "up", "down"))
