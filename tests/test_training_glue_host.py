"""Host-side contract of the caller glue (no GPU): hidden-state discovery in model outputs, the
model-input id check and the ZeRO-3 parameter-gather context, on the cases the reference's own tests
assert (tests/test_deepspeed_training_worker.py:296-373 of the reference) plus the remaining
branches of the rule set."""
from contextlib import nullcontext
from types import SimpleNamespace

import pytest
import torch

from rl_kernel_amd import training as T


def test_final_hidden_state_wins_over_the_per_layer_stack():
    want = torch.randn(2, 3, 5)
    out = {"hidden_states": (torch.randn(2, 3, 5), torch.randn(2, 3, 5)), "last_hidden_state": want}
    assert T.extract_hidden_states(out) is want


def test_last_entry_of_the_per_layer_stack():
    layers = (torch.randn(2, 3, 5), torch.randn(2, 3, 5), torch.randn(2, 3, 5))
    assert T.extract_hidden_states({"hidden_states": layers}) is layers[-1]
    assert T.extract_hidden_states(SimpleNamespace(hidden_states=list(layers))) is layers[-1]


def test_structured_member_of_a_tuple_wins_over_bare_logits():
    want = torch.randn(2, 3, 5)
    out = (torch.tensor(1.0), torch.randn(2, 3, 11), {"last_hidden_state": want})
    assert T.extract_hidden_states(out) is want


def test_two_candidate_tensors_in_a_tuple_are_ambiguous():
    with pytest.raises(TypeError, match="hidden-state tensor"):
        T.extract_hidden_states((torch.randn(2, 3, 11), torch.randn(2, 3, 5)))


def test_expected_hidden_dim_disambiguates_and_rank_breaks_ties():
    logits, hidden = torch.randn(1, 3, 13), torch.randn(1, 3, 5)
    assert T.extract_hidden_states((torch.tensor(1.0), logits, hidden), expected_hidden_dim=5) is hidden
    pooled, seq = torch.randn(4, 5), torch.randn(4, 7, 5)
    assert T.extract_hidden_states((pooled, seq)) is seq        # the unique tensor of highest rank
    assert T.extract_hidden_states(hidden) is hidden
    assert T.extract_hidden_states(SimpleNamespace(hidden=hidden, logits=logits)) is hidden
    assert T.extract_hidden_states([{"other": 1}, [hidden]]) is hidden   # nested plain sequence
    for bad in (torch.tensor(1.0), {"logits": logits}, None, (torch.tensor(1.0),)):
        with pytest.raises(TypeError, match="hidden-state tensor"):
            T.extract_hidden_states(bad)
    with pytest.raises(TypeError, match="hidden-state tensor"):
        T.extract_hidden_states(hidden, expected_hidden_dim=6)


def test_model_input_ids_must_be_vocabulary_entries():
    T.validate_model_input_token_ids(torch.tensor([[0, 5, 22]]), vocab_size=23)
    with pytest.raises(ValueError, match=r"must be in \[0, 22\], got \[-100, 7\]"):
        T.validate_model_input_token_ids(torch.tensor([[7, -100]]), vocab_size=23)
    with pytest.raises(ValueError, match=r"got \[1, 23\]"):
        T.validate_model_input_token_ids(torch.tensor([1, 23]), vocab_size=23)


class _Model(torch.nn.Module):
    def __init__(self, bias):
        super().__init__()
        self.lm_head = torch.nn.Linear(4, 9, bias=bias)


def test_parameter_gather_context_follows_the_zero_stage_contract():
    calls = []

    def gathered(params, modifier_rank="unset"):
        calls.append((list(params), modifier_rank))
        return nullcontext("gathered")

    runtime = SimpleNamespace(zero=SimpleNamespace(GatheredParameters=gathered))
    model = _Model(bias=True)
    # nothing is partitioned below stage 3 or on a single rank
    assert isinstance(T.linear_logp_parameter_context(runtime, model, zero_stage=2, world_size=8), nullcontext)
    assert isinstance(T.linear_logp_parameter_context(None, model, zero_stage=3, world_size=1), nullcontext)
    assert calls == []
    with T.linear_logp_parameter_context(runtime, model, zero_stage=3, world_size=2) as tag:
        assert tag == "gathered"
    assert len(calls) == 1 and calls[0][1] is None
    assert calls[0][0][0] is model.lm_head.weight and calls[0][0][1] is model.lm_head.bias
    T.linear_logp_parameter_context(runtime, _Model(bias=False), zero_stage=3, world_size=2)
    assert len(calls[1][0]) == 1
    with pytest.raises(TypeError, match="lm_head"):
        T.linear_logp_parameter_context(runtime, torch.nn.Linear(2, 2), zero_stage=3, world_size=2)
    with pytest.raises(T.ParameterGatherUnavailableError, match="GatheredParameters"):
        T.linear_logp_parameter_context(SimpleNamespace(), model, zero_stage=3, world_size=2)


def test_extract_logps_takes_a_model_and_its_output_like_the_reference():
    """Same call shape as the reference's _extract_logps (model output, model, ids, mask, op): here
    with a stand-in op on the CPU that records what it was given."""
    seen = {}

    class Op:
        def __call__(self, hidden, weight, ids, bias):
            seen.update(hidden=hidden, weight=weight, ids=ids, bias=bias)
            return torch.full(ids.shape, -1.5)

    model = _Model(bias=True)
    hidden = torch.randn(2, 3, 4)
    ids = torch.tensor([[1, 2, 3], [4, 5, 6]])
    mask = torch.tensor([[True, False, True], [True, True, False]])
    out = T.extract_logps((torch.tensor(0.0), torch.randn(2, 3, 9), hidden), model, ids, mask, Op())
    assert seen["hidden"] is hidden and seen["weight"] is model.lm_head.weight
    assert torch.equal(seen["ids"], ids.masked_fill(~mask, 0))
    assert torch.equal(out, torch.full((2, 3), -1.5).masked_fill(~mask, 0.0))
    with pytest.raises(TypeError, match="lm_head"):
        T.extract_logps(hidden, torch.nn.ReLU(), ids, mask, Op())
