"""The generate() adapter against model and cache interfaces of different transformers
releases (reference cudagraph_utils.py:52-80), driven with mock objects on the CPU: the
recorded step is replaced by a recorder that simply calls the function."""
import types

import pytest
import torch

from bf16_huffman_infer_amd.cudagraph_utils import _max_cache_len, apply_graphed


class _Eager:
    """Recorder stand-in: no graph, the step function is called on every use."""
    def __init__(self, fn, sample_args):
        self.fn = fn
        fn(*sample_args)                     # what a capture would do: run once on the sample

    def __call__(self, *args):
        return self.fn(*args)


class _Cache:
    def __init__(self, style, n=16):
        self.seen = 0
        self.resets = 0
        if style == "get_max_length":
            self.get_max_length = lambda: n
        elif style == "get_max_cache_shape":
            self.get_max_cache_shape = lambda: n
        else:
            self.max_cache_len = n

    def reset(self):
        self.seen = 0
        self.resets += 1

    def get_seq_length(self):
        return self.seen


def _model(with_cache_position: bool, log: list):
    """A model whose logits are the input ids as floats; records what forward received."""
    m = types.SimpleNamespace(device=torch.device("cpu"), dtype=torch.float32)

    def record(input_ids, attention_mask, position_ids, past_key_values, cache_position, use_cache):
        log.append(dict(ids=input_ids.clone(), mask=attention_mask, pos=position_ids, cache=past_key_values,
                        cache_position=cache_position, use_cache=use_cache))
        past_key_values.seen += input_ids.shape[1]
        return types.SimpleNamespace(logits=input_ids.float()[..., None])

    if with_cache_position:
        def forward(input_ids=None, attention_mask=None, position_ids=None, past_key_values=None, use_cache=None,
                    cache_position=None, return_dict=None, output_attentions=None, output_hidden_states=None):
            return record(input_ids, attention_mask, position_ids, past_key_values, cache_position, use_cache)
    else:
        def forward(input_ids=None, attention_mask=None, position_ids=None, past_key_values=None, use_cache=None,
                    return_dict=None):
            return record(input_ids, attention_mask, position_ids, past_key_values, None, use_cache)
    m.forward = forward

    def generate(input_ids, past_key_values=None, max_new_tokens=2, **kwargs):
        log.append(dict(generate_kwargs=sorted(kwargs), cache=past_key_values))
        out = m.forward(input_ids=input_ids)                       # prefill, no cache_position given
        tok = input_ids[:, -1:]
        for _ in range(max_new_tokens):
            out = m.forward(input_ids=tok, cache_position=None)
        return out.logits
    m.generate = generate
    return m


@pytest.mark.parametrize("style", ["get_max_length", "get_max_cache_shape", "max_cache_len"])
def test_cache_length_is_found_under_every_name(style):
    assert _max_cache_len(_Cache(style, n=24)) == 24


@pytest.mark.parametrize("with_cache_position", [True, False])
@pytest.mark.parametrize("style", ["get_max_length", "get_max_cache_shape", "max_cache_len"])
def test_patched_forward_with_both_model_signatures(with_cache_position, style):
    log = []
    cache = _Cache(style)
    model = _model(with_cache_position, log)
    apply_graphed(model, cache, recorder=_Eager)
    assert cache.resets == 1 and cache.seen == 0       # the sample run of the recorder is wiped
    log.clear()

    # prefill: several tokens, eager, positions derived from the cache when none are given
    out = model.forward(input_ids=torch.tensor([[5, 6, 7]]), past_key_values="ignored", use_cache=False, foo=1)
    assert out.logits.shape == (1, 3, 1) and out.past_key_values is cache
    assert log[-1]["cache"] is cache and log[-1]["use_cache"] is True
    if with_cache_position:
        assert log[-1]["cache_position"].tolist() == [0, 1, 2]

    # one token: goes through the recorded step with a full-length additive mask
    out = model.forward(input_ids=torch.tensor([[9]]))
    assert out.logits.flatten().tolist() == [9.0]
    step = log[-1]
    assert step["mask"].shape == (1, 1, 1, 16) and step["pos"].tolist() == [[3]]
    assert (step["mask"][0, 0, 0, :4] == 0).all() and torch.isinf(step["mask"][0, 0, 0, 4:]).all()
    if with_cache_position:
        assert step["cache_position"].tolist() == [3]

    # generate(): cache reset and passed on; keywords the release does not know are not invented
    log.clear()
    model.generate(torch.tensor([[1, 2]]), max_new_tokens=2)
    assert cache.resets == 2 and log[0]["cache"] is cache
    assert log[0]["generate_kwargs"] in ([], ["disable_compile"])
    assert [e["ids"].shape[1] for e in log[1:]] == [2, 1, 1]
