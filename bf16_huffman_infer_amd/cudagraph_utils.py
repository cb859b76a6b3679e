"""HIP-graph capture of the one-token decode step.

Counterpart of the reference's ``bf16_huffman_infer/cudagraph_utils.py``
(``apply_graphed`` ``:11-80``, ``get_graphed_model`` ``:83-86``): the single-token forward of
a causal LM with a static KV cache is recorded once and replayed per token, prefill runs
eagerly, and ``generate`` is patched to reuse the one cache.  The reference goes through
``torch.cuda.make_graphed_callables``; here the step is recorded straight into a
``torch.cuda.CUDAGraph`` (a hipGraph on ROCm) over static input buffers, because the step
runs under ``no_grad`` and needs none of the autograd plumbing -- and because the fused
kernels are launched through the C ABI on the capturing stream, which is all a capture
needs from them.

:class:`GraphedCallable` is the model-independent part: any function of tensors whose
launches stay on the current stream can be recorded with it.
"""
import inspect
from typing import Callable, Sequence

import torch
from torch import nn

from .utils import shallow_copy_model

__all__ = ["GraphedCallable", "apply_graphed", "get_graphed_model"]


class GraphedCallable:
    """``fn(*tensors) -> tensor(s)`` recorded into one graph.

    ``sample_args`` fix shapes, dtypes and devices; they become the static input buffers.
    Calling the object copies the arguments into those buffers, replays the graph and
    returns the static output tensor(s) -- the same storage on every call, so a caller
    that keeps results across calls must clone them.

    No memset is recorded by this class itself; ``fn`` must not clear memory through paths
    that record memset nodes -- ``torch.zeros(...)`` inside a capture is one (build the
    tensor with an elementwise kernel, or clear a preallocated one with ``tensor.zero_()``).
    """

    def __init__(self, fn: Callable, sample_args: Sequence[torch.Tensor], warmup: int = 3):
        # The graph reads every tensor ``fn`` closes over by ADDRESS.  Holding ``fn`` keeps
        # those tensors alive for as long as the graph can be replayed; without it they are
        # freed when the caller's scope ends and the allocator hands their memory to
        # somebody else while replays still read it.
        self.fn = fn
        self.static_inputs = [a.clone() for a in sample_args]
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side), torch.no_grad():
            for _ in range(warmup):
                fn(*self.static_inputs)
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        self.graph = torch.cuda.CUDAGraph()
        with torch.no_grad(), torch.cuda.graph(self.graph):
            self.static_outputs = fn(*self.static_inputs)

    def __call__(self, *args: torch.Tensor):
        assert len(args) == len(self.static_inputs)
        for dst, src in zip(self.static_inputs, args):
            if src is not dst:
                dst.copy_(src)
        self.graph.replay()
        return self.static_outputs

    def replay(self):
        """Replay on the current contents of the static inputs."""
        self.graph.replay()
        return self.static_outputs


def _max_cache_len(cache) -> int:
    for name in ("get_max_length", "get_max_cache_shape"):
        fn = getattr(cache, name, None)
        if fn is not None:
            return int(fn())
    return int(cache.max_cache_len)


def _accepted(fn: Callable, kwargs: dict) -> dict:
    """``kwargs`` without the names ``fn`` does not take (everything when it has ``**kwargs``).

    ``forward`` and ``generate`` of transformers models gained and lost keywords over the
    releases (``cache_position``, ``disable_compile``, ``output_attentions`` ...); the adapter
    passes what the installed release understands instead of pinning one."""
    try:
        params = inspect.signature(fn).parameters
    except (TypeError, ValueError):
        return kwargs
    if any(p.kind is inspect.Parameter.VAR_KEYWORD for p in params.values()):
        return kwargs
    return {k: v for k, v in kwargs.items() if k in params}


def apply_graphed(model, cache, replace_generate: bool = True, recorder=None) -> None:
    """Patch ``model.forward`` in place: one-token calls replay a graph, longer calls
    (prefill) run eagerly; both write into ``cache``.  With ``replace_generate`` the
    model's ``generate`` resets and passes that cache on every call
    (reference ``cudagraph_utils.py:11-80``).

    ``recorder(fn, sample_args)`` turns the one-token step into the callable that replays it;
    the default is :class:`GraphedCallable`."""
    from transformers.modeling_outputs import CausalLMOutputWithPast

    _old_forward = model.forward
    device = model.device
    dtype = model.dtype
    max_len = _max_cache_len(cache)
    key_index = torch.arange(max_len, device=device)

    def _forward(input_ids, attention_mask, position_ids, cache_position):
        with torch.no_grad():
            return _old_forward(**_accepted(_old_forward, dict(
                input_ids=input_ids,
                attention_mask=attention_mask,
                position_ids=position_ids,
                past_key_values=cache,
                output_attentions=False,
                output_hidden_states=False,
                use_cache=True,
                cache_position=cache_position,
                return_dict=True,
            ))).logits

    zero = torch.zeros((), dtype=dtype, device=device)
    minus_inf = torch.full((), float("-inf"), dtype=dtype, device=device)

    def _step(input_ids, cache_position):
        # the one-token step sees every cache slot up to its own position; an additive
        # mask over the whole static cache keeps every shape independent of the position.
        # One elementwise kernel from two constants: nothing is zero-filled inside the
        # capture, so no memset node is recorded.
        visible = key_index[None, None, None, :] <= cache_position.view(1, 1, 1, 1)
        mask = torch.where(visible, zero, minus_inf)
        return _forward(input_ids, mask, cache_position.view(1, 1), cache_position)

    # recorded at the last cache slot so that the warm-up runs do not disturb a prompt
    step = (recorder or GraphedCallable)(_step, (
        torch.zeros(1, 1, dtype=torch.int64, device=device),
        torch.tensor([max_len - 1], dtype=torch.int64, device=device),
    ))
    cache.reset()

    def forward(input_ids=None, attention_mask=None, position_ids=None, cache_position=None, **unused):
        # `unused` swallows what generate() passes besides (past_key_values, use_cache, ...):
        # the cache is the one given to apply_graphed, outputs are logits only
        if cache_position is None:
            start = cache.get_seq_length()
            cache_position = torch.arange(start, start + input_ids.shape[1], device=input_ids.device)
        if input_ids.shape[0] == 1 and input_ids.shape[1] == 1:
            logits = step(input_ids, cache_position.view(1)).clone()
        else:
            logits = _forward(input_ids, attention_mask, position_ids, cache_position)
        return CausalLMOutputWithPast(logits=logits, past_key_values=cache)

    model.forward = forward

    if replace_generate:
        _old_generate = model.generate

        def generate(*args, **kwargs):
            cache.reset()
            # `disable_compile` exists where generate() would otherwise compile the decode
            # step itself; releases without it do not need it
            extra = _accepted(_old_generate, dict(disable_compile=True))
            if extra and 'disable_compile' not in inspect.signature(_old_generate).parameters:
                from transformers import GenerationConfig
                if not hasattr(GenerationConfig(), 'disable_compile'):
                    extra = {}
            return _old_generate(*args, past_key_values=cache, **extra, **kwargs)

        model.generate = generate


def get_graphed_model(model: nn.Module, cache) -> nn.Module:
    """A copy of ``model`` that shares its weights and decodes through a recorded graph
    (reference ``cudagraph_utils.py:83-86``)."""
    graphed_model = shallow_copy_model(model)
    apply_graphed(graphed_model, cache)
    return graphed_model
