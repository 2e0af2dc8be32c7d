"""The Python entry point: a model on the GPU with its cache, and generate().

The reference's entry points are a binary per architecture (`gemma_run <model> <prompt>`,
runtime/src/bin/gemma_run.rs:1-19) and a C ABI of session_new / generate / session_free
(runtime/include/trapetum.h:13-29); its request options are max_tokens, temperature, top_p and
repetition_penalty (runtime/src/bin/serve.rs:1285-1292).  The same names are used here.
"""
import json
import os

from ..registry import architecture, config_from_folder
from ..sampling.sampler import SamplingParams
from ..weights import RandomWeights, load_folder, load_into
from .generate import generate as _generate
from .model import Model
from .runtime import Runtime


def read_stop_ids(folder):
    """eos_token_id (a number or a list) of generation_config.json, then config.json: runtime/src/bin/serve.rs:83-101."""
    ids = []
    for name in ("generation_config.json", "config.json"):
        path = os.path.join(folder, name)
        if not os.path.isfile(path):
            continue
        try:
            with open(path) as f:
                v = json.load(f).get("eos_token_id")
        except (json.JSONDecodeError, AttributeError):
            continue
        if isinstance(v, int) and not isinstance(v, bool):
            ids.append(v)
        elif isinstance(v, list):
            ids.extend(x for x in v if isinstance(x, int) and not isinstance(x, bool))
    return tuple(sorted(set(ids)))


class Engine:
    """A model ready to generate.

    max_tokens_in_cache: tokens that live sequences may hold together (each rounded up to a page);
    max_context: the longest single sequence; max_batch: sequences that run together.
    """

    def __init__(self, model, config, stop_ids=(), max_tokens_in_cache=16384, max_context=None, max_batch=64,
                 page_size=64, use_graph=True):
        self.model = model
        self.config = config
        self.stop_ids = tuple(stop_ids)
        self.max_batch = max_batch
        limit = getattr(config, "max_position_embeddings", None)
        if max_context is None:
            max_context = min(max_tokens_in_cache, limit) if limit else max_tokens_in_cache
        self.cache = model.new_cache(max_tokens_in_cache, max_context=max_context, max_slots=max_batch, page_size=page_size)
        self.graphed = None
        from .. import flags
        if use_graph and model.rt.device.type == "cuda" and flags.graphs_allowed():
            from .graphs import GraphedDecode
            self.graphed = GraphedDecode(model, self.cache)

    @classmethod
    def from_folder(cls, folder, dtype="bfloat16", device="cuda:0", **kw):
        arch, config = config_from_folder(folder)
        model = Model(arch.build_spec(config), Runtime(dtype=dtype, device=device))
        load_folder(model, folder)
        return cls(model, config, stop_ids=read_stop_ids(folder), **kw)

    @classmethod
    def from_config(cls, config, seed=0, sigma=0.02, sigma_norm=0.1, dtype="bfloat16", device="cuda:0",
                    draw_on_device=False, **kw):
        """Random weights without a folder: drawn as `write_model_folder` draws them, or (draw_on_device) on
        the GPU, which is quicker for large models and gives other values."""
        arch = architecture(config.architecture)
        model = Model(arch.build_spec(config), Runtime(dtype=dtype, device=device))
        load_into(model, RandomWeights(model.tensor_layout(), seed, sigma, sigma_norm,
                                       draw_on=device if draw_on_device else None))
        return cls(model, config, stop_ids=(), **kw)

    def generate(self, prompts, max_tokens=256, temperature=0.0, top_p=0.95, top_k=256, repetition_penalty=1.0,
                 seed=0, stop_ids=None, on_tokens=None, with_reasons=False, request_ids=None):
        """prompts: a list of token-id lists.  Returns the generated ids of each prompt.  request_ids (integers, default
        a prompt's place in the list) key the sampler's random numbers beside `seed`: a request keeps its tokens
        whatever else is in the call if it keeps its id."""
        if prompts and isinstance(prompts[0], int):
            raise TypeError("prompts is a list of token-id lists (one list per request)")
        params = SamplingParams(temperature=temperature, top_p=top_p, top_k=top_k, repetition_penalty=repetition_penalty)
        stops = self.stop_ids if stop_ids is None else tuple(stop_ids)
        return _generate(self.model, self.cache, prompts, max_tokens=max_tokens, params=params, seed=seed,
                         stop_ids=stops, max_batch=self.max_batch, on_tokens=on_tokens, with_reasons=with_reasons,
                         graphs=self.graphed, request_ids=request_ids)


def load_model(folder, **kw):
    return Engine.from_folder(folder, **kw)
