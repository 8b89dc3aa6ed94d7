"""Loading a model and generating with it: the Python entry point.

In the manner of the reference: `load_model(name, device, dtype)` (serve/utils.py:41-58),
`Request(input_ids, input_length, max_new_tokens, generated_tokens, logits)`
(serve/run.py:16-22) and `generate(model, requests, temperature, return_logits)`
(serve/run.py:238-308) keep their names and meanings; `model_name` is a model folder
(config.json + model.safetensors), since nothing is downloaded here.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import List, Optional, Sequence, Union

import torch

from ..config.engine import EngineConfig
from ..models.model import Model
from ..parts.base import Runtime
from ..registry import get_architecture, load_config
from ..sampling.sampler import Sampler
from ..weights.loader import load_weights, random_reader
from ..weights.safetensors_io import CheckpointReader
from .runner import ModelRunner, require_gpu, _TORCH_DTYPE
from .scheduler import GenerationRequest, Scheduler


@dataclass
class Request:
    """A generation request and, after `generate`, its result (serve/run.py:16-22)."""

    input_ids: torch.Tensor
    input_length: int
    max_new_tokens: int
    generated_tokens: torch.Tensor = field(default_factory=lambda: torch.tensor([], dtype=torch.long))
    logits: Optional[torch.Tensor] = None
    # why the request ended without (all of) its tokens: it exceeds max_context, does not fit into
    # the cache, has an empty prompt; None when it ran to its end
    error: Optional[str] = None


def _dtype_name(dtype) -> str:
    if isinstance(dtype, torch.dtype):
        for k, v in _TORCH_DTYPE.items():
            if v == dtype:
                return k
        raise ValueError(f"dtype {dtype} is not supported; use torch.bfloat16 or torch.float32")
    name = {"bf16": "bfloat16", "fp32": "float32"}.get(str(dtype), str(dtype))
    if name not in _TORCH_DTYPE:
        raise ValueError(f"dtype {dtype!r} is not supported; use 'bfloat16' or 'float32'")
    return name


class Engine:
    """A model on one GPU with its cache, step function, scheduler and sampler."""

    def __init__(self, model: Model, runner: ModelRunner, cfg: EngineConfig, model_config=None):
        self.model, self.runner, self.cfg, self.model_config = model, runner, cfg, model_config
        self.sampler = Sampler(cfg.seed, runner.rt.device)

    # -- construction -----------------------------------------------------------------------------
    @staticmethod
    def _build(arch, config, reader, cfg: EngineConfig) -> "Engine":
        cfg.validate()
        device = require_gpu(cfg.device)
        rt = Runtime(device, _TORCH_DTYPE[cfg.dtype], max_context=cfg.max_context)
        model = Model(arch.build_spec(config))
        with torch.cuda.device(device):
            load_weights(model, reader(model) if callable(reader) else reader, rt)
            runner = ModelRunner(model, rt, cfg)
        return Engine(model, runner, cfg, config)

    @staticmethod
    def from_folder(folder: str, cfg: Optional[EngineConfig] = None) -> "Engine":
        """Load `folder/config.json` and `folder/model.safetensors` (or its shards)."""
        arch, config = load_config(folder)
        return Engine._build(arch, config, CheckpointReader(folder), cfg or EngineConfig())

    @staticmethod
    def from_config(config, seed: int, cfg: Optional[EngineConfig] = None,
                    weight_dtype: torch.dtype = torch.bfloat16) -> "Engine":
        """Random weights for a typed configuration, without a folder on disk."""
        arch = get_architecture(config.architecture)
        return Engine._build(arch, config, lambda m: random_reader(m, seed, weight_dtype), cfg or EngineConfig())

    # -- use --------------------------------------------------------------------------------------
    def step(self, segments) -> torch.Tensor:
        return self.runner.step(segments)

    def stop_ids(self, stop_token_ids) -> Optional[List[int]]:
        """None; "eos": the end-of-sequence ids of the model's configuration; or a list of ids."""
        if stop_token_ids is None:
            return None
        if isinstance(stop_token_ids, str):
            if stop_token_ids != "eos":
                raise ValueError(f"stop_token_ids must be None, 'eos' or a list of token ids, not {stop_token_ids!r}")
            ids = self.model.spec.eos_token_ids
            if not ids:
                raise ValueError("stop_token_ids='eos': the model's configuration names no eos_token_id")
            return list(ids)
        ids = [int(t) for t in stop_token_ids]
        for t in ids:
            if not 0 <= t < self.model.spec.vocab_size:
                raise ValueError(f"stop token {t} is outside the vocabulary [0, {self.model.spec.vocab_size})")
        return ids

    def generate(self, requests: Sequence[Request], temperature: Union[float, Sequence[float]] = 0.0,
                 return_logits: Union[bool, str] = False, stop_token_ids=None,
                 raise_on_error: bool = False, step_log: Optional[list] = None) -> List[Request]:
        """Generate up to `max_new_tokens` tokens for every request; results in the order given
        (serve/run.py:304).  `temperature` 0 is greedy (serve/run.py:56-57); one value for all
        requests as in the reference, or one per request.  `return_logits`: False / "none"; True /
        "last": the fp32 logits [V] that the last token was drawn from, as the reference returns
        them (serve/run.py:229-230); "all": those of every generated token, [generated, V].
        `stop_token_ids`: None (the reference's behaviour: a request ends at `max_new_tokens`
        only, serve/run.py:222), "eos" (the configuration's end-of-sequence ids) or a list of
        ids; a request ends with the first of them it generates, which stays in its tokens.
        A request that cannot run (longer than max_context, larger than the cache, empty) comes
        back with `error` set and without tokens; with `raise_on_error` that is a ValueError
        naming all of them, raised after the others have finished.  `step_log`: a list that
        receives one record per step (requests, their token counts, who was sampled)."""
        if return_logits not in (False, True, "none", "last", "all"):
            raise ValueError(f"return_logits must be False, True, 'none', 'last' or 'all', not {return_logits!r}")
        keep_all = return_logits == "all"
        keep_last = return_logits is True or return_logits == "last"
        temps = list(temperature) if isinstance(temperature, (list, tuple)) else [float(temperature)] * len(requests)
        if len(temps) != len(requests):
            raise ValueError("one temperature per request is needed")
        gen = []
        for i, (r, t) in enumerate(zip(requests, temps)):
            ids = r.input_ids.tolist() if isinstance(r.input_ids, torch.Tensor) else list(r.input_ids)
            if r.input_length != len(ids):
                raise ValueError(f"request {i}: input_length {r.input_length} != len(input_ids) {len(ids)}")
            gen.append(GenerationRequest(req_id=i, prompt=ids, max_new_tokens=int(r.max_new_tokens),
                                         temperature=float(t), keep_logits=keep_last, keep_all_logits=keep_all))
        sched = Scheduler(self.runner, self.sampler, self.cfg, eos_token_ids=self.stop_ids(stop_token_ids),
                          record_steps=step_log is not None)
        try:
            done = sched.run(gen)
        except BaseException:
            # a step failed: give back what this call's requests hold, so that the engine can go on
            sched.abort()
            raise
        finally:
            if step_log is not None:
                step_log.extend(sched.step_log)
        out = []
        for r, g in zip(requests, done):
            out.append(Request(input_ids=r.input_ids, input_length=r.input_length,
                               max_new_tokens=r.max_new_tokens,
                               generated_tokens=torch.tensor(g.generated, dtype=torch.long),
                               logits=(torch.stack(g.logit_rows) if keep_all and g.logit_rows
                                       else g.last_logits if keep_last else None),
                               error=g.error))
        failed = [(i, o.error) for i, o in enumerate(out) if o.error]
        if failed and raise_on_error:
            raise ValueError("requests that could not run: " + "; ".join(f"request {i}: {e}" for i, e in failed))
        return out


# ---------------------------------------------------------------------------------------------
# the reference's function names
# ---------------------------------------------------------------------------------------------

def load_model(model_name: str, device: str = "cuda", dtype=torch.bfloat16, **engine_options) -> Engine:
    """serve/utils.py:41-58.  `model_name` is the folder of the model.  Returns the engine (the
    reference also returns a tokenizer, which `generate` never uses: it takes token ids)."""
    dev = "cuda:0" if device in ("cuda", "gpu") else device
    cfg = EngineConfig(dtype=_dtype_name(dtype), device=dev, **engine_options)
    return Engine.from_folder(model_name, cfg)


def generate(model: Engine, requests: Sequence[Request], temperature: float = 0.0,
             return_logits: Union[bool, str] = False, stop_token_ids=None,
             raise_on_error: bool = False) -> List[Request]:
    """serve/run.py:238-308; `stop_token_ids` and `raise_on_error` as in `Engine.generate`."""
    return model.generate(requests, temperature=temperature, return_logits=return_logits,
                          stop_token_ids=stop_token_ids, raise_on_error=raise_on_error)
