"""The Python entry point in the reference's own manner.

The reference's program fills a ``ModelConfig`` by hand, then calls
``load_model``, ``init_runtime_context``, ``encode`` and ``infer`` on an
``LLMInferRuntime`` (test/main.cu:17-66; the class in
src/core/runtime/InferRuntime.h:32-157).  The same four calls work here, with
the same option names where the reference has them; prompts are lists of token
ids, since the engine holds no tokenizer.

    rt = LLMInferRuntime()
    cfg = ModelConfig(); cfg._use_f16 = True; cfg._n_output = 1
    rt.load_model(["/path/to/model_dir"], cfg)
    rt.init_runtime_context()
    rt.encode([[1, 2, 3], [4, 5]])
    out = []; rt.infer(64, out)        # out: one list of new token ids per prompt
"""
from __future__ import annotations

import json
import os
from dataclasses import dataclass, field

import torch

from . import log
from .engine.llm_engine import EngineOptions, LLMEngine
from .models import build_model_skeleton, config_from_dict, load_config
from .sampling import SamplingConfig
from .weights import load_model_dir

MAX_SEQ_LENGTH = 8192   # the reference's default _n_ctx (src/core/global/GlobalDefine.h:40)


@dataclass
class ModelConfig:
    """Caller-set options under the reference's names
    (src/core/model/BaseDefine.h:101-149).  Sizes of the model are not here:
    they come from the model folder's config.json."""
    _use_f16: bool = True              # True: the 16-bit path (bfloat16 here); False: true 32-bit
    _kv_data_type: str | None = None   # must agree with the path's type if given ("bf16" / "f32")
    _is_fuse_op: bool = True           # the engine always runs its fused kernels
    _use_mmap: bool = True             # weight files are always memory-mapped
    _n_ctx: int = MAX_SEQ_LENGTH       # longest sequence (capped by max_position_embeddings)
    _n_output: int = 1                 # logits rows per step and request; only 1 is meaningful
    _rope_freq_base: float | None = None   # overrides config.json's rope_theta when set (test/main.cu:26)
    _rope_freq_scale: float = 1.0      # carried and unused by the reference; must stay 1
    _sampling_config: SamplingConfig = field(default_factory=SamplingConfig)
    # engine options that the reference fixes at compile time
    _page_size: int = 16               # PAGE_SIZE (src/core/runtime/KVCache.h:16), 32 there
    _max_batches: int = 8              # most sequences in flight
    _max_batch_tokens: int = 2048      # token budget of a step
    _prefill_chunk: int = 512
    _kv_tokens: int | None = None      # tokens the cache holds, or
    _num_pages: int | None = None      # pages per group of layers, or
    _kv_bytes: int | None = None       # bytes of device memory for keys and values
    _use_graphs: bool = True
    _warm_up: bool = False


class LLMInferRuntime:
    def __init__(self):
        self._model = None
        self._model_config = None
        self._params = None
        self._engine = None
        self._prompts = []

    def _check_params(self, params: ModelConfig) -> torch.dtype:
        if params._rope_freq_scale != 1.0:
            raise ValueError("_rope_freq_scale other than 1 is not supported")
        if params._n_output != 1:
            raise ValueError("_n_output other than 1 is not supported")
        dtype = torch.bfloat16 if params._use_f16 else torch.float32
        if params._kv_data_type is not None:
            want = {"bf16": torch.bfloat16, "bfloat16": torch.bfloat16, "f32": torch.float32,
                    "float32": torch.float32}.get(str(params._kv_data_type).lower())
            if want != dtype:
                raise ValueError(f"_kv_data_type={params._kv_data_type!r} does not match the "
                                 f"{'16' if params._use_f16 else '32'}-bit path")
        return dtype

    @staticmethod
    def _apply_caller_options(config, params: ModelConfig):
        """Options of the caller that override the model's own configuration.  Which key of the
        architecture an option means is the configuration class's business (``caller_options``)."""
        if params._rope_freq_base is not None:
            key = getattr(config, "caller_options", {}).get("rope_freq_base")
            if key is None:
                raise ValueError(f"{type(config).__name__} has no rotation base that _rope_freq_base could override")
            config = config.with_overrides(**{key: float(params._rope_freq_base)})
        return config

    def load_model(self, model_files_path, params: ModelConfig) -> bool:
        """``model_files_path``: a list whose first entry is the model folder
        (or a file in it), as the reference takes a list of files."""
        path = model_files_path[0] if isinstance(model_files_path, (list, tuple)) else model_files_path
        if os.path.isfile(path):
            path = os.path.dirname(path)
        dtype = self._check_params(params)
        config = self._apply_caller_options(load_config(path), params)
        model = build_model_skeleton(config)
        model.load_tensors(load_model_dir(path), dtype, "cuda:0", where=path)
        self._model, self._model_config, self._params = model, config, params
        log.info("model %s: %s, %s", path, type(config).__name__, "bfloat16" if params._use_f16 else "float32")
        return True

    def random_model(self, config, seed: int, params: ModelConfig, on_device: bool = False) -> bool:
        """A model with seeded random weights and no files: ``config`` is a config.json path, its
        dict or a typed configuration.  The weights are those that ``write_random_model`` puts
        into a folder for the same seed (``on_device``: drawn on the GPU instead, another stream
        of numbers, for models too large to draw on the host in reasonable time)."""
        if isinstance(config, (str, os.PathLike)):
            with open(config) as f:
                config = json.load(f)
        if isinstance(config, dict):
            config = config_from_dict(config)
        dtype = self._check_params(params)
        config = self._apply_caller_options(config, params)
        model = build_model_skeleton(config)
        model.init_random(int(seed), dtype, "cuda:0", on_device=on_device)
        self._model, self._model_config, self._params = model, config, params
        log.info("random model from seed %d: %s", seed, type(config).__name__)
        return True

    def init_runtime_context(self) -> bool:
        """Sets up the cache and the step function (the reference's
        ``init_kvcache`` + weight upload, src/core/runtime/InferRuntime.cu:81-171)."""
        if self._model is None:
            return False
        p = self._params
        opt = EngineOptions(dtype=self._model.dtype, page_size=p._page_size, max_num_seqs=p._max_batches,
                            max_num_batched_tokens=p._max_batch_tokens, prefill_chunk=p._prefill_chunk,
                            max_model_len=p._n_ctx, kv_tokens=p._kv_tokens, num_pages=p._num_pages,
                            kv_bytes=p._kv_bytes, use_graphs=p._use_graphs, warm_up=p._warm_up)
        self._engine = LLMEngine(self._model, opt)
        return True

    @property
    def engine(self) -> LLMEngine:
        return self._engine

    def encode(self, prompt_batches) -> int:
        """Takes the prompts (token id lists).  Returns the number of tokens.
        The reference tokenizes strings here and truncates what is longer than
        the context (src/core/runtime/InferRuntime.cu:383-425); ids are taken
        as they are and too long a prompt is refused when it is added."""
        self._prompts = []
        for p in prompt_batches:
            if isinstance(p, str):
                raise TypeError("prompts are lists of token ids; the engine holds no tokenizer")
            self._prompts.append([int(t) for t in p])
        return sum(len(p) for p in self._prompts)

    def infer(self, n_predict: int, generate_out: list) -> bool:
        """Generates up to ``n_predict`` tokens for every encoded prompt and
        appends one list of new token ids per prompt to ``generate_out``."""
        if self._engine is None or not self._prompts:
            return False
        res = self._engine.generate(self._prompts, self._params._sampling_config, max_new_tokens=n_predict)
        generate_out.extend(r.output for r in res)
        return True
