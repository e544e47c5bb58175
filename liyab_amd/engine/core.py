"""The engine's core: a model on the device with its cache and step function.

`EngineCore` is what generation, the scheduler and trace replay all drive:
it owns the model, the cache manager with its device memory, and the one
step function. It corresponds to the reference's `Transformer` with its
contexts (`src/core/transformer.h:191-217, 725-764`): `open`/`close` are
`make_context` and its release, `step` is `forward_batch`.
"""

from __future__ import annotations

from typing import Hashable, Optional, Sequence

import torch

from ..cache.pages import CacheManager
from ..cache.storage import CacheStorage
from .. import log
from ..errors import InvalidArgument, KernelError
from ..models.loading import load_model, resolve_dtype
from .step import StepFunction, StepItem


class EngineCore:
    def __init__(self, model_dir: Optional[str] = None, *, dtype="bfloat16", device="cuda:0", page_size: int = 16,
                 num_pages: Optional[int] = None, max_tokens: Optional[int] = None, max_requests: int = 64,
                 context_length: Optional[int] = None, use_graphs: bool = True, model=None, config=None,
                 batch_invariant: bool = False):
        """`model_dir`: a folder with config.json and model.safetensors (or pass a built
        `model`, see `from_plan`). `num_pages`: pages per cache group; or `max_tokens`: the
        most tokens live requests hold together (rounded up to whole pages per request by the
        caller's accounting). With neither, every request slot can reach the full context.
        `batch_invariant`: a request's bfloat16 logits have the same bits alone and in any batch
        (kernels chosen from sizes and positions only: slower; float32 is so either way)."""
        if not torch.cuda.is_available():
            raise KernelError("no GPU is visible: this engine runs on gfx950 only and has no CPU path")
        from ..kernels import ops

        ops.check_device()
        self.device = torch.device(device)
        self.dtype = resolve_dtype(dtype)
        if model is None:
            if model_dir is None:
                raise InvalidArgument("a model folder or a built model is needed")
            self.config, self.model = load_model(model_dir, self.dtype, self.device)
        else:
            self.config, self.model = config, model
        max_positions = self.model.max_positions
        if context_length is not None:
            if context_length <= 0:
                raise InvalidArgument("the context length must be positive")
            max_positions = min(max_positions, context_length)
        if page_size <= 0:
            raise InvalidArgument("page_size must be positive")
        if num_pages is None:
            if max_tokens is not None:
                num_pages = -(-max_tokens // page_size)
            else:
                num_pages = max_requests * (-(-max_positions // page_size))
        self.manager = CacheManager(self.model.cache_groups(), page_size=page_size, num_pages=max(1, num_pages),
                                    max_requests=max_requests, max_positions=max_positions)
        self.storage = CacheStorage(self.manager, self.dtype, self.device, self.model.state_specs())
        self.step_fn = StepFunction(self.model, self.manager, self.storage, self.device, use_graphs=use_graphs,
                                    batch_invariant=batch_invariant)
        # one line at load with the geometry and the cache's cost a token, as the reference logs
        # (src/core/transformer.cpp:880-884)
        plan = self.model.plan
        log.info("%s: %d layers (%d runs), width %d, vocabulary %d, context %d, %s; cache: %d groups, %d pages of %d "
                 "positions each, %.1f KiB a token, %.1f MiB in all",
                 plan.architecture, len(plan.layers), len(plan.order), plan.width, plan.vocab_size, max_positions,
                 str(self.dtype).replace("torch.", ""), len(self.manager.groups), max(1, num_pages), page_size,
                 self.storage.bytes_per_token() / 1024.0, self.storage.bytes_allocated() / 2.0 ** 20)

    @classmethod
    def from_plan(cls, plan, tensors, *, dtype="float32", device="cuda:0", **kw) -> "EngineCore":
        """An engine for a plan and a dict of CPU tensors by name: how a model is built
        without a folder (tests build toy architectures so)."""
        from ..models.decoder import DecoderModel
        from ..weights.loader import WeightStore

        dt = resolve_dtype(dtype)
        store = WeightStore(dict(tensors), device=device, compute_dtype=dt, name_prefixes=plan.name_prefixes,
                            ignorable=plan.ignorable)
        model = DecoderModel(plan, store, dt)
        store.finish()
        return cls(None, dtype=dt, device=device, model=model, config=None, **kw)

    # -- requests -----------------------------------------------------------
    def open(self, rid: Hashable) -> None:
        slot = self.manager.open(rid)
        if self.storage.states:
            self.storage.reset_slot(slot)

    def close(self, rid: Hashable) -> None:
        self.manager.close(rid)

    def is_open(self, rid: Hashable) -> bool:
        return self.manager.is_open(rid)

    def length(self, rid: Hashable) -> int:
        return self.manager.length(rid)

    def truncate(self, rid: Hashable, length: int) -> None:
        if self.storage.states:
            raise InvalidArgument("a model with per-request state cannot be truncated")
        self.manager.truncate(rid, length)

    # -- the step -------------------------------------------------------------
    def step(self, items: Sequence[StepItem]) -> Optional[torch.Tensor]:
        return self.step_fn.run(items)

    @property
    def vocab_size(self) -> int:
        return self.model.vocab_size

    @property
    def max_positions(self) -> int:
        return self.manager.max_positions
