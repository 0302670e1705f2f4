"""The generic decoder: embedding, blocks in a run order, final norm, output projection.

The model is data: a list of layers (each a block put together from registered parts) and a run
order that may name a layer twice or let an entry read an earlier entry's cache.  Nothing here
knows an architecture; a builder registered under the architecture's name makes one of these from
its configuration (see ``models/qwen2.py``).

Order of a step as in the reference's batched pass (crates/vipera-backend-cpu/src/model.rs:956-1237):
embed, the layers, then norm and output projection for the rows whose logits are wanted.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, List, Optional

import torch

from ..config.base import ModelConfig, ScheduleEntry
from ..errors import InvalidArgumentError
from ..parts.base import KVCacheSpec, StateSpec, part_class
from ..weights.checkpoint import TensorSpec


@dataclass
class CacheNeed:
    """What one entry of the run order keeps per request; ``owner`` is the entry whose storage it uses."""

    owner: int
    kv: Optional[KVCacheSpec]
    state: Optional[StateSpec]


def check_schedule(schedule: List[ScheduleEntry], num_layers: int) -> None:
    for index, entry in enumerate(schedule):
        if not 0 <= entry.layer < num_layers:
            raise InvalidArgumentError(f"run order entry {index} names layer {entry.layer} of {num_layers}")
        if entry.cache_of is not None:
            if not 0 <= entry.cache_of < index:
                raise InvalidArgumentError(
                    f"run order entry {index} reads the cache of entry {entry.cache_of}, which does not come before it")
            if schedule[entry.cache_of].cache_of is not None:
                raise InvalidArgumentError(
                    f"run order entry {index} reads the cache of entry {entry.cache_of}, which owns none")


def declare_model(config: ModelConfig) -> List[TensorSpec]:
    """Every tensor the model of ``config`` needs. Touches no GPU."""
    specs: List[TensorSpec] = []
    emb = config.embedding_spec()
    specs += part_class("embedding", emb.kind).declare(emb, "")
    for layer in config.layer_specs():
        specs += part_class("block", layer.block).declare(layer)
    norm = config.final_norm_spec()
    specs += part_class("norm", norm.kind).declare(norm, "")
    head = config.head_spec()
    specs += part_class("head", head.kind).declare(head, "")
    seen = set()
    for spec in specs:
        if spec.name in seen:
            raise InvalidArgumentError(f"tensor \"{spec.name}\" is declared twice")
        seen.add(spec.name)
    return specs


def check_model(config: ModelConfig, dtype) -> None:
    """Raise ``UnsupportedError`` if some part of ``config``'s model has a size that no kernel takes in a run of
    ``dtype``.  Touches no GPU and reads no weight: it is what opening a model does first."""
    emb = config.embedding_spec()
    part_class("embedding", emb.kind).check_supported(emb, dtype)
    for layer in config.layer_specs():
        part_class("block", layer.block).check_supported(layer, dtype)
    norm = config.final_norm_spec()
    part_class("norm", norm.kind).check_supported(norm, dtype)
    head = config.head_spec()
    part_class("head", head.kind).check_supported(head, dtype)


def declare_cache_needs(config: ModelConfig) -> List[CacheNeed]:
    """What every entry of ``config``'s run order keeps per request, from the configuration alone. Touches no GPU."""
    layers = config.layer_specs()
    schedule = list(config.schedule())
    check_schedule(schedule, len(layers))
    needs = []
    for index, entry in enumerate(schedule):
        mixer = layers[entry.layer].mixer
        kv, state = part_class("mixer", mixer.kind).declare_cache(mixer)
        needs.append(CacheNeed(index if entry.cache_of is None else entry.cache_of, kv, state))
    return needs


class DecoderModel:
    def __init__(self, config: ModelConfig, runtime):
        self.config = config
        self.runtime = runtime
        check_model(config, runtime.dtype)    # sizes that no kernel takes are refused here, before weights are read
        emb, norm, head = config.embedding_spec(), config.final_norm_spec(), config.head_spec()
        self.embedding = part_class("embedding", emb.kind)(emb, "", runtime)
        self.layers = [part_class("block", spec.block)(spec, runtime) for spec in config.layer_specs()]
        self.final_norm = part_class("norm", norm.kind)(norm, "", runtime)
        self.head = part_class("head", head.kind)(head, "", runtime)
        self.schedule = list(config.schedule())
        check_schedule(self.schedule, len(self.layers))
        self.vocab_size = self.head.vocab
        self.loaded = False

    def tensor_specs(self) -> List[TensorSpec]:
        return declare_model(self.config)

    def load(self, tensors: Dict[str, torch.Tensor]) -> None:
        self.embedding.load(tensors)
        for layer in self.layers:
            layer.load(tensors)
        self.final_norm.load(tensors)
        self.head.load(tensors)
        self.loaded = True

    def cache_needs(self) -> List[CacheNeed]:
        needs = []
        for index, entry in enumerate(self.schedule):
            mixer = self.layers[entry.layer].mixer
            owner = index if entry.cache_of is None else entry.cache_of
            needs.append(CacheNeed(owner, mixer.cache_spec(), mixer.state_spec()))
        for index, need in enumerate(needs):
            if need.owner != index and (needs[need.owner].kv != need.kv or needs[need.owner].state != need.state):
                raise InvalidArgumentError(
                    f"run order entry {index} reads the cache of entry {need.owner}, whose shape differs")
        return needs

    def forward(self, batch, storage) -> Optional[torch.Tensor]:
        """Run the step's tokens through the run order; returns ``[wanted rows, vocab]`` 32-bit logits."""
        # what parts share within a step is computed anew in every run: a run that is being captured into a graph
        # must launch it too, or the graph would replay with what an earlier run left
        batch.shared.clear()
        batch.launch_plans.clear()
        x = self.embedding.embed(batch)
        tokens = x.shape[0]
        incoming = None
        for index, entry in enumerate(self.schedule):
            owner = index if entry.cache_of is None else entry.cache_of
            layer = self.layers[entry.layer]
            if not layer.hands_off:
                layer.forward(x, batch, storage.kv[owner], storage.state[owner], reads_only=entry.cache_of is not None)
                incoming = None
                continue
            # the next layer's first norm may be prepared by this layer's last product (see parts.NormHandoff)
            outgoing = None
            if index + 1 < len(self.schedule) and layer.fills_outgoing():
                following = self.layers[self.schedule[index + 1].layer]
                if following.hands_off:
                    outgoing = following.accepts_incoming(tokens, batch)
            layer.forward(x, batch, storage.kv[owner], storage.state[owner], reads_only=entry.cache_of is not None,
                          incoming=incoming, outgoing=outgoing)
            incoming = outgoing
        if batch.num_logit_rows == 0:
            return None
        h = self.final_norm.forward(x, rows=batch.logit_rows)
        return self.head.forward(h)
