"""Turns a ModelSpec into objects: parts from the registries, tensors from a checkpoint, and the
forward pass over a step's batch."""
from __future__ import annotations

from typing import Any, Dict, List, Mapping, Optional, Tuple

import torch

from .. import parts as _parts  # noqa: F401  (registers the built-in part kinds)
from . import llama as _llama   # noqa: F401  (registers LlamaForCausalLM)
from ..config.registry import (BLOCKS, FEED_FORWARDS, MIXERS, NORMS, architecture_for)
from ..models.spec import LayerCall, ModelSpec, TensorSpec
from ..ops import kernels as K
from ..parts.base import Block, KVCacheSpec, KVView, MixerContext, NormedRows, StateSpec
from ..parts.linear import Linear


def spec_for_config(config_dict: Mapping[str, Any]) -> Tuple[Any, ModelSpec]:
    arch = architecture_for(config_dict)
    config = arch.parse_config(config_dict)
    return config, arch.build_spec(config)


def build_blocks(spec: ModelSpec) -> List[Block]:
    blocks = []
    for ls in spec.layers:
        mixer = MIXERS.get(ls.mixer.kind)(**ls.mixer.params)
        ffn = FEED_FORWARDS.get(ls.feed_forward.kind)(**ls.feed_forward.params)
        norms = {name: NORMS.get(ns.kind)(**ns.params) for name, ns in ls.norms.items()}
        blocks.append(BLOCKS.get(ls.block.kind)(mixer, ffn, norms, **ls.block.params))
    return blocks


def model_tensor_specs(spec: ModelSpec, blocks: List[Block], final_norm) -> Dict[str, TensorSpec]:
    out: Dict[str, TensorSpec] = {spec.embedding_name: TensorSpec((spec.vocab_size, spec.hidden_size))}
    for b in blocks:
        for part in b.parts():
            for name, ts in part.tensor_specs().items():
                if name in out and out[name] != ts:
                    raise ValueError(f"tensor {name!r} is declared twice with different specs")
                out[name] = ts
    out.update(final_norm.tensor_specs())
    if spec.head_name is not None:
        out[spec.head_name] = TensorSpec((spec.vocab_size, spec.hidden_size))
    return out


def tensor_specs_for_config(config_dict: Mapping[str, Any]) -> Dict[str, TensorSpec]:
    """Names, shapes and init rules of every tensor a model folder for this config holds."""
    _, spec = spec_for_config(config_dict)
    blocks = build_blocks(spec)
    final_norm = NORMS.get(spec.final_norm.kind)(**spec.final_norm.params)
    return model_tensor_specs(spec, blocks, final_norm)


def resolve_order(spec: ModelSpec) -> List[Tuple[LayerCall, int]]:
    """(call, cache slot id) per entry of the run order; ``cache=None`` gets a private slot."""
    used = {c.cache for c in spec.order if c.cache is not None}
    nxt = (max(used) + 1) if used else 0
    out = []
    for call in spec.order:
        if not 0 <= call.layer < len(spec.layers):
            raise ValueError(f"run order names layer {call.layer}, the model has {len(spec.layers)}")
        slot = call.cache
        if slot is None:
            slot, nxt = nxt, nxt + 1
        out.append((call, slot))
    return out


class Model:
    """Parts built from a ModelSpec, holding their tensors, run over a StepBatch."""

    def __init__(self, spec: ModelSpec, dtype: torch.dtype, device):
        self.spec, self.dtype, self.device = spec, dtype, torch.device(device)
        self.blocks = build_blocks(spec)
        self.final_norm = NORMS.get(spec.final_norm.kind)(**spec.final_norm.params)
        self.calls = resolve_order(spec)
        self.embedding: Optional[torch.Tensor] = None
        self.head: Optional[Linear] = None

    # ---- what the cache manager has to provide
    @property
    def portion_multiple(self) -> int:
        """Positions at whose multiples a prompt may be cut into portions: the least common
        multiple of what the layers' mixers ask for."""
        import math
        m = 1
        for block in self.blocks:
            m = math.lcm(m, max(1, int(getattr(block.mixer, "portion_multiple", 1))))
        return m

    def cache_requirements(self):
        """(groups, states): groups = [(KVCacheSpec, [cache slot ids])] for slots that need paged
        K/V, states = {cache slot id: StateSpec}."""
        slot_spec: Dict[int, KVCacheSpec] = {}
        slot_writer: Dict[int, bool] = {}
        states: Dict[int, StateSpec] = {}
        for call, slot in self.calls:
            mixer = self.blocks[call.layer].mixer
            kv = mixer.kv_cache_spec()
            if kv is not None:
                if slot in slot_spec and slot_spec[slot] != kv:
                    raise ValueError(f"cache slot {slot} is shared by mixers with different needs")
                slot_spec[slot] = kv
                slot_writer[slot] = slot_writer.get(slot, False) or call.writes_cache
            st = mixer.state_spec()
            if st is not None:
                if slot in states and states[slot] != st:
                    raise ValueError(f"state slot {slot} is shared by mixers with different state")
                states[slot] = st
        for slot, has_writer in slot_writer.items():
            if not has_writer:
                raise ValueError(f"cache slot {slot} is read but no layer call writes it")
        groups: Dict[KVCacheSpec, List[int]] = {}
        for slot in sorted(slot_spec):
            groups.setdefault(slot_spec[slot], []).append(slot)
        return list(groups.items()), states

    def step_activation_bytes(self, tokens: int, logit_rows: Optional[int] = None) -> int:
        """Upper estimate of the device memory one step of ``tokens`` tokens needs beside weights
        and cache: the residual stream and a branch output, twice the widest layer's intermediate
        results (one layer's are freed while the next one's are made) and fp32 logits at
        ``logit_rows`` places (default: every token).  The engine reserves this much once, and
        leaves it out when it sizes the cache pool from leftover memory."""
        elem = torch.empty((), dtype=self.dtype).element_size()
        widest = max((sum(part.activation_elements() for part in b.parts()) for b in self.blocks), default=0)
        rows = int(tokens if logit_rows is None else logit_rows)
        return int(tokens) * (3 * self.spec.hidden_size + 2 * widest) * elem + rows * 4 * self.spec.vocab_size

    def graph_safe(self) -> bool:
        """Whether every part may be captured into a HIP graph."""
        parts = [self.final_norm]
        for b in self.blocks:
            parts.append(b)
            parts.extend(b.parts())
            pos = getattr(b.mixer, "position", None)
            if pos is not None:
                parts.append(pos)
        return all(getattr(p, "graph_safe", False) for p in parts)

    def limit_positions(self, positions: int) -> None:
        """Tells every part that keeps something per position (tables of a position encoding) that
        no position at or past ``positions`` will be asked for."""
        for b in self.blocks:
            for part in (*b.parts(), getattr(b.mixer, "position", None)):
                limit = getattr(part, "limit_positions", None)
                if limit is not None:
                    limit(positions)
                    part.tables(self.device)        # made now: they count when the cache pool is sized from what is left

    # ---- weights
    def tensor_specs(self) -> Dict[str, TensorSpec]:
        return model_tensor_specs(self.spec, self.blocks, self.final_norm)

    def load(self, tensors: Dict[str, torch.Tensor]) -> None:
        self.embedding = tensors[self.spec.embedding_name]
        for b in self.blocks:
            for part in b.parts():
                part.load(tensors)
        self.final_norm.load(tensors)
        head = tensors[self.spec.head_name] if self.spec.head_name is not None else self.embedding
        self.head = Linear(head)

    @staticmethod
    def block_linears(block) -> List[Linear]:
        """Every Linear the block's parts hold as an attribute, or inside an attribute that wraps
        one as ``.linear``."""
        out = []
        for part in block.parts():
            for v in vars(part).values():
                if isinstance(v, Linear):
                    out.append(v)
                elif isinstance(getattr(v, "linear", None), Linear):
                    out.append(v.linear)
        return out

    def linears(self) -> List[Linear]:
        """Every Linear of every block, in layer order."""
        return [lin for b in self.blocks for lin in self.block_linears(b)]

    def tune_products(self, row_counts, say=None) -> List[dict]:
        """For every row count, has the vendor GEMM library's algorithms timed for each shape of
        bf16 Linear that goes to the library at that many rows (``ops.kernels.gemm_vendor_tune``;
        the same projection of all layers shares a shape and the layers' weights are used in
        turn).  Seconds per shape: start-up work.  Returns one record per (rows, shape)."""
        from ..ops.gemm_bf16 import use_skinny
        shapes: Dict[tuple, List[Linear]] = {}
        for lin in self.linears():
            if lin.weight.is_cuda and lin.weight.dtype == torch.bfloat16:
                shapes.setdefault((lin.out_features, lin.in_features, lin.halves), []).append(lin)
        report = []
        for rows in sorted(set(int(r) for r in row_counts)):
            for (n, k, halves), lins in shapes.items():
                if lins[0].tiled is not None and (use_skinny(rows, n, k, halves == 2) or use_skinny(rows, n, k)):
                    continue                                    # the few-rows kernel takes these
                first, best, tried = K.gemm_vendor_tune(rows, [lin.weight for lin in lins[:16]])
                report.append(dict(rows=rows, n=n, k=k, heuristic_us=round(first, 2), kept_us=round(best, 2),
                                   algorithms_run=tried))
                if say is not None:
                    say(f"vendor product {rows} x {k} -> {n}: {first:.1f} us by the library's choice, "
                        f"{best:.1f} us by the fastest of {tried}")
        return report

    # ---- forward
    GATHER_PREP_MAX_ROWS = 64       # steps of at most this many tokens gather and prepare the first norm in one kernel

    def forward(self, batch, cache) -> torch.Tensor:
        """Runs the batch's tokens through every layer call and returns fp32 logits
        ``[len(batch.logit_rows), vocab]``."""
        T = batch.num_tokens
        hidden = torch.empty((T, self.spec.hidden_size), dtype=self.dtype, device=self.device)
        delta = None
        first_norm = self.blocks[self.calls[0][0].layer].first_norm() if self.calls else self.final_norm
        prep = first_norm.prepared_by_product() if first_norm is not None else None
        if (T <= self.GATHER_PREP_MAX_ROWS and prep is not None and prep[1] == self.spec.hidden_size
                and self.dtype == torch.bfloat16 and self.embedding.dtype == torch.bfloat16
                and self.spec.hidden_size % 8 == 0 and self.spec.embedding_scale == 1.0):
            # a few tokens: the gather prepares the first norm as a product's epilogue would, and
            # the first product finishes it (or one kernel does, as the norm kernel would have)
            scaled = torch.empty_like(hidden)
            sumsq = torch.empty((T, 1), dtype=torch.float32, device=self.device)
            K.embed_gather_prep(self.embedding, batch.token_ids, hidden, scaled, sumsq, prep[0],
                                getattr(batch, "feedback", None))
            delta = NormedRows(scaled, sumsq, prep[1], prep[2], first_norm)
        else:
            K.embed_gather(self.embedding, batch.token_ids, hidden, getattr(batch, "feedback", None))
            if self.spec.embedding_scale != 1.0:
                K.scale_softcap(hidden, self.spec.embedding_scale)
        for i, (call, slot) in enumerate(self.calls):
            block = self.blocks[call.layer]
            # the norm that reads the residual stream after this block
            next_norm = (self.blocks[self.calls[i + 1][0].layer].first_norm()
                         if i + 1 < len(self.calls) else self.final_norm)
            ctx = MixerContext(batch=batch)
            group = cache.group_of(slot)
            if group is not None:
                _, arrays = cache.kv_arrays(slot)
                ctx.kv = KVView(arrays, group.table_dev, batch.slot_mapping[group.index],
                                group.page_size, writes=call.writes_cache)
            if slot in cache.state:
                ctx.state = cache.state[slot]
            hidden, delta = block.forward(hidden, delta, ctx, next_norm)
        R = batch.num_logit_rows
        logits = torch.empty((R, self.spec.vocab_size), dtype=torch.float32, device=self.device)
        if R == 0:
            return logits
        if isinstance(delta, NormedRows):
            if R == T and batch.logits_for_all_rows:
                x = delta                    # the head's product finishes the final norm
            else:
                x = delta.materialize(batch.logit_rows)
        else:
            x = self.final_norm.forward(hidden, delta=delta, row_idx=batch.logit_rows)
        self.head(x, out=logits)
        if self.spec.logit_scale != 1.0 or self.spec.logit_softcap > 0.0:
            K.scale_softcap(logits, self.spec.logit_scale, self.spec.logit_softcap)
        return logits
