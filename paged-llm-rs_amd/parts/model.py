"""The generic decoder: embedding, the layers in the order the schedule gives,
final norm on the wanted rows, output projection (reference: model/mod.rs).

The model is put together from a ModelSpec alone.  Which architecture the spec
came from is not known here.
"""

from __future__ import annotations

from pathlib import Path

import torch

from .. import kernels
from ..cache.layout import CacheLayout
from ..config import load_config
from ..errors import ConfigError, UnsupportedError, WeightError
from ..weights.loader import ParamDecl, load_weights
from . import attention, block, mlp, norm  # noqa: F401  (register the built-in parts)
from .linear import Linear, linears_of
from .norm import PendingNorm
from .registry import BLOCKS, EMBED_TRANSFORMS, LOGIT_TRANSFORMS, NORMS, lookup, prefixed, scoped
from .trace import ActivationTrace

DTYPES = {"float32": torch.float32, "f32": torch.float32, "bfloat16": torch.bfloat16, "bf16": torch.bfloat16,
          torch.float32: torch.float32, torch.bfloat16: torch.bfloat16}


def _transforms(spec) -> list:
    """(attribute, class) of the transforms the spec names: of the stream behind the embedding and of the logits."""
    found = []
    for key, registry, what in (("embed_transform", EMBED_TRANSFORMS, "embedding transform"),
                                ("logit_transform", LOGIT_TRANSFORMS, "logit transform")):
        kind = (spec.extra or {}).get(key)
        if kind is not None:
            found.append((key, lookup(registry, kind, what)))
    return found


def declare_parameters(spec) -> list:
    """Every tensor the model needs, by checkpoint name (reference: model/mod.rs:178-227)."""
    decls = [ParamDecl(spec.embed_name, (spec.vocab_size, spec.hidden_size), "embedding")]
    for layer in spec.layers:
        cls = lookup(BLOCKS, layer.block, "block")
        decls += prefixed(cls.declare(layer, spec.hidden_size), layer.weight_prefix)
    final = lookup(NORMS, spec.final_norm.kind, "norm")
    stem = spec.final_norm_name.rsplit(".", 1)[0]
    decls += prefixed(final.declare(spec.final_norm, spec.hidden_size), stem)
    # A tied checkpoint may still store the output projection; the stored tensor wins.
    decls.append(ParamDecl(spec.head_name, (spec.vocab_size, spec.hidden_size), "matrix", optional=True))
    for _, cls in _transforms(spec):
        if hasattr(cls, "declare"):
            decls += list(cls.declare(spec))
    return decls


class LayerContext:
    """What one run of one layer sees of the step: the batch, its own pages (or
    the pages of the layer it reads from) and its state slots."""

    __slots__ = ("batch", "cache", "layer", "cache_layer", "writes_cache", "residual", "trace", "hand", "handed",
                 "norm_after", "handed_out")

    def __init__(self, batch, cache, layer: int, cache_layer: int, writes_cache: bool):
        self.batch = batch
        self.cache = cache
        self.layer = layer
        self.cache_layer = cache_layer
        self.writes_cache = writes_cache
        # the 32-bit stream, while a mixer that adds its own output runs; None otherwise
        self.residual = None
        # an ActivationTrace for the part that runs, when named activations are recorded; None otherwise
        self.trace = None
        # Norms handed forward (``kernels.HandedNorm``; all optional, a part that knows nothing of them loses
        # nothing).  ``hand``: while a mixer that adds its own output runs, room for the norm that follows the
        # stream then.  ``handed``: what the layer before left of this layer's first norm.  ``norm_after``: the
        # norm that the next layer applies to the stream first; a block that can leaves its work in ``handed_out``.
        self.hand = None
        self.handed = None
        self.norm_after = None
        self.handed_out = None

    def kv(self):
        return self.cache.layer_view(self.cache_layer, self.batch)

    def state(self):
        """[slots, ...] state tensor of this layer; ``batch.state_slots`` says which slot each request has."""
        return self.cache.layer_state(self.layer)


class DecoderModel:
    # The embedding takes a row's id from ``batch.fed_tokens[batch.token_src[t]]`` where ``batch.token_src[t]`` names
    # a row of the step before: the runner and the engine may then queue a decoding step before the host has read
    # the tokens of the one before.  (A model class without the attribute, or with False, is stepped the ordinary way.)
    takes_fed_tokens = True

    def __init__(self, spec, params: dict, dtype: torch.dtype, device):
        self.spec = spec
        self.dtype = dtype
        self.device = torch.device(device)
        self.shared: dict = {}
        self.embed_tokens = params[spec.embed_name]
        self.blocks = []
        for layer in spec.layers:
            cls = lookup(BLOCKS, layer.block, "block")
            self.blocks.append(cls(layer, spec.hidden_size, scoped(params, layer.weight_prefix), dtype,
                                   self.device, self.shared))
        stem = spec.final_norm_name.rsplit(".", 1)[0]
        self.norm = lookup(NORMS, spec.final_norm.kind, "norm")(
            spec.final_norm, spec.hidden_size, scoped(params, stem), dtype, self.device)
        if spec.head_name in params:
            head = params[spec.head_name]
        elif spec.tie_word_embeddings:
            head = self.embed_tokens
        else:
            raise WeightError(f"no {spec.head_name}, and the config does not tie the embeddings")
        self.lm_head = Linear(head)
        self.embed_transform = self.logit_transform = None
        for key, cls in _transforms(spec):
            setattr(self, key, cls(spec, params, dtype, self.device))
        for entry in spec.schedule:
            if not 0 <= entry.layer < len(self.blocks):
                raise ConfigError(f"the schedule names layer {entry.layer} of {len(self.blocks)}")
            if entry.cache_from is not None and not 0 <= entry.cache_from < len(self.blocks):
                raise ConfigError(f"the schedule reads the cache of layer {entry.cache_from} of {len(self.blocks)}")
        self.cache_layout = CacheLayout.from_blocks(self.blocks, spec.schedule)
        self.graph_safe = (all(getattr(b, "graph_safe", True) for b in self.blocks)
                           and getattr(self.embed_transform, "graph_safe", True)
                           and getattr(self.logit_transform, "graph_safe", True))
        # Mixers that hand requests of few tokens to a kernel of their own say from how many tokens on a
        # request counts as a long portion; a step reports the tokens of the shorter ones for each such limit.
        self.portion_limits = tuple(sorted({int(limit) for b in self.blocks
                                            for limit in [getattr(getattr(b, "mixer", None), "short_portion", None)]
                                            if limit}))

    def matrix_bytes(self) -> tuple:
        """(bytes of the weight matrices as stored, bytes of their second copies in strips)."""
        stored = strips = 0
        tensors = set()
        for linear in linears_of(self):
            for which, t in (("stored", linear.weight), ("strips", linear.strips)):
                if t is None or t.data_ptr() in tensors:
                    continue
                tensors.add(t.data_ptr())
                if which == "stored":
                    stored += t.numel() * t.element_size()
                else:
                    strips += t.numel() * t.element_size()
        return stored, strips

    # -- the forward pass of one step -------------------------------------------------

    def forward(self, batch, cache, trace: dict | None = None) -> torch.Tensor:
        """Run the tokens of ``batch`` from ``cache`` and return 32-bit logits
        [wanted rows, vocabulary].  Pages are written; no length is moved.

        ``trace``: a dict that receives the output of every module under the module's checkpoint
        name plus ``.out`` (reference: model/mod.rs:34-80), rows in the order of the batch's tokens;
        the final norm, the head and ``logits`` hold the wanted rows only.  32-bit models only."""
        top = None
        if trace is not None:
            if self.dtype != torch.float32:
                raise UnsupportedError("named activations are recorded on the 32-bit path only: in bfloat16 "
                                       "most of them are stages inside kernels and never written")
            top = ActivationTrace(trace)
        fed = getattr(batch, "fed_tokens", None)
        resid = kernels.embed(batch.token_ids, self.embed_tokens,
                              src=batch.token_src if fed is not None else None, fed=fed)
        if self.embed_transform is not None:
            resid = self.embed_transform(resid, batch)
        if top is not None:
            top.record(self.spec.embed_name.rsplit(".", 1)[0] + ".out", resid)
        delta = None
        handed = None
        schedule = self.spec.schedule
        for at, entry in enumerate(schedule):
            own = entry.cache_from is None
            ctx = LayerContext(batch, cache, entry.layer, entry.layer if own else entry.cache_from, own)
            if top is not None:
                ctx.trace = top.child(self.spec.layers[entry.layer].weight_prefix)
            ctx.handed = handed
            if at + 1 < len(schedule):
                ctx.norm_after = getattr(self.blocks[schedule[at + 1].layer], "first_norm", None)
            delta = self.blocks[entry.layer].forward(resid, delta, ctx)
            handed = ctx.handed_out if delta is None else None
            if top is not None:
                after = resid.clone()
                if delta is not None:
                    kernels.residual_add(after, delta)
                ctx.trace.record("out", after)
        m = batch.num_logit_rows
        if m == 0:
            # A portion in the middle of a prompt runs only to fill the cache.
            # Nothing further is launched for it.
            return torch.empty((0, self.spec.vocab_size), dtype=torch.float32, device=self.device)
        if delta is None:
            normed = PendingNorm(self.norm, resid, self.dtype, rows=batch.logit_rows)
        else:
            normed = self.norm.apply(resid, delta, self.dtype, rows=batch.logit_rows)
        if top is not None:
            if isinstance(normed, PendingNorm):
                normed = normed.materialize()
            top.record(self.spec.final_norm_name.rsplit(".", 1)[0] + ".out", normed)
        logits = self.lm_head.forward(normed, out_dtype=torch.float32)
        if self.logit_transform is not None:
            logits = self.logit_transform(logits, batch)
        if top is not None:
            top.record(self.spec.head_name.rsplit(".", 1)[0] + ".out", logits)
            top.record("logits", logits)
        return logits


def build_model(config, params: dict, dtype, device) -> DecoderModel:
    return DecoderModel(config.model_spec(), params, DTYPES[dtype], device)


def load_model(model_dir, dtype="bfloat16", device="cuda:0", strips: bool = True):
    """(typed configuration, model) from a folder with config.json and model.safetensors.
    The model class is chosen by config.json through the architecture registry.
    ``strips``: keep every bfloat16 matrix a second time in the order the product of few rows reads fastest
    (``Linear.keep_strips``): faster decoding for twice the memory of the weights."""
    if dtype not in DTYPES:
        raise ConfigError(f"dtype {dtype!r}, which is neither bfloat16 nor float32")
    model_dir = Path(model_dir)
    config = load_config(model_dir)
    spec = config.model_spec()
    params = load_weights(model_dir, declare_parameters(spec), DTYPES[dtype], device, ignored=spec.ignored_tensors)
    before = Linear.keep_strips
    Linear.keep_strips = bool(strips)
    try:
        return config, DecoderModel(spec, params, DTYPES[dtype], device)
    finally:
        Linear.keep_strips = before
