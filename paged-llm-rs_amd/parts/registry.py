"""Registries of parts.  A spec's ``kind`` names the class that implements it.

A part is built from its own spec and the width of the residual stream, asks
for its tensors by local name, and never learns which model it is in.  New
parts are added by registering a class; no file of the package has to change.

Interfaces
----------
mixer         ``declare(spec, hidden) -> [ParamDecl]`` (local names);
              ``__init__(spec, hidden, params, dtype, device, shared)``;
              ``cache_spec() -> KVCacheSpec | None``; ``state_spec() -> StateSpec | None``;
              ``forward(x[n,hidden], ctx: LayerContext) -> [n,hidden]``.
              Optional ``graph_safe = False`` when its forward cannot be captured as a HIP graph.
feed-forward  ``declare``; ``__init__`` as above; ``forward(x) -> [n,hidden]``.
norm          ``declare(spec, width)``; ``__init__(spec, width, params, dtype, device)``;
              ``apply(resid, delta, out_dtype, rows=None) -> normed`` which adds
              ``delta`` into the 32-bit residual stream and returns the normalised rows.
position      ``__init__(spec, device)`` giving ``dim`` (how many elements of a head are rotated),
              ``cos`` and ``sin`` ([max_positions, dim/2], 32-bit, on the device) and
              ``max_positions``; optionally ``neighbours = True`` when an angle turns the elements
              2 i and 2 i + 1 rather than i and i + dim/2.  The angles are the encoding's own.
block         ``declare(layer_spec, hidden)``; ``__init__(layer_spec, hidden, params, dtype,
              device, shared)``; ``forward(resid, delta, ctx) -> delta`` where the returned
              delta is the output not yet added to the residual stream.
transform     of the stream behind the embedding (``register_embed_transform``) or of the logits
              (``register_logit_transform``), named by ``ModelSpec.extra["embed_transform"]`` /
              ``["logit_transform"]``: optional ``declare(spec) -> [ParamDecl]`` (checkpoint names);
              ``__init__(spec, params, dtype, device)`` (``params``: all tensors by checkpoint name);
              ``__call__(x, batch) -> x``: the 32-bit stream [rows, hidden] (padding rows have
              position -1), or the 32-bit logits [wanted rows, vocabulary]; it may work in place.
"""

from __future__ import annotations

from ..errors import UnsupportedError

MIXERS: dict = {}
FEED_FORWARDS: dict = {}
NORMS: dict = {}
BLOCKS: dict = {}
POSITIONS: dict = {}
EMBED_TRANSFORMS: dict = {}
LOGIT_TRANSFORMS: dict = {}


def register_mixer(kind: str, cls) -> None:
    MIXERS[kind] = cls


def register_feed_forward(kind: str, cls) -> None:
    FEED_FORWARDS[kind] = cls


def register_norm(kind: str, cls) -> None:
    NORMS[kind] = cls


def register_block(kind: str, cls) -> None:
    BLOCKS[kind] = cls


def register_position(kind: str, cls) -> None:
    POSITIONS[kind] = cls


def register_embed_transform(kind: str, cls) -> None:
    EMBED_TRANSFORMS[kind] = cls


def register_logit_transform(kind: str, cls) -> None:
    LOGIT_TRANSFORMS[kind] = cls


def lookup(registry: dict, kind: str, what: str):
    if kind not in registry:
        raise UnsupportedError(f"{what} {kind!r}, the registry knows {', '.join(sorted(registry)) or 'none'}")
    return registry[kind]


def scoped(params: dict, prefix: str) -> dict:
    """The tensors under ``prefix.``, by their local names."""
    cut = len(prefix) + 1
    return {k[cut:]: v for k, v in params.items() if k.startswith(prefix + ".")}


def prefixed(decls, prefix: str) -> list:
    from ..weights.loader import ParamDecl

    return [ParamDecl(f"{prefix}.{d.name}", d.shape, d.role, d.optional) for d in decls]
