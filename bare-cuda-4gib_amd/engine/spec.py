"""A model as data: which parts make each layer, and in which order layers run.

An architecture's ``describe(config)`` returns a :class:`ModelSpec`; nothing
below it knows which architecture it came from.
"""
from __future__ import annotations

import dataclasses
from typing import Any, Dict, List, Optional, Tuple


@dataclasses.dataclass
class PartSpec:
    """One part: its registered kind, its sizes and constants, and the prefix
    its tensors carry in the weight file (``rename`` maps a part's own tensor
    names to other file names where an architecture calls them differently)."""
    kind: str
    params: Dict[str, Any] = dataclasses.field(default_factory=dict)
    prefix: str = ""
    rename: Dict[str, str] = dataclasses.field(default_factory=dict)


@dataclasses.dataclass
class LayerSpec:
    """One layer: an arrangement (``block``) of a mixer, a feed-forward and
    their norms.  Every layer has its own, so layers of one model may differ.
    A layer may have no feed-forward (``ffn`` and ``ffn_norm`` None), and an
    arrangement that has more parts than these four names them in ``extras``:
    the block's own parameter name -> (category, PartSpec)."""
    block: str
    mixer: PartSpec
    ffn: Optional[PartSpec] = None
    mixer_norm: Optional[PartSpec] = None
    ffn_norm: Optional[PartSpec] = None
    extras: Dict[str, Tuple[str, PartSpec]] = dataclasses.field(default_factory=dict)


@dataclasses.dataclass
class ScheduleEntry:
    """One execution of a layer.  ``cache`` names the cache stream its mixer
    uses (any hashable id; entries that share an id share the cache), and
    ``writes`` says whether this execution appends to that stream or only
    reads what another entry wrote.  ``add_embedding``: the embedding's output is added to the
    residual stream right before this execution (a stack that runs some of its layers several times
    feeds its input in again at the start of every further pass).  ``reenter``: the number of the pass that begins with this
    execution -- right before it the model's ``reentry`` part replaces the stream by a map of the stream and the
    embedding's output (None: nothing happens)."""
    layer: int
    cache: Optional[Any] = None
    writes: bool = True
    add_embedding: bool = False
    reenter: Optional[int] = None


@dataclasses.dataclass
class ModelSpec:
    vocab_size: int
    hidden_size: int
    max_seq_len: int
    embedding: PartSpec
    layers: List[LayerSpec]
    schedule: List[ScheduleEntry]
    final_norm: PartSpec
    head: PartSpec
    # copies of the residual stream that the layers keep side by side, [T, streams, H] (1: the plain stream [T, H]); all
    # start as the embedding's output, and the model's last norm reads their sum
    streams: int = 1
    # what replaces the stream before the schedule entries that say ``reenter`` (a part of category "reentry")
    reentry: Optional[PartSpec] = None
