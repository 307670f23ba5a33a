"""Per-step attention metadata, handed from the model runner to ``Attention`` out of band.

The interface is the reference's (``infer/context.py:4-26``: ``get_context`` / ``set_context`` /
``reset_context`` and the eight attribute names ``Attention.forward`` reads).  Here there is ONE
context object for the life of the process and the setters overwrite its fields: a captured HIP graph and
the modules of the model may keep the object they got from ``get_context()`` and still see the current
step's tensors."""
from __future__ import annotations

_FIELDS = (
    # name, value after reset
    ("is_prefill", False),
    ("cu_seqlens_q", None),      # int32 [num_seqs + 1], prefill only
    ("cu_seqlens_k", None),
    ("max_seqlen_q", 0),
    ("max_seqlen_k", 0),
    ("slot_mapping", None),      # int32 [tokens], -1 = padding
    ("context_lens", None),      # int32 [batch], decode only
    ("block_tables", None),      # int32 [batch, max blocks]
)


class Context:
    __slots__ = tuple(name for name, _ in _FIELDS)

    def __init__(self, *values, **named):
        self.assign(*values, **named)

    def assign(self, *values, **named) -> None:
        """Positional values follow the order of ``_FIELDS``; anything not given goes back to its reset value."""
        if len(values) > len(_FIELDS):
            raise TypeError(f"Context takes at most {len(_FIELDS)} values")
        unknown = set(named) - set(self.__slots__)
        if unknown:
            raise TypeError(f"Context has no field {sorted(unknown)[0]!r}")
        for i, (name, default) in enumerate(_FIELDS):
            if i < len(values):
                if name in named:
                    raise TypeError(f"Context field {name!r} given twice")
                setattr(self, name, values[i])
            else:
                setattr(self, name, named.get(name, default))

    def __repr__(self):
        return "Context(" + ", ".join(f"{n}={getattr(self, n)!r}" for n in self.__slots__) + ")"


_current = Context()


def get_context() -> Context:
    return _current


def set_context(is_prefill, cu_seqlens_q=None, cu_seqlens_k=None, max_seqlen_q=0, max_seqlen_k=0,
                slot_mapping=None, context_lens=None, block_tables=None) -> None:
    _current.assign(is_prefill, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k, slot_mapping,
                    context_lens, block_tables)


def reset_context() -> None:
    _current.assign()
