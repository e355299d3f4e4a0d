"""What a mixer tells the cache manager it needs to keep between steps."""
from __future__ import annotations

import dataclasses
from typing import Optional, Tuple


@dataclasses.dataclass(frozen=True)
class PagedKVSpec:
    """Keys and values that grow by one row per token, kept in pages.

    window None: every key stays until the request ends. window w: a query at
    position p reads keys at positions p-w+1..p, and pages that lie wholly before
    that are given back while the request still runs. keep_first n: the keys at positions
    below n stay readable whatever the window; the cache manager then keeps every page of the
    request (the kernels skip what lies between the kept keys and the window).
    value_dim: size of a value row where it differs from a key row's head_dim (None: the same); the
    key pool and the value pool are then two tensors of their own widths.
    chunk c: a query at position p reads keys from floor(p / c) * c on (chunks counted from position 0
    of the request), and pages that lie wholly before the chunk of the next token are given back.
    """
    num_kv_heads: int
    head_dim: int
    window: Optional[int] = None
    keep_first: int = 0
    value_dim: Optional[int] = None
    chunk: Optional[int] = None

    def first_needed(self, next_pos: int) -> Optional[int]:
        """The earliest position that the query at next_pos, or any later one, still reads; None: every
        key stays (no window or chunk, or kept first keys, which hold every page)."""
        if self.keep_first:
            return None
        first = None
        if self.window is not None:
            first = next_pos - self.window + 1
        if self.chunk is not None:
            c = next_pos // self.chunk * self.chunk
            first = c if first is None else max(first, c)
        return first


@dataclasses.dataclass(frozen=True)
class StateSpec:
    """State of fixed size per request: named tensors (name, shape, dtype name), zero at the start.

    The reference's LinearStateCache is of this kind: conv tail [C, K] bf16 and a
    recurrent matrix [Hv, dk, dv] fp32 per session (rollout/cache.py:340-356).
    """
    tensors: Tuple[Tuple[str, Tuple[int, ...], str], ...]
