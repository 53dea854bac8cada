"""Tokens the host has not seen: how a step names them.

When the next step is queued before the last one's choices have been read back, a decoding
request's input token is known to the device only.  The step function takes a negative id
for it, ``fed_token(r)``: "what sampling row ``r`` of the latest step chose".  The sampling
kernels leave their choices in a buffer of the runner, one row per chosen token, and the
embedding kernel reads row ``r`` of it.  (The reference writes -1 and gathers by slot,
rapid_llm/engine/scheduler.py:241-249; naming the row needs no scatter by slot.)
"""

from __future__ import annotations


def fed_token(row: int) -> int:
    if row < 0:
        raise ValueError(f"a fed token names a sampling row, got {row}")
    return -(row + 1)


def fed_row(token: int) -> int:
    """The sampling row a placeholder names."""
    return -token - 1
