"""How a step's rows belong to requests, on the device, for parts that keep state of fixed size per request
(``ops.RowsOfRequests``). Built once per step from what the step function has laid out and shared by every such
part of every layer."""
from __future__ import annotations

from .. import ops


def rows_of_requests(ctx) -> ops.RowsOfRequests:
    return ctx.memo("rows of requests", lambda: _build(ctx))


def _build(ctx) -> ops.RowsOfRequests:
    n, n_slots = len(ctx.spans), ctx.fn.cache.max_requests
    if ctx.max_q_len == 1:      # every request brings one row: request r owns row r
        return ops.RowsOfRequests(ctx.request_slots, None, None, n, ctx.tokens, n_slots)
    return ops.RowsOfRequests(ctx.request_slots, ctx.row_offsets, ctx.req_of_token, n, ctx.tokens, n_slots)
