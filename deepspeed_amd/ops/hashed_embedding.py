"""Hashed pair ("bigram") embedding rows for ragged serving batches.

Beside its own row, a token reads one row of a second table chosen by a hash
of the pair (previous token, token):

    row = (previous * mul_prev + token * mul_cur) mod buckets

A sequence's first token has no previous one and takes row ``buckets`` (the
table holds ``buckets + 1`` rows). The previous token of a step's first token
is carried per request slot, so a sequence can be cut anywhere; ``prev`` is
that state ([slots] int64) and is advanced to each sequence's last token.
The sum of the two rows is ``ops.norms.embed_rows(..., add_table, add_ids)``.
"""

import torch


def _sk():
    from . import serving_kernels
    return serving_kernels


def pair_hash_rows(ids, batch, prev, mul_prev, mul_cur, buckets):
    """ids [T] int64, the flat tokens of ``batch``; prev [slots] int64,
    updated in place. Returns the hashed table's row per token [T] int64."""
    ids = ids.reshape(-1).to(torch.int64)
    if ids.is_cuda and _sk().enabled():
        return _sk().pair_hash_rows(ids, batch, prev, mul_prev, mul_cur,
                                    buckets)
    before = torch.empty_like(ids)
    before[1:] = ids[:-1]
    at = 0
    for slot, count in zip(batch.slots, batch.counts):
        if count:
            before[at] = prev[slot]
            prev[slot] = ids[at + count - 1]
        at += count
    rows = (before * mul_prev + ids * mul_cur) % buckets
    first = batch.tok_pos.to(ids.device) == 0
    return torch.where(first, torch.full_like(rows, buckets), rows)
