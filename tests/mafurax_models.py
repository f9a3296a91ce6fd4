"""Small Mafurax configurations for the tests, as ``config.json`` dictionaries. They differ from each
other in every size and constant: heads and groups (also one group per head, one head), key and
value sizes that are no multiples of anything and differ from each other, windows shorter than a
page and none at all, kept first tokens or none, capped and uncapped scores, distance tables of 6 to
12 rows, decay ranks, branch scales, a layer without a feed-forward, a logit scale. ``scale`` is
large on purpose: with unit-norm queries and keys it makes the softmax sharp, so that a key which is
wrongly seen or missed moves the logits far more than rounding does."""

from __future__ import annotations


def left(heads, kv_heads, dim, vdim, scale, softcap, bias_max, window, keep_first, bias_rows):
    return {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale, "softcap": softcap,
            "bias_max": bias_max, "mask": {"size": window, "keep_first": keep_first}, "bias_rows": bias_rows}


def right(heads, dim, vdim, tau, rank):
    return {"heads": heads, "dim": dim, "vdim": vdim, "tau": tau, "rank": rank}


def layer(l, r, left_scale, right_scale, ff=None, limit=1.0):
    return {"type": "parallel", "mixer": {"left": l, "right": r, "left_scale": left_scale, "right_scale": right_scale},
            "mlp": None if ff is None else {"kind": "dense", "ff": ff, "limit": limit}}


def model(vocab, width, layers, eps=1e-5, logit_scale=1.0):
    return {"architecture": "Mafurax", "vocab": vocab, "width": width, "layers": layers, "norm": {"eps": eps},
            "logit_scale": logit_scale}


#: three layers of different geometry; windows of 20 and 7 tokens on pages of 8 or 16, one layer that sees everything
SMALL = model(97, 48, [
    layer(left(4, 2, 24, 16, 0.5, 6.0, 40, 20, 3, 10), right(2, 16, 24, 4.0, 5), 1.3, 0.7, ff=80, limit=1.5),
    layer(left(3, 3, 40, 8, 0.3, 0.0, 9, 0, 0, 6), right(1, 70, 70, 1.5, 3), 0.8, 1.1),
    layer(left(2, 1, 12, 36, 0.9, 4.0, 25, 7, 0, 12), right(3, 8, 10, 9.0, 2), 1.0, 1.0, ff=33, limit=0.6),
], eps=1e-5, logit_scale=1.7)

#: one layer, sizes of one: a single head everywhere, a window of one token beside two kept ones
ONES = model(31, 20, [
    layer(left(1, 1, 5, 3, 1.1, 2.0, 6, 1, 2, 4), right(1, 3, 5, 2.0, 1), 2.0, 0.5, ff=7, limit=3.0),
], eps=1e-3, logit_scale=0.25)

#: eight query heads on two groups (two blocks of four per group and tile), key heads beyond the tile kernel's 128
WIDE = model(64, 64, [
    layer(left(8, 2, 32, 32, 0.4, 8.0, 50, 33, 5, 8), right(2, 32, 96, 6.0, 4), 1.0, 1.0, ff=64, limit=2.0),
    layer(left(2, 2, 136, 20, 0.2, 10.0, 30, 18, 1, 8), right(2, 130, 16, 3.0, 4), 0.9, 1.2),
], eps=1e-6, logit_scale=1.0)
