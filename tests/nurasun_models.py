"""Small Nurasun configurations for the tests, as ``config.json`` dictionaries. They differ from each other in every
size and constant: heads and groups (one group per head, one group for all, one head), heads whose size is no
multiple of anything, rotation of part of a head, of all of it and none, runs of positions shorter than a page and
none at all, compressed rows of 2 to 136 elements (beyond what the tile kernel holds), key and value sizes that
differ, a layer that reads another's rows, mixtures of 1 to 70 experts with and without a shared one, a layer
without a feed-forward, with and without squashed logits. ``scale`` is large on purpose: it makes the softmax sharp,
so that a key which is wrongly seen or missed moves the logits far more than rounding does."""

from __future__ import annotations


def attention(heads, kv_heads, dim, scale, chunk=0, rot=None, base=10000.0):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "scale": scale}
    if chunk:
        m["mask"] = {"size": chunk}
    if rot:
        m["rot"] = {"dims": rot, "base": base}
    return "attention", m


def latent(heads, dim, vdim, rank, scale, kv_from=None):
    m = {"heads": heads, "dim": dim, "vdim": vdim, "kv_rank": rank, "scale": scale}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return "latent_attention", m


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(experts, top, ff, shared=0):
    m = {"kind": "moe", "router": {"experts": experts, "top": top}, "expert": {"ff": ff}}
    if shared:
        m["shared"] = {"ff": shared}
    return m


def layer(mixer, mlp=None):
    return {"type": mixer[0], "mixer": mixer[1], "mlp": mlp}


def model(vocab, width, layers, eps=1e-5, mult=1.0, softcap=0.0):
    return {"architecture": "Nurasun", "vocab": vocab, "width": width, "layers": layers, "norm": {"eps": eps},
            "residual_mult": mult, "logit_softcap": softcap}


#: five layers of different geometry; runs of 20 and 7 positions on pages of 4 to 16, a layer reading another's rows
SMALL = model(113, 40, [
    layer(attention(4, 2, 24, 0.6, chunk=20, rot=16, base=500.0), dense(56)),
    layer(latent(3, 16, 24, 40, 0.9), moe(5, 2, 24, shared=16)),
    layer(latent(2, 8, 8, 40, 1.5, kv_from=1)),
    layer(attention(2, 2, 10, 0.8, chunk=7, rot=10), moe(4, 4, 12)),
    layer(latent(1, 5, 3, 12, 2.0), dense(33)),
], eps=1e-5, mult=0.45, softcap=9.0)

#: sizes of one: a single head everywhere, a run of one position, one expert, a compressed row of two elements
ONES = model(31, 20, [
    layer(attention(1, 1, 6, 1.1, chunk=1, rot=2, base=7.0), moe(1, 1, 3)),
    layer(latent(1, 1, 1, 2, 1.3), dense(1)),
], eps=1e-3, mult=1.7, softcap=2.5)

#: plain causal attention without rotation, eight heads on eight groups; a compressed row beyond the tile kernel's 128
#: elements; more experts than a wave has lanes
WIDE = model(64, 64, [
    layer(attention(8, 8, 32, 0.5), moe(70, 6, 8, shared=24)),
    layer(latent(4, 32, 16, 136, 0.4), dense(96)),
    layer(attention(6, 1, 16, 0.7, chunk=33, rot=8, base=90.0), dense(40)),
], eps=1e-6, mult=1.0, softcap=0.0)

#: sizes that are multiples of nothing, so that no kernel's form for whole 16-byte pieces takes them
ODD = model(77, 50, [
    layer(attention(3, 1, 10, 0.9, chunk=11, rot=6, base=40.0), moe(3, 2, 5, shared=3)),
    layer(latent(3, 5, 7, 9, 1.4), dense(9)),
    layer(latent(2, 3, 3, 9, 0.8, kv_from=1), moe(6, 1, 7)),
], eps=1e-4, mult=0.6, softcap=4.0)
