"""The Zaluvik design on the GPU against the plain oracle of tests/zaluvik_oracle.py: every mechanism on a configuration of its own, prompts against
token-by-token decoding, portions down to two tokens, mixed batches, slots and pages that are used again, keys just inside and just outside every window
(in prompts and in decoding, in both kinds of attention, in every pass of the loop), far keys, page borders, the first tokens of a sequence, long
decoding, and greedy generation through the slot scheduler, tgx_forward / tgx_sample / tgx_decode, the C++ engine, the command line and bin/trace_run.
Models are config dictionaries of the checkpoint format, so the configuration reader is on the path of every test.  fp32 storage is the sharp
comparison (nothing is rounded: 1e-4 of the largest logit); bf16 storage rounds the cached rows (3e-2)."""
import copy
import json
import os
import subprocess
import sys

import numpy as np
import pytest

import zaluvik_oracle as zo
from test_hip_modepel import write_model_dir
from tinygpt_amd.desc import stack_desc_from_config
from tinygpt_amd.ffi import GREEDY, Model, TgxError
from tinygpt_amd.serving import SlotEngine

pytestmark = pytest.mark.gpu
TOL = {"fp32": 1e-4, "bf16": 3e-2}


# ---- configurations ---------------------------------------------------------------------------------------------------------------
def dense(n=20):
    return {"kind": "dense", "ff": n}


def moe(experts=6, top=2, ff=10, groups=(3, 2), shared=7):
    r = {"experts": experts, "top": top}
    if groups:
        r["groups"] = {"count": groups[0], "keep": groups[1]}
    f = {"kind": "moe", "expert": {"ff": ff}, "router": r}
    if shared:
        f["shared"] = {"ff": shared}
    return f


def attn(mlp=None, **kw):
    m = dict(heads=4, kv_heads=2, dim=8, vdim=6, mask={"size": 11}, scale=0.9)
    m.update(kw)
    return {"type": "attention", "mixer": {k: v for k, v in m.items() if v is not None}, "mlp": mlp}


def lat(mlp=None, **kw):
    m = dict(heads=3, dim=6, rot_dim=4, vdim=5, kv_rank=10, mask={"size": 13}, scale=0.6)
    m.update(kw)
    if m.get("rot_dim"):
        m.setdefault("rot", {"base": 300.0, "dims": m["rot_dim"]})
    else:
        m.pop("rot", None); m.pop("rot_dim", None)
    return {"type": "latent_attention", "mixer": {k: v for k, v in m.items() if v is not None}, "mlp": mlp}


def config(layers=None, width=24, vocab=67, eps=1e-5, mult=0.6, scale=2.5, loop=(1, 3, 2)):
    cfg = {"architecture": "Zaluvik", "width": width, "vocab": vocab, "norm": {"eps": eps}, "residual_mult": mult, "embedding": {"scale": scale},
           "layers": copy.deepcopy(layers) if layers is not None else [attn(dense()), lat(moe()), attn(moe(groups=None, shared=0)), lat(dense(9)), attn()]}
    if loop and loop[1] <= len(cfg["layers"]):
        cfg["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    return cfg


def engine(cfg, dtype="fp32", seed=0, overrides=None, **kw):
    w = zo.random_tensors(cfg, seed, overrides)
    kw = dict(dict(max_seqs=4, max_ctx=1024, budget_tokens=2048), **kw)
    eng = SlotEngine(desc=stack_desc_from_config(cfg, dtype, **kw), tensors={k: np.asarray(v, np.float32) for k, v in w.items()})
    return eng, w


def tokens(cfg, n, seed=0):
    return np.random.default_rng(100 + seed).integers(0, cfg["vocab"], n).tolist()


def want_of(cfg, w, toks):
    return zo.forward(cfg, w, toks)


def check(got, want, dtype, what=""):
    err = np.abs(got - want).max() / np.abs(want).max()
    assert err < TOL[dtype], f"{what}: {err:.3e}"


def run_whole(eng, rid, toks):
    return eng.step([(rid, toks, list(range(len(toks))))], [rid])


# ---- every mechanism on a configuration of its own --------------------------------------------------------------------------------------
MECH = {
    "sigmoid_attention_alone": ([attn()], None),
    "window_of_one": ([attn(mask={"size": 1})], None),                               # a token sees itself only
    "window_longer_than_the_sequence": ([attn(mask={"size": 500})], None),
    "no_mask": ([attn(mask=None), lat(mask=None)], None),
    "one_key_head_per_query_head": ([attn(kv_heads=4)], None),
    "one_key_head_for_all": ([attn(heads=6, kv_heads=1)], None),
    "one_head": ([attn(heads=1, kv_heads=1)], None),                                 # the mixing matrix is one number
    "wide_heads": ([attn(heads=2, kv_heads=1, dim=80, vdim=72, scale=0.3)], None),
    "many_heads": ([attn(heads=12, kv_heads=4, dim=16, vdim=24)], None),             # more than 256 output channels: several per thread
    "latent_alone": ([lat()], None),
    "latent_without_rotated_part": ([lat(rot_dim=0)], None),
    "latent_two_of_the_rotated_channels_turn": ([lat(rot_dim=6, rot={"base": 50.0, "dims": 2})], None),
    "latent_wide": ([lat(heads=2, dim=20, rot_dim=8, vdim=33, kv_rank=70, rot={"base": 10000.0, "dims": 8})], None),
    "latent_one_head": ([lat(heads=1)], None),
    "latent_window_of_one": ([lat(mask={"size": 1})], None),
    "dense_only": ([attn(dense(33)), lat(dense(5))], None),
    "experts_top_one": ([attn(moe(top=1))], None),
    "experts_all_chosen": ([attn(moe(experts=4, top=4, groups=None))], None),
    "experts_one_group_kept": ([lat(moe(experts=8, top=3, groups=(2, 1)))], None),
    "experts_groups_of_one": ([attn(moe(experts=5, top=2, groups=(5, 3)))], None),   # a group's score is its only member's
    "experts_every_group_kept": ([attn(moe(experts=6, top=3, groups=(2, 2)))], None),
    "experts_no_shared": ([lat(moe(shared=0))], None),
    "experts_many": ([attn(moe(experts=72, top=5, groups=(8, 3), ff=4))], None),
    "no_feed_forward_anywhere": ([attn(), lat(), attn()], (0, 2, 3)),
    "no_loop": ([attn(dense()), lat(moe())], None),
    "loop_of_one_pass": ([attn(dense()), lat(moe()), attn()], (1, 2, 1)),            # the input product still comes first
    "loop_from_the_first_layer": ([lat(dense()), attn(moe())], (0, 1, 3)),
    "loop_over_everything": ([attn(dense()), lat()], (0, 2, 4)),
    "loop_to_the_last_layer": ([attn(), lat(dense()), attn(moe())], (1, 3, 2)),
    "wide_stream": ([attn(dense(8)), lat()], (1, 2, 2)),                               # a width beyond what the seam keeps in registers
    "ragged_sizes": ([attn(dense(19), heads=6, kv_heads=3, dim=5, vdim=7), lat(moe(experts=9, top=4, groups=(3, 2), ff=11, shared=3), heads=5, dim=7, rot_dim=6, vdim=3, kv_rank=13)], (0, 2, 2)),
    "deep": ([attn(dense()), lat(moe()), attn(moe(groups=None, shared=0)), lat(dense(9)), attn(), lat(), attn(dense())], (2, 6, 3)),
}
EXTRA = {"ragged_sizes": dict(width=27, vocab=53), "wide_heads": dict(width=40), "deep": dict(mult=1.0, scale=1.0), "many_heads": dict(width=40), "wide_stream": dict(width=4104)}
SEEDS = {"deep": 5}      # (with the default seed two router scores of one token lie closer than bf16 rounding: the choice, a discrete one, flips)


@pytest.mark.parametrize("dtype", ["fp32", "bf16"])
@pytest.mark.parametrize("name", list(MECH))
def test_mechanism(name, dtype):
    layers, loop = MECH[name]
    cfg = config(layers, loop=loop, **EXTRA.get(name, {}))
    eng, w = engine(cfg, dtype, seed=SEEDS.get(name, len(name)))
    toks = tokens(cfg, 23, seed=len(name))
    want = want_of(cfg, w, toks)
    check(run_whole(eng, "a", toks), want, dtype, name)
    # ... and the same tokens one by one through every run's cache
    got = np.concatenate([eng.step([("b", [t], [0])]) for t in toks])
    check(got, want, dtype, name + " by steps")
    eng.close()


# ---- prompts, decoding, portions --------------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", ["fp32", "bf16"])
def test_prompt_then_token_by_token(dtype):
    cfg = config()
    eng, w = engine(cfg, dtype, 1)
    toks = tokens(cfg, 40)
    want = want_of(cfg, w, toks)
    got = [eng.step([("r", toks[:9], list(range(9)))])]
    for i in range(9, 40):
        got.append(eng.step([("r", [toks[i]], [0])]))
    check(np.concatenate(got), want, dtype)
    eng.release("r")
    got = np.concatenate([eng.step([("s", [toks[i]], [0])]) for i in range(6)])      # the first tokens of a sequence in a slot that held another one
    check(got, want[:6], dtype, "from the first token")
    eng.close()


@pytest.mark.parametrize("dtype", ["fp32", "bf16"])
@pytest.mark.parametrize("sizes", [[2] * 20, [3, 2, 5, 2, 7, 1, 11, 2, 2], [64, 2, 63, 1], [1, 128, 2, 65], [5, 59, 64, 2], [1, 1, 1, 2, 1, 3, 17]])
def test_portions(sizes, dtype):
    """portions cut through windows and pages"""
    cfg = config()
    eng, w = engine(cfg, dtype, 2)
    toks = tokens(cfg, sum(sizes), seed=len(sizes))
    want = want_of(cfg, w, toks)
    got, at = [], 0
    for n in sizes:
        got.append(eng.step([("r", toks[at:at + n], list(range(n)))]))
        at += n
    check(np.concatenate(got), want, dtype)
    eng.close()


@pytest.mark.parametrize("n", [1, 63, 64, 65, 127, 128, 129, 200])
def test_contexts_around_page_borders(n):
    cfg = config([attn(mask={"size": 70}, scale=2.0), lat(dense(), mask={"size": 128}), attn(moe(), mask={"size": 129})], loop=(1, 3, 2))
    eng, w = engine(cfg, "fp32", 4)
    toks = tokens(cfg, n + 3, seed=n)
    want = want_of(cfg, w, toks)
    got = [eng.step([("r", toks[:n], [n - 1])])]
    got += [eng.step([("r", [toks[n + i]], [0])]) for i in range(3)]      # decoding across the border
    check(np.concatenate(got), want[n - 1:], "fp32")
    eng.close()


# ---- keys that stand out: a window's edge that is one token off shows as a large error -----------------------------------------------------
def loud(cfg, seed, q_name, k_name, q_rows, k_row):
    """weights in which token id 7 carries a key that every query asks for: its embedding row is one loud coordinate (0) that no other token has, the key
    projection turns that coordinate into a large key channel, and a coordinate that every token shares (1) drives every query towards that channel.
    The first norm passes its input on unchanged in scale (weight one, bias zero)."""
    w0 = zo.random_tensors(cfg, seed)
    emb = w0["embed"].copy()
    emb[:, 0] = 0.0; emb[:, 1] = 2.0; emb[7] = 0.0; emb[7, 0] = 6.0; emb[7, 1] = 2.0
    k = w0[k_name].copy(); k[:, 0] = 0.0; k[:, 1] = 0.0; k[k_row] = 0.0; k[k_row, 0] = 8.0      # no other token has anything in that key channel
    q = w0[q_name].copy(); q[:, 0] = 0.0; q[:, 1] = 0.0
    for r in q_rows:
        q[r] = 0.0; q[r, 1] = 3.0
    return {"embed": emb, k_name: k, q_name: q, "l0.norm1": np.ones_like(w0["l0.norm1"]), "l0.norm1.b": np.zeros_like(w0["l0.norm1.b"])}


def edge_case(cfg, over, seed, size, at, dtype):
    """the loud key sits at position `at`: the queries up to at + size - 1 see it, the query at at + size is the first that does not.  The prompt ends
    before, at and behind the edge and the rest is decoded."""
    n = at + size + 6
    toks = [t if t != 7 else 8 for t in tokens(cfg, n, seed=size)]
    toks[at] = 7
    edge = at + size
    for cut in (n, edge - 1, edge, edge + 1, max(at + 1, edge - 3)):
        eng, w = engine(cfg, dtype, seed, over)
        want = want_of(cfg, w, toks)
        if cut == n:
            without = list(toks); without[at] = 9
            other = want_of(cfg, w, without)
            assert np.abs(other[edge - 1] - want[edge - 1]).max() / np.abs(want).max() > 0.03      # inside: the key decides the logits
            assert np.abs(other[edge:] - want[edge:]).max() == 0.0                                 # outside: it is gone
        places = sorted({p for p in (at, edge - 2, edge - 1, edge, edge + 1, n - 1) if at <= p < n})
        got = [eng.step([("r", toks[:cut], [p for p in places if p < cut])])]
        got += [eng.step([("r", [toks[i]], [0] if i in places else [])]) for i in range(cut, n)]
        check(np.concatenate([g for g in got if len(g)]), want[places], dtype, f"prompt of {cut}")
        eng.close()


@pytest.mark.parametrize("dtype", ["fp32", "bf16"])
@pytest.mark.parametrize("size,at", [(5, 3), (64, 0), (64, 10), (65, 63), (100, 130), (256, 1), (300, 2)])
def test_sigmoid_attention_window_edges(size, at, dtype):
    cfg = config([attn(heads=2, kv_heads=1, dim=8, vdim=8, mask={"size": size}, scale=10.0)], width=16, mult=1.0, scale=1.0, loop=None)
    over = loud(cfg, 6, "l0.mix.q", "l0.mix.k", (5, 13), 5)
    over["l0.mix.pb"] = np.full(2, -60.0)                  # an ordinary key weighs next to nothing, the loud one nearly one
    over["l0.mix.talk"] = np.array([[1.0, 0.5], [-0.25, 1.0]])
    edge_case(cfg, over, 6, size, at, dtype)


@pytest.mark.parametrize("dtype", ["fp32", "bf16"])
@pytest.mark.parametrize("size,at", [(5, 3), (64, 0), (64, 10), (65, 63), (100, 130), (256, 1)])
def test_latent_attention_window_edges(size, at, dtype):
    """the loud key lives in the rotated part that all heads share; with two rotated channels and a huge base the rotation nearly leaves it alone"""
    cfg = config([lat(heads=2, dim=6, rot_dim=8, vdim=8, kv_rank=8, mask={"size": size}, rot={"base": 1e9, "dims": 2}, scale=1.0)], width=16, mult=1.0, scale=1.0, loop=None)
    # q rows: head h's rotated part starts at h * (6 + 8) + 6; channel 5 of it (not turned) asks for channel 5 of the shared key part (dkv row 8 + 5)
    over = loud(cfg, 7, "l0.mix.q", "l0.mix.dkv", (6 + 5, 14 + 6 + 5), 8 + 5)
    edge_case(cfg, over, 7, size, at, dtype)


def test_window_edges_in_every_pass_of_the_loop():
    """the looped layer's caches are per pass: a window that is one off in any pass shows"""
    cfg = config([attn(heads=2, kv_heads=1, dim=8, vdim=8, mask={"size": 9}, scale=6.0), lat(mask={"size": 5})], width=16, mult=1.0, scale=1.0, loop=(0, 2, 3))
    eng, w = engine(cfg, "fp32", 3)
    toks = tokens(cfg, 40)
    want = want_of(cfg, w, toks)
    got = [eng.step([("r", toks[:7], list(range(7)))]), eng.step([("r", toks[7:19], list(range(12)))])]
    got += [eng.step([("r", [t], [0])]) for t in toks[19:]]
    check(np.concatenate(got), want, "fp32")
    eng.close()


def test_one_far_key_stands_out():
    """the loud key occurs once, at position 3 of 400, under a window that still holds it: every later query must find it among hundreds of keys, across
    page borders, in portions and in decoded tokens"""
    cfg = config([attn(heads=2, kv_heads=1, dim=8, vdim=8, mask={"size": 450}, scale=10.0)], width=16, mult=1.0, scale=1.0, loop=None)
    over = loud(cfg, 8, "l0.mix.q", "l0.mix.k", (5, 13), 5)
    over["l0.mix.pb"] = np.full(2, -60.0)
    eng, w = engine(cfg, "fp32", 8, over)
    toks = [t if t != 7 else 8 for t in tokens(cfg, 400)]
    toks[3] = 7
    want = want_of(cfg, w, toks)
    without = list(toks); without[3] = 9
    assert np.abs(want_of(cfg, w, without)[390:] - want[390:]).max() / np.abs(want).max() > 5e-3      # one key among 400 unnormalised ones, behind a layer norm: fifty times the tolerance
    got = [eng.step([("r", toks[:200], [2, 3, 4, 199])]), eng.step([("r", toks[200:390], [0, 189])])]
    got += [eng.step([("r", [toks[390 + i]], [0])]) for i in range(10)]
    check(np.concatenate(got), want[[2, 3, 4, 199, 200, 389] + list(range(390, 400))], "fp32")
    eng.close()


def test_split_keys_form_equals_the_direct_form():
    cfg = config([attn(mask={"size": 300}, scale=2.0), lat(dense(), mask={"size": 256}), attn(mask=None)], loop=(1, 2, 2))
    eng, w = engine(cfg, "fp32", 6)
    toks = tokens(cfg, 700)
    want = want_of(cfg, w, toks)
    eng.step([("r", toks[:690], [])])
    eng.model.set_option("attn.split_min", 64)            # steps of few tokens now divide the keys between workgroups
    got = np.concatenate([eng.step([("r", [toks[690 + i]], [0])]) for i in range(10)])
    check(got, want[690:], "fp32")
    eng.close()


# ---- other sizes: random layer lists, head counts, windows, loops and constants -------------------------------------------------------------------
def random_config(rng):
    layers = []
    for _ in range(int(rng.integers(2, 6))):
        if rng.random() < 0.6:
            heads = int(rng.choice([2, 4, 6, 8, 12])); kv = int(rng.choice([g for g in (1, 2, 3, 4, 6) if heads % g == 0]))
            dim = int(rng.choice([8, 16, 24, 32, 64]))
            layer = attn(heads=heads, kv_heads=kv, dim=dim, vdim=int(rng.choice([8, 16, 32, 40])), mask={"size": int(rng.integers(1, 90))}, scale=float(rng.uniform(2.0, 12.0)) / dim ** 0.5)
        else:
            dim, rd = int(rng.choice([8, 16, 32])), int(rng.choice([0, 4, 8, 16]))
            layer = lat(heads=int(rng.choice([1, 2, 3, 4, 8])), dim=dim, rot_dim=rd, vdim=int(rng.choice([8, 16, 24])), kv_rank=int(rng.choice([12, 32, 48, 112])),
                        mask={"size": int(rng.integers(1, 90))}, scale=float((dim + rd) ** -0.5), rot={"base": float(rng.choice([100.0, 10000.0, 500000.0])), "dims": rd} if rd else None)
        r = rng.random()
        if r < 0.35:
            layer["mlp"] = dense(int(rng.choice([12, 40, 100])))
        elif r < 0.8:
            experts = int(rng.choice([4, 6, 8, 12])); count = int(rng.choice([g for g in (1, 2, 3, 4) if experts % g == 0])); keep = int(rng.integers(1, count + 1))
            layer["mlp"] = moe(experts=experts, top=int(rng.integers(1, min(4, keep * (experts // count)) + 1)), ff=int(rng.choice([6, 16, 24])), groups=(count, keep) if count > 1 else None,
                               shared=int(rng.choice([0, 5, 16])))
        layers.append(layer)
    loop = None
    if rng.random() < 0.8:
        a = int(rng.integers(0, len(layers))); loop = (a, int(rng.integers(a + 1, len(layers) + 1)), int(rng.integers(1, 4)))
    return config(layers, width=int(rng.choice([24, 40, 64, 72])), vocab=int(rng.choice([53, 131, 300])), eps=float(rng.choice([1e-5, 1e-6])), mult=float(rng.choice([0.3, 0.5, 1.0])),
                  scale=float(rng.choice([1.0, 3.0, 8.0])), loop=loop)


@pytest.mark.parametrize("seed", range(10))
def test_random_configurations(seed):
    """whole prompts and portions of 1 .. 64 tokens against the oracle in fp32 (a router choice is discrete: with 16-bit storage a near tie may fall the other way)"""
    rng = np.random.default_rng(1000 + seed)
    cfg = random_config(rng)
    eng, w = engine(cfg, "fp32", seed)
    n = int(rng.integers(100, 200))
    toks = tokens(cfg, n, seed)
    want = want_of(cfg, w, toks)
    check(run_whole(eng, "a", toks), want, "fp32", "whole")
    got, at = [], 0
    while at < n:
        c = min(int(rng.choice([1, 2, 3, 17, 64])), n - at)
        got.append(eng.step([("b", toks[at:at + c], list(range(c)))])); at += c
    check(np.concatenate(got), want, "fp32", "portions")
    eng.close()


# ---- batches, slots, pages ----------------------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", ["fp32", "bf16"])
def test_unequal_requests_in_one_batch(dtype):
    cfg = config()
    eng, w = engine(cfg, dtype, 7)
    seqs = {"a": tokens(cfg, 70, 1), "b": tokens(cfg, 9, 2), "c": tokens(cfg, 33, 3), "d": tokens(cfg, 1, 4)}
    want = {k: want_of(cfg, w, v) for k, v in seqs.items()}
    cuts = {"a": [17, 2, 30, 1, 1, 19], "b": [1, 1, 1, 2, 4, 0], "c": [2, 0, 2, 29, 0, 0], "d": [0, 0, 1, 0, 0, 0]}      # 0: the request sits the step out
    got = {k: [] for k in seqs}
    at = {k: 0 for k in seqs}
    for step in range(6):
        entries = []
        for k in seqs:
            n = cuts[k][step]
            if n:
                entries.append((k, seqs[k][at[k]:at[k] + n], list(range(n))))
        out = eng.step(entries)
        o = 0
        for k, tk, _ in entries:
            got[k].append(out[o:o + len(tk)]); o += len(tk); at[k] += len(tk)
    for k in seqs:
        g = np.concatenate(got[k])
        check(g, want[k][:len(g)], dtype, k)
        assert len(g) == min(len(seqs[k]), sum(cuts[k]))
    eng.close()


def test_slots_and_pages_are_used_again():
    """a slot's next request reads nothing the request before left in the pages, in any pass of the loop"""
    cfg = config()
    eng, w = engine(cfg, "fp32", 8, budget_tokens=256, max_ctx=256, max_seqs=2)      # four pages of 64 tokens, two slots
    assert eng.free_tokens == 256
    for rnd in range(5):
        a, b = tokens(cfg, 100 + rnd, 10 + rnd), tokens(cfg, 60 + rnd, 20 + rnd)
        out = eng.step([(("a", rnd), a, [0, 1, 2, len(a) - 1]), (("b", rnd), b[:-1], [])])
        assert eng.free_tokens == 256 - 128 - 64
        with pytest.raises(RuntimeError):      # both slots are taken
            eng.step([(("c", rnd), [1], [])])
        out2 = eng.step([(("b", rnd), b[-1:], [0])], end=[("a", rnd)])
        wa = want_of(cfg, w, a)
        check(np.concatenate([out, out2]), np.stack([wa[0], wa[1], wa[2], wa[-1], want_of(cfg, w, b)[-1]]), "fp32", f"round {rnd}")
        eng.release(("b", rnd))
        assert eng.free_tokens == 256
    eng.step([("big", tokens(cfg, 200), [])])          # the pool refuses what it cannot hold and leaves the slots as they were
    with pytest.raises(TgxError):
        eng.step([("more", tokens(cfg, 100), [])])
    assert eng.length("big") == 200 and eng.length("more") == 0
    eng.close()


def test_a_request_is_the_same_alone_and_beside_others():
    """nothing a token computes reads another entry of the batch; what differs is the summation order of the products (few rows stream the weights,
    many take the matrix-core tiles)"""
    cfg = config()
    eng, w = engine(cfg, "fp32", 9)
    a, b, c = tokens(cfg, 50, 1), tokens(cfg, 20, 2), tokens(cfg, 3, 3)
    alone = np.concatenate([eng.step([("a", a[:31], [30])]), eng.step([("a", a[31:], [18])], ["a"])])
    eng.step([("c", c, [])])
    mixed = np.concatenate([eng.step([("b", b[:7], []), ("a", a[:31], [30])]), eng.step([("a", a[31:], [18]), ("c", [5], []), ("b", b[7:], [])], ["a", "b", "c"])])
    assert np.abs(alone - mixed).max() / np.abs(alone).max() < 1e-5
    eng.close()


# ---- generation ---------------------------------------------------------------------------------------------------------------------------
def oracle_greedy(cfg, w, prompt, n):
    seq = list(prompt)
    for _ in range(n):
        seq.append(int(np.argmax(want_of(cfg, w, seq)[-1])))
    return seq[len(prompt):]


def test_greedy_generation_through_the_slot_scheduler():
    cfg = config()
    eng, w = engine(cfg, "fp32", 9, max_seqs=2)
    prompts = [tokens(cfg, 11, 1), tokens(cfg, 5, 2), tokens(cfg, 23, 3)]      # three requests on two slots
    want = [oracle_greedy(cfg, w, p, 6) for p in prompts]
    assert eng.generate(prompts, 6) == want
    assert eng.generate(prompts, 6, portion=4) == want
    eng.close()


def test_long_decoding_through_forward_sample_decode():
    cfg = config([attn(dense(), mask={"size": 40}), lat(moe(), mask={"size": 90}), attn(mask={"size": 70})], loop=(1, 3, 2))
    w = zo.random_tensors(cfg, 10)
    m = Model(stack_desc_from_config(cfg, "fp32", max_seqs=2, max_ctx=512)).load_state({k: np.asarray(v, np.float32) for k, v in w.items()}, strict=True).finalize()
    prompts = np.array([tokens(cfg, 7, 1), tokens(cfg, 7, 2)])
    m.forward(prompts)
    first = m.sample(GREEDY)
    rest = np.concatenate([m.decode(75, GREEDY), m.decode(75, GREEDY)])      # crosses two page borders and every window; positions advance on the device
    for b in range(2):
        got = [int(first[b])] + rest[:, b].tolist()
        seq = prompts[b].tolist() + got
        lg = want_of(cfg, w, seq[:-1])
        top2 = np.sort(lg[6:], -1)[:, -2:]
        clear = (top2[:, 1] - top2[:, 0]) > 1e-3 * np.abs(lg).max()
        assert (np.argmax(lg[6:], -1)[clear] == np.array(got)[clear]).all()
        assert clear.mean() > 0.9
    assert m.past_length == 7 + 150
    m.close()


# ---- the C++ host engine, the command line, the trace replay ---------------------------------------------------------------------------------
def test_host_engine_and_cli_generate_greedy(tmp_path):
    from host_util import HostEngine, host_lib
    from tinygpt_amd import build
    cfg = config([attn(dense()), lat(moe()), attn(moe(groups=None)), lat()], loop=(1, 3, 2))
    w = zo.random_tensors(cfg, 11)
    write_model_dir(str(tmp_path), cfg, w)
    prompts = [tokens(cfg, 9, 1), tokens(cfg, 4, 2), tokens(cfg, 13, 3)]           # unequal lengths: no padding is fed
    want = [oracle_greedy(cfg, w, p, 5) for p in prompts]
    e = HostEngine(host_lib(), model_dir=str(tmp_path), device="mi355x", dtype=0, max_batch=4)
    assert e.prepare(), e.error()
    e.reconfigure(max_new=5)
    ids, new, fin = e.generate_sync(prompts)
    assert new == 5 and [ids[b, -5:].tolist() for b in range(3)] == want
    e.reconfigure(max_new=5)
    ids2, new2, fin2, seen = e.generate_async(prompts[2])
    assert ids2[-5:].tolist() == want[2]
    e.close()
    build.build_host()
    arg = ";".join(",".join(str(x) for x in p) for p in prompts)
    r = subprocess.run([build.HOST_CLI, "--model", str(tmp_path), "--dtype", "fp32", "--max-tokens", "5", "--temperature", "0", "--top-p", "1", "--prompt-ids", arg,
                        "--context", "256"], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stderr
    outs = [[int(x) for x in line.split(":")[1].split()] for line in r.stdout.splitlines() if line.startswith("Output ids")]
    assert outs == want


def test_trace_replay_script(tmp_path):
    cfg = config([attn(dense()), lat(moe()), attn()], loop=(0, 2, 2))
    w = zo.random_tensors(cfg, 12)
    mdir, out = tmp_path / "m", tmp_path / "o"
    mdir.mkdir()
    write_model_dir(str(mdir), cfg, w)
    a, b = tokens(cfg, 30, 1), tokens(cfg, 12, 2)
    steps = [{"step": 0, "entries": [{"id": "x", "tokens": a[:20], "want": [0, 19]}], "end": []},
             {"step": 1, "entries": [{"id": "y", "tokens": b[:11], "want": []}, {"id": "x", "tokens": a[20:22], "want": [1]}], "end": []},
             {"step": 2, "entries": [{"id": "x", "tokens": a[22:], "want": [7]}, {"id": "y", "tokens": b[11:], "want": [0]}], "end": ["x", "y"]}]
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    for dtype, tol in (("float32", "fp32"), ("bfloat16", "bf16")):
        r = subprocess.run([sys.executable, f"{root}/bin/trace_run", "--model", str(mdir), "--dtype", dtype, "--out", str(out), "--max-tokens", "128"],
                           input="\n".join(json.dumps(s) for s in steps) + "\n", capture_output=True, text=True, timeout=300)
        assert r.returncode == 0, r.stderr
        assert [l for l in r.stdout.splitlines() if l.startswith("done")] == ["done 0", "done 1", "done 2"]
        wa, wb = want_of(cfg, w, a), want_of(cfg, w, b)
        check(np.fromfile(out / "0.f32", "<f4").reshape(2, -1), wa[[0, 19]], tol)
        check(np.fromfile(out / "1.f32", "<f4").reshape(1, -1), wa[[21]], tol)
        check(np.fromfile(out / "2.f32", "<f4").reshape(2, -1), np.stack([wa[29], wb[11]]), tol)


def test_what_the_library_refuses():
    for bad, loop in (([attn(kv_heads=3)], None),                         # query heads not a multiple of the key heads
                      ([attn(mask={"size": 0})], None),
                      ([lat(rot_dim=4, rot={"base": 10.0, "dims": 3})], None),      # an odd number of rotated channels
                      ([lat(rot_dim=4, rot={"base": 10.0, "dims": 6})], None),      # more than the rotated part has
                      ([attn(moe(experts=6, top=3, groups=(3, 1)))], None),         # the kept groups hold fewer experts than are chosen
                      ([attn(), lat()], (1, 3, 2))):                                # a loop beyond the last layer
        cfg = config(bad, loop=None)
        if loop:
            cfg["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
        with pytest.raises((TgxError, ValueError)):
            Model(stack_desc_from_config(cfg, "fp32"))
    cfg = config([attn()], loop=None)
    w = zo.random_tensors(cfg, 0)
    m = Model(stack_desc_from_config(cfg, "fp32"))
    del w["l0.mix.talk"]
    m.load_state({k: np.asarray(v, np.float32) for k, v in w.items()}, strict=True)
    with pytest.raises(TgxError, match="l0.mix.talk"):
        m.finalize()
    m.close()


# ---- attention on the matrix cores (16-bit storage) ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("size", [1, 33, 64, 100, 0])
@pytest.mark.parametrize("kind,shape", [("attention", dict(heads=4, kv_heads=1, dim=64, vdim=32)), ("attention", dict(heads=8, kv_heads=2, dim=128, vdim=128)),
                                        ("attention", dict(heads=6, kv_heads=3, dim=48, vdim=96)), ("attention", dict(heads=3, kv_heads=3, dim=16, vdim=64)),
                                        ("attention", dict(heads=16, kv_heads=2, dim=32, vdim=32)),
                                        ("latent", dict(heads=4, dim=24, rot_dim=32, vdim=40, kv_rank=96)), ("latent", dict(heads=16, dim=64, rot_dim=64, vdim=64, kv_rank=192)),
                                        ("latent", dict(heads=3, dim=32, rot_dim=0, vdim=32, kv_rank=128))])
def test_matrix_core_attention_equals_the_lane_kernels(kind, shape, size):
    """the same bf16 weights and cached rows through both forms of each attention, under windows that start inside a key tile: portions whose 32-row tiles
    cut through tokens and windows, a mixed batch, decoding, contexts across page borders, and divided windows"""
    mask = {"size": size} if size else None
    mk_layer = attn if kind == "attention" else lat
    scale = 2.0 if kind == "attention" else 0.2
    cfg = config([mk_layer(dense(), mask=mask, scale=scale, **shape), mk_layer(mask={"size": size + 7} if size else None, scale=scale, **shape)], width=64, loop=(0, 1, 2))
    w = zo.random_tensors(cfg, shape["heads"])
    tens = {k: np.asarray(v, np.float32) for k, v in w.items()}
    mk = lambda: SlotEngine(desc=stack_desc_from_config(cfg, "bf16", max_seqs=4, max_ctx=1024, budget_tokens=2048), tensors=tens)
    fast, slow, paired = mk(), mk(), mk()
    slow.model.set_option("attn.mfma", 0)
    paired.model.set_option("attn.mix_groups", 2)          # two key / value heads per workgroup share one set of scores (by itself only on grids that fill the chip)
    a, b, c = tokens(cfg, 200, 1), tokens(cfg, 75, 2), tokens(cfg, 9, 3)
    want = want_of(cfg, w, a)[[0, 1, 69, 130, 131, 199]]
    outs = []
    for eng in (fast, slow, paired):
        o = [eng.step([("a", a[:70], [0, 1, 69]), ("b", b[:3], [2])])]
        o.append(eng.step([("a", a[70:131], [60]), ("c", c, [8]), ("b", b[3:4], [0])]))
        o.append(eng.step([("b", b[4:], [70]), ("a", a[131:132], [0])]))
        o.append(eng.step([("a", a[132:199], [])]))
        eng.model.set_option("attn.split_min", 64)
        o.append(eng.step([("a", a[199:], [0]), ("b", [5], [0])]))
        outs.append(np.concatenate(o))
    assert np.abs(outs[0] - outs[1]).max() / np.abs(outs[1]).max() < 1e-3
    assert np.abs(outs[0] - outs[2]).max() == 0.0                  # the same sums in the same order
    check(outs[0][[0, 1, 2, 4, 8, 9]], want, "bf16")               # a's positions 0, 1, 69, 130, 131, 199 in the order the steps returned them
    check(outs[0][[6, 7]], want_of(cfg, w, b)[[3, 74]], "bf16")
    fast.close(); slow.close(); paired.close()
