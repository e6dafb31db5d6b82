"""The Vitudra design on the GPU against the plain oracle of tests/vitudra_oracle.py: every mechanism on a configuration of its own, prompts against
token-by-token decoding, portions down to two tokens, mixed batches, slots and pages that are used again, keys just inside and just outside every window
and chunk (in prompts and in decoding), far keys, page borders, long decoding through the recurrent states, and greedy generation through the slot
scheduler, tgx_forward / tgx_sample / tgx_decode, the C++ engine, the command line and bin/trace_run.  Models are config dictionaries of the checkpoint
format, so the configuration reader is on the path of every test.  fp32 storage is the sharp comparison (nothing is rounded: 1e-4 of the largest
logit); bf16 storage rounds the cached keys and values (3e-2)."""
import copy
import json
import os
import subprocess
import sys

import numpy as np
import pytest

import vitudra_oracle as vo
from test_hip_modepel import write_model_dir
from tinygpt_amd.desc import stack_desc_from_config
from tinygpt_amd.ffi import GREEDY, Model, TgxError
from tinygpt_amd.serving import SlotEngine

pytestmark = pytest.mark.gpu
TOL = {"fp32": 1e-4, "bf16": 3e-2}


# ---- configurations ---------------------------------------------------------------------------------------------------------------
def ff(n=20):
    return {"kind": "dense", "ff": n}


def attn(mlp=None, **kw):
    m = dict(heads=4, kv_heads=2, dim=8, vdim=6, mask={"size": 11}, q_temp={"coef": 0.4, "every": 5}, scale=0.7)
    m.update(kw)
    return {"type": "attention", "mixer": {k: v for k, v in m.items() if v is not None}, "mlp": mlp}


def wkv(mlp=None, **kw):
    m = dict(heads=3, dim=6)
    m.update(kw)
    return {"type": "wkv", "mixer": m, "mlp": mlp}


def par(mlp=None, left=None, right=None, left_scale=0.8, right_scale=1.3):
    l = dict(heads=4, kv_heads=2, dim=8, vdim=10, mask={"size": 9}, rot={"base": 300.0, "dims": 4, "scaling": {"factor": 3.0}}, scale=0.5, softcap=4.0)
    r = dict(conv=4, dim=6, heads=4, kv_heads=2, vdim=5)
    l.update(left or {}); r.update(right or {})
    return {"type": "parallel", "mixer": {"left": {k: v for k, v in l.items() if v is not None}, "right": r, "left_scale": left_scale, "right_scale": right_scale}, "mlp": mlp}


def config(layers=None, width=24, vocab=67, eps=1e-5, mult=0.4):
    return {"architecture": "Vitudra", "width": width, "vocab": vocab, "norm": {"eps": eps}, "residual_mult": mult,
            "layers": copy.deepcopy(layers) if layers is not None else [wkv(ff()), par(ff(13)), attn(ff()), par(), attn(ff(9), kv_from=2)]}


def engine(cfg, dtype="fp32", seed=0, overrides=None, decay_rank=5, **kw):
    w = vo.random_tensors(cfg, seed, overrides, decay_rank)
    kw = dict(dict(max_seqs=4, max_ctx=1024, budget_tokens=2048), **kw)
    eng = SlotEngine(desc=stack_desc_from_config(cfg, dtype, **kw), tensors={k: np.asarray(v, np.float32) for k, v in w.items()})
    return eng, w


def tokens(cfg, n, seed=0):
    return np.random.default_rng(100 + seed).integers(0, cfg["vocab"], n).tolist()


def want_of(cfg, w, toks):
    return vo.forward(cfg, w, toks)


def check(got, want, dtype, what=""):
    err = np.abs(got - want).max() / np.abs(want).max()
    assert err < TOL[dtype], f"{what}: {err:.3e}"


def run_whole(eng, rid, toks):
    return eng.step([(rid, toks, list(range(len(toks))))], [rid])


# ---- every mechanism on a configuration of its own --------------------------------------------------------------------------------------
MECH = {
    "wkv_alone": [wkv()],
    "wkv_one_wide_head": [wkv(heads=1, dim=70)],                           # two column chunks
    "wkv_many_small_heads": [wkv(heads=8, dim=3)],
    "wkv_large_keys": [wkv(heads=2, dim=130)],
    "wkv_twice": [wkv(ff()), wkv()],
    "window_attention_alone": [attn()],
    "window_of_one": [attn(mask={"size": 1})],                              # a token sees itself only
    "window_longer_than_the_sequence": [attn(mask={"size": 500})],
    "no_mask_no_temperature": [attn(mask=None, q_temp=None)],
    "temperature_every_position": [attn(q_temp={"coef": 1.5, "every": 1})],
    "one_key_head_per_query_head": [attn(kv_heads=4)],
    "one_key_head_for_all": [attn(heads=6, kv_heads=1)],
    "wide_heads": [attn(heads=2, kv_heads=1, dim=80, vdim=72, scale=0.2)],  # more than one channel per lane
    "shared_keys_and_values": [attn(ff()), attn(ff(), kv_from=0, mask={"size": 4}, q_temp={"coef": 0.9, "every": 3})],
    "shared_twice_across_other_layers": [attn(), wkv(), attn(kv_from=0), par(), attn(kv_from=0, mask={"size": 30})],
    "parallel_alone": [par()],
    "parallel_left_half_only": [par(right_scale=0.0)],
    "parallel_right_half_only": [par(left_scale=0.0)],
    "all_dimensions_rotated": [par(left={"rot": {"base": 10000.0, "dims": 8, "scaling": {"factor": 1.0}}})],
    "two_dimensions_rotated_no_scaling": [par(left={"rot": {"base": 7.0, "dims": 2}})],
    "no_rotation_no_cap_no_mask": [par(left={"rot": None, "softcap": None, "mask": None})],
    "tight_cap": [par(left={"softcap": 0.5, "scale": 3.0})],
    "chunks_of_one": [par(left={"mask": {"size": 1}})],
    "chunks_longer_than_the_sequence": [par(left={"mask": {"size": 400}})],
    "left_groups": [par(left={"heads": 6, "kv_heads": 1, "dim": 10, "vdim": 4})],
    "one_tap": [par(right={"conv": 1})],
    "two_taps": [par(right={"conv": 2})],
    "eight_taps": [par(right={"conv": 8})],
    "more_taps_than_tokens_in_a_page": [par(right={"conv": 30})],
    "delta_every_head_its_own_keys": [par(right={"heads": 3, "kv_heads": 3})],
    "delta_one_key_head": [par(right={"heads": 6, "kv_heads": 1})],
    "delta_wide_values": [par(right={"heads": 2, "kv_heads": 1, "dim": 12, "vdim": 70})],
    "delta_large_keys": [par(right={"heads": 2, "kv_heads": 2, "dim": 130, "vdim": 9})],
    "feed_forward_everywhere": [wkv(ff(33)), par(ff(8)), attn(ff(19))],
    "no_feed_forward_anywhere": [attn(), par(), wkv()],
    "ragged_sizes": [wkv(ff(19), heads=3, dim=5), par(ff(11), left={"heads": 6, "kv_heads": 3, "dim": 6, "vdim": 5, "rot": {"base": 50.0, "dims": 6}}, right={"dim": 7, "vdim": 3, "conv": 3}),
                     attn(heads=3, kv_heads=3, dim=5, vdim=7)],
    "deep": [wkv(ff()), par(ff(13)), attn(ff()), par(), attn(ff(9), kv_from=2), wkv(ff()), par(ff(13)), attn(ff()), par(), attn(ff(9), kv_from=7)],
}
EXTRA = {"ragged_sizes": dict(width=27, vocab=53), "wide_heads": dict(width=40), "deep": dict(mult=1.0), "wkv_twice": dict(mult=1.0)}
RANKS = {"wkv_alone": 1, "wkv_twice": 9, "wkv_large_keys": 16}


@pytest.mark.parametrize("dtype", ["fp32", "bf16"])
@pytest.mark.parametrize("name", list(MECH))
def test_mechanism(name, dtype):
    cfg = config(MECH[name], **EXTRA.get(name, {}))
    eng, w = engine(cfg, dtype, seed=len(name), decay_rank=RANKS.get(name, 5))
    toks = tokens(cfg, 23, seed=len(name))
    want = want_of(cfg, w, toks)
    check(run_whole(eng, "a", toks), want, dtype, name)
    # ... and the same tokens one by one through the cache and the recurrent states
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
    """portions cut through windows, chunks, the convolution's taps and the token shift"""
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
    cfg = config([attn(mask={"size": 70}, scale=2.0), par(left={"mask": {"size": 128}}), attn(ff(), kv_from=0, mask={"size": 129})])
    eng, w = engine(cfg, "fp32", 4)
    toks = tokens(cfg, n + 3, seed=n)
    want = want_of(cfg, w, toks)
    got = [eng.step([("r", toks[:n], [n - 1])])]
    got += [eng.step([("r", [toks[n + i]], [0])]) for i in range(3)]      # decoding across the border
    check(np.concatenate(got), want[n - 1:], "fp32")
    eng.close()


# ---- keys that stand out: a window's or a chunk's edge that is one token off shows as a large error --------------------------------------------
def loud(cfg, seed, q_name, k_name, q_rows, k_row):
    """weights in which token id 7 carries a key that every query asks for: its embedding row is one loud coordinate (0) that no other token has, the key
    projection turns that coordinate into a large key channel, and a coordinate that every token shares (1) drives every query towards that channel"""
    w0 = vo.random_tensors(cfg, seed)
    emb = w0["embed"].copy()
    emb[:, 0] = 0.0; emb[:, 1] = 2.0; emb[7] = 0.0; emb[7, 0] = 6.0; emb[7, 1] = 2.0
    k = w0[k_name].copy(); k[:, 0] = 0.0; k[:, 1] = 0.0; k[k_row, 0] = 8.0
    q = w0[q_name].copy(); q[:, 0] = 0.0; q[:, 1] = 0.0
    for r in q_rows:
        q[r, 1] = 3.0
    n1 = np.zeros_like(w0["l0.norm1"])
    return {"embed": emb, k_name: k, q_name: q, "l0.norm1": n1}


@pytest.mark.parametrize("dtype", ["fp32", "bf16"])
@pytest.mark.parametrize("size,at", [(5, 3), (64, 0), (64, 10), (65, 63), (100, 130), (200, 1)])
def test_window_edges_in_prompts_and_in_decoding(size, at, dtype):
    """the loud key sits at position `at`: the queries up to at + size - 1 see it, the query at at + size is the first that does not"""
    cfg = config([attn(heads=2, kv_heads=1, dim=8, vdim=8, mask={"size": size}, scale=1.0, q_temp=None)], width=16, mult=1.0)
    over = loud(cfg, 6, "l0.mix.q", "l0.mix.k", (5, 13), 5)
    n = at + size + 6
    toks = [t if t != 7 else 8 for t in tokens(cfg, n, seed=size)]
    toks[at] = 7
    edge = at + size                                       # the first position that no longer sees the key
    for cut in (n, edge - 1, edge, edge + 1, max(at + 1, edge - 3)):      # the prompt ends before, at and behind the edge; the rest is decoded
        eng, w = engine(cfg, dtype, 6, over)
        want = want_of(cfg, w, toks)
        if cut == n:
            without = list(toks); without[at] = 9
            other = want_of(cfg, w, without)
            assert np.abs(other[edge - 1] - want[edge - 1]).max() / np.abs(want).max() > 0.05      # inside: the key decides the logits
            assert np.abs(other[edge:] - want[edge:]).max() == 0.0                                 # outside: it is gone
        places = sorted({p for p in (at, edge - 2, edge - 1, edge, edge + 1, n - 1) if at <= p < n})
        got = [eng.step([("r", toks[:cut], [p for p in places if p < cut])])]
        got += [eng.step([("r", [toks[i]], [0] if i in places else [])]) for i in range(cut, n)]
        check(np.concatenate([g for g in got if len(g)]), want[places], dtype, f"prompt of {cut}")
        eng.close()


@pytest.mark.parametrize("dtype", ["fp32", "bf16"])
@pytest.mark.parametrize("size,at", [(4, 5), (64, 64), (64, 127), (70, 75), (130, 131), (200, 3)])
def test_chunk_edges_in_prompts_and_in_decoding(size, at, dtype):
    """the loud key sits at position `at`: the rest of its block of `size` positions sees it, the next block's first position does not"""
    left = {"heads": 2, "kv_heads": 1, "dim": 8, "vdim": 8, "mask": {"size": size}, "scale": 1.0, "softcap": 30.0, "rot": {"base": 10000.0, "dims": 2}}
    cfg = config([par(left=left, right_scale=0.0)], width=16, mult=1.0)
    over = loud(cfg, 7, "l0.mix.left.q", "l0.mix.left.k", (5, 13), 5)
    edge = (at // size + 1) * size                         # the first position of the next block
    n = edge + 5
    toks = [t if t != 7 else 8 for t in tokens(cfg, n, seed=size)]
    toks[at] = 7
    for cut in (n, edge - 1, edge, edge + 1, at + 1):
        eng, w = engine(cfg, dtype, 7, over)
        want = want_of(cfg, w, toks)
        if cut == n and edge - 1 > at:
            without = list(toks); without[at] = 9
            other = want_of(cfg, w, without)
            assert np.abs(other[edge - 1] - want[edge - 1]).max() / np.abs(want).max() > 0.05
            assert np.abs(other[edge:] - want[edge:]).max() == 0.0
        places = sorted({p for p in (at, edge - 2, edge - 1, edge, edge + 1, n - 1) if at <= p < n})
        got = [eng.step([("r", toks[:cut], [p for p in places if p < cut])])]
        got += [eng.step([("r", [toks[i]], [0] if i in places else [])]) for i in range(cut, n)]
        check(np.concatenate([g for g in got if len(g)]), want[places], dtype, f"prompt of {cut}")
        eng.close()


def test_one_far_key_stands_out():
    """the loud key occurs once, at position 3 of 400, under a window that still holds it: every later query must find it among hundreds of keys, across
    page borders, in portions and in decoded tokens, against the distance bias"""
    cfg = config([attn(heads=2, kv_heads=1, dim=8, vdim=8, mask={"size": 450}, scale=1.0, q_temp={"coef": 0.2, "every": 64})], width=16, mult=1.0)
    over = loud(cfg, 8, "l0.mix.q", "l0.mix.k", (5, 13), 5)
    eng, w = engine(cfg, "fp32", 8, over)
    toks = [t if t != 7 else 8 for t in tokens(cfg, 400)]
    toks[3] = 7
    want = want_of(cfg, w, toks)
    without = list(toks); without[3] = 9
    assert np.abs(want_of(cfg, w, without)[390:] - want[390:]).max() / np.abs(want).max() > 0.05
    got = [eng.step([("r", toks[:200], [2, 3, 4, 199])]), eng.step([("r", toks[200:390], [0, 189])])]
    got += [eng.step([("r", [toks[390 + i]], [0])]) for i in range(10)]
    check(np.concatenate(got), want[[2, 3, 4, 199, 200, 389] + list(range(390, 400))], "fp32")
    eng.close()


def test_split_keys_form_equals_the_direct_form():
    cfg = config([attn(mask={"size": 300}, scale=2.0), par(left={"mask": {"size": 256}}), attn(mask=None, kv_from=0)])
    eng, w = engine(cfg, "fp32", 6)
    toks = tokens(cfg, 700)
    want = want_of(cfg, w, toks)
    eng.step([("r", toks[:690], [])])
    eng.model.set_option("attn.split_min", 64)            # steps of few tokens now divide the keys between workgroups
    got = np.concatenate([eng.step([("r", [toks[690 + i]], [0])]) for i in range(10)])
    check(got, want[690:], "fp32")
    eng.close()


def test_long_memory_through_the_recurrent_states():
    """decays held near one: both matrix states still carry the first token after hundreds of steps, through portions and single tokens"""
    cfg = config([wkv(ff()), par(left_scale=0.0), wkv()])
    w0 = vo.random_tensors(cfg, 7)
    over = {"l0.mix.w0": np.full_like(w0["l0.mix.w0"], -7.0), "l0.mix.w2": w0["l0.mix.w2"] * 0.05, "l2.mix.w0": np.full_like(w0["l2.mix.w0"], -7.0), "l2.mix.w2": w0["l2.mix.w2"] * 0.05,
            "l1.mix.right.A_log": np.full_like(w0["l1.mix.right.A_log"], -7.0)}
    eng, w = engine(cfg, "fp32", 7, over)
    toks = tokens(cfg, 330)
    want = want_of(cfg, w, toks)
    other = want_of(cfg, w, [toks[0] + 1] + toks[1:])
    assert np.abs(other[-1] - want[-1]).max() / np.abs(want).max() > 1e-3      # the first token still matters at the end
    got = [eng.step([("r", toks[:5], [4])]), eng.step([("r", toks[5:130], [0, 124])]), eng.step([("r", toks[130:300], [169])])]
    got += [eng.step([("r", [toks[300 + i]], [0])]) for i in range(30)]
    check(np.concatenate(got), want[[4, 5, 129, 299] + list(range(300, 330))], "fp32")
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
    """a slot's next request starts from empty states, token shift and convolution tails, whatever the request before left there"""
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
    cfg = config([wkv(ff()), par(ff()), attn(mask={"size": 40}), attn(kv_from=2, mask={"size": 90})])
    w = vo.random_tensors(cfg, 10)
    m = Model(stack_desc_from_config(cfg, "fp32", max_seqs=2, max_ctx=512)).load_state({k: np.asarray(v, np.float32) for k, v in w.items()}, strict=True).finalize()
    prompts = np.array([tokens(cfg, 7, 1), tokens(cfg, 7, 2)])
    m.forward(prompts)
    first = m.sample(GREEDY)
    rest = np.concatenate([m.decode(75, GREEDY), m.decode(75, GREEDY)])      # crosses two page borders, the windows and many chunks; positions, states and their buffer parity (an odd count) advance on the device
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
    cfg = config([wkv(ff()), par(ff()), attn(), attn(kv_from=2)])
    w = vo.random_tensors(cfg, 11, decay_rank=7)           # (the C++ reader leaves the decay rank to the tensors)
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
    cfg = config([attn(ff()), wkv(), par(ff()), attn(kv_from=0)])
    w = vo.random_tensors(cfg, 12, decay_rank=3)
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
    for bad in ([attn(kv_heads=3)],                       # query heads not a multiple of the key heads
                [attn(), attn(kv_from=0, dim=4)],         # a sharing layer whose key size is not the pool's
                [attn(kv_from=0)],                        # a layer cannot read its own (missing) pool
                [wkv(), attn(kv_from=0)],                 # ... nor a layer without keys
                [par(right={"heads": 4, "kv_heads": 3})],
                [par(right={"conv": 65})],
                [attn(mask={"size": 0})]):
        with pytest.raises(TgxError):
            Model(stack_desc_from_config(config(bad), "fp32"))
    cfg = config([wkv()])
    w = vo.random_tensors(cfg, 0)
    m = Model(stack_desc_from_config(cfg, "fp32"))
    del w["l0.mix.mu.g"]
    m.load_state({k: np.asarray(v, np.float32) for k, v in w.items()}, strict=True)
    with pytest.raises(TgxError, match="l0.mix.mu.g"):
        m.finalize()
    m.close()
    w = vo.random_tensors(cfg, 0, decay_rank=4)
    m = Model(stack_desc_from_config(cfg, "fp32"))
    w["l0.mix.w2"] = w["l0.mix.w2"][:, :3]                # the two halves of the decay product disagree about its inner size
    with pytest.raises(TgxError, match="w2"):
        m.load_state({k: np.asarray(v, np.float32) for k, v in w.items()}, strict=True)
    m.close()


# ---- attention on the matrix cores (16-bit storage; key sizes 64 / 128 / 256, value sizes in steps of 32) --------------------------------------
@pytest.mark.parametrize("kind,size", [("window", 1), ("window", 33), ("window", 64), ("window", 100), ("chunk", 1), ("chunk", 31), ("chunk", 64), ("chunk", 150), ("none", 0)])
@pytest.mark.parametrize("heads,kv,dim,vdim", [(4, 1, 64, 32), (8, 2, 128, 128), (6, 3, 64, 96)])
def test_matrix_core_attention_equals_the_lane_kernel(heads, kv, dim, vdim, kind, size):
    """the same bf16 weights and cached rows through both attention kernels, under every mask: portions whose 32-row tiles cut through tokens, windows and
    chunks that start inside a key tile, a mixed batch, decoding, contexts across page borders, and the split-keys form"""
    mask = {"size": size} if size else None
    if kind == "chunk" or kind == "none":
        layers = [par(left=dict(heads=heads, kv_heads=kv, dim=dim, vdim=vdim, mask=mask if kind == "chunk" else None, rot={"base": 10000.0, "dims": 32, "scaling": {"factor": 2.0}},
                                scale=1.2 * dim ** -0.5, softcap=1.5))]
    else:
        layers = [attn(heads=heads, kv_heads=kv, dim=dim, vdim=vdim, mask=mask, scale=1.2 * dim ** -0.5), attn(heads=heads, kv_heads=kv, dim=dim, vdim=vdim, mask={"size": size + 7}, scale=dim ** -0.5, kv_from=0)]
    cfg = config(layers, width=64)
    w = vo.random_tensors(cfg, heads)
    tens = {k: np.asarray(v, np.float32) for k, v in w.items()}
    mk = lambda: SlotEngine(desc=stack_desc_from_config(cfg, "bf16", max_seqs=4, max_ctx=1024, budget_tokens=2048), tensors=tens)
    fast, slow = mk(), mk()
    slow.model.set_option("attn.mfma", 0)
    a, b, c = tokens(cfg, 200, 1), tokens(cfg, 75, 2), tokens(cfg, 9, 3)
    want = want_of(cfg, w, a)[[0, 1, 69, 130, 131, 199]]
    outs = []
    for eng in (fast, slow):
        o = [eng.step([("a", a[:70], [0, 1, 69]), ("b", b[:3], [2])])]
        o.append(eng.step([("a", a[70:131], [60]), ("c", c, [8]), ("b", b[3:4], [0])]))
        o.append(eng.step([("b", b[4:], [70]), ("a", a[131:132], [0])]))
        o.append(eng.step([("a", a[132:199], [])]))
        eng.model.set_option("attn.split_min", 64)
        o.append(eng.step([("a", a[199:], [0]), ("b", [5], [0])]))
        outs.append(np.concatenate(o))
    assert np.abs(outs[0] - outs[1]).max() / np.abs(outs[1]).max() < 3e-4
    check(outs[0][[0, 1, 2, 4, 8, 9]], want, "bf16")               # a's positions 0, 1, 69, 130, 131, 199 in the order the steps returned them
    check(outs[0][[6, 7]], want_of(cfg, w, b)[[3, 74]], "bf16")
    fast.close(); slow.close()
