"""The batched serving store (kr_serve_*) with the Pamulix design against the plain float64 restatement in tests/oracle_pamulix.py.

Small random models of several shapes; every comparison is between what the store's step function returns (logits, or the residual stream after each
layer) and the oracle run on the whole sequence.  The f32 store is held to 2e-4 of the stream's scale; the bf16 store is judged row by row (typical
row within 3 %), since a router's close call may fall the other way for single tokens."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest

from tests import oracle_pamulix as O

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
YARN = (3.0, 64, 8.0, 2.0)          # factor, original, fast, slow: the ramp lies inside the pair range of small rotations


def engine(cfg, W, dtype="float32", max_tokens=1024, max_slots=4):
    from krasis_amd import model_registry as R
    from krasis_amd.scheduler import BatchEngine
    eng = BatchEngine(R.pamulix_spec(cfg), dtype=dtype, max_tokens=max_tokens, max_slots=max_slots)
    eng.load_arrays(W)
    return eng


def rel(got, ref):
    """largest row error, relative to the root mean square of the reference rows"""
    d = np.asarray(got, np.float64) - ref
    return float(np.sqrt((d ** 2).mean(-1)).max() / np.sqrt((ref ** 2).mean()))


# every size differs from layer to layer and none is 1 or equal to another by accident; both mixers in both orders; a layer without feed-forward; value
# mixing over a gap (layer 1 has none); top == experts and top == 1; a layer without a mask; rotation with and without scaled frequencies
def cfg_varied():
    return O.make_config(width=96, vocab=101, eps=1e-5, residual_mult=0.7, layers=[
        O.layer(O.attn(6, 3, 24, 16, 7, v_mix=True, scale=0.31), O.moe(12, 3, 24)),
        O.layer(O.latent(5, 12, 6, 20, 28, 18, base=300.0, scaling=YARN, scale=0.3), O.moe(6, 2, 20)),
        O.layer(O.attn(4, 2, 16, 24, 19, v_mix=True, scale=0.2), None),
        O.layer(O.attn(4, 4, 12, 20, 0, scale=0.3), O.moe(8, 8, 16)),
        O.layer(O.latent(3, 8, 4, 8, 10, 12, base=50.0, scale=0.4), O.moe(5, 1, 12)),
        O.layer(O.attn(12, 4, 8, 12, 33, v_mix=True, scale=0.45), O.moe(7, 2, 12)),
    ])


def cfg_wide():
    """rows that are multiples of 16 bytes (vector loads) and head shapes of the matrix-instruction attention: four / sixteen / two heads per key head,
    a latent whose key row is 128 wide with 64 of them values, and one whose value width has no matrix tiling"""
    return O.make_config(width=128, vocab=260, eps=1e-6, residual_mult=0.4, layers=[
        O.layer(O.attn(8, 2, 64, 64, 150, v_mix=True, scale=0.12), O.moe(16, 4, 32)),
        O.layer(O.latent(8, 32, 64, 32, 48, 64, base=1e4, scaling=(4.0, 256, 16.0, 1.0), scale=0.11), O.moe(4, 2, 48)),
        O.layer(O.attn(16, 1, 32, 64, 70, scale=0.2), None),
        O.layer(O.attn(4, 2, 32, 64, 0, v_mix=True, scale=0.2), O.moe(8, 3, 40)),
        O.layer(O.latent(16, 16, 32, 16, 32, 96, base=777.0, scale=0.15), O.moe(6, 2, 24)),
    ])


def tokens(cfg, n, seed):
    return [int(t) for t in np.random.default_rng(seed).integers(0, cfg["vocab"], n)]


@pytest.mark.parametrize("make,n", [(cfg_varied, 75), (cfg_wide, 200)])
def test_every_layer_and_logits_f32(make, n):
    cfg = make(); W = O.random_weights(cfg, 1); toks = tokens(cfg, n, 2)
    ref_logits, ref_streams = O.forward(cfg, W, toks)
    eng = engine(cfg, W)
    eng.store.set_capture(True)
    logits, amax = eng.step([("a", toks, list(range(n)))])
    streams = eng.store.read_capture(n)
    for li in range(len(cfg["layers"])):
        assert rel(streams[li], ref_streams[li]) < 2e-4, f"layer {li}"
    assert rel(logits, ref_logits) < 2e-4
    assert np.array_equal(amax, logits.argmax(-1))


@pytest.mark.parametrize("make,n", [(cfg_varied, 75), (cfg_wide, 150)])
def test_bf16_store_close_to_oracle(make, n):
    cfg = make(); W = O.random_weights(cfg, 3); toks = tokens(cfg, n, 4)
    ref_logits, _ = O.forward(cfg, W, toks)
    eng = engine(cfg, W, "bfloat16")
    logits, _ = eng.step([("a", toks, list(range(n)))])
    # a token whose two candidate experts score within the bf16 rounding of the router's input may take the other one: the rows are judged one by
    # one.  Every sublayer's output is normed to unit size before it joins the stream, so the rounding of eleven sublayers of width 8 - 24 heads adds up
    # undamped, and a flipped expert moves a whole normed sublayer output: the typical row has to be within 3 %, six in seven within 5 %
    d = logits - ref_logits
    e = np.sqrt((d ** 2).mean(-1)) / np.sqrt((ref_logits ** 2).mean())
    assert np.median(e) < 3e-2 and (e < 5e-2).mean() >= 0.85


def small_model(layers, width=64, vocab=50, mult=0.6):
    return O.make_config(width=width, vocab=vocab, eps=1e-5, residual_mult=mult, layers=layers)


@pytest.mark.parametrize("name,layers", [
    ("attention_no_mask", [O.layer(O.attn(4, 2, 16, 16, 0, scale=0.4), None)]),
    ("chunk_3", [O.layer(O.attn(4, 4, 16, 8, 3, scale=0.6), None)]),
    ("chunk_1_sees_itself_only", [O.layer(O.attn(2, 1, 8, 8, 1, scale=0.6), None)]),
    ("chunk_64_is_a_page", [O.layer(O.attn(2, 1, 8, 8, 64, scale=0.6), None)]),
    ("values_mixed_over_three_layers", [O.layer(O.attn(4, 2, 16, 12, 0, v_mix=True, scale=0.4), None), O.layer(O.attn(2, 1, 8, 24, 5, v_mix=True, scale=0.4), None),
                                        O.layer(O.attn(6, 3, 8, 8, 0, v_mix=True, scale=0.4), None)]),
    ("latent_plain_rotation", [O.layer(O.latent(4, 8, 8, 12, 20, 16, base=30.0, scale=0.3), None)]),
    ("latent_scaled_rotation", [O.layer(O.latent(4, 8, 12, 12, 20, 16, base=300.0, scaling=YARN, scale=0.3), None)]),
    ("latent_one_head", [O.layer(O.latent(1, 16, 4, 8, 9, 7, base=20.0, scaling=(2.0, 40, 4.0, 1.0), scale=0.3), None)]),
    ("experts_top_3_of_5", [O.layer(O.attn(2, 1, 8, 8, 0, scale=0.3), O.moe(5, 3, 12))]),
    ("experts_all_chosen", [O.layer(O.attn(2, 1, 8, 8, 0, scale=0.3), O.moe(4, 4, 12))]),
    ("experts_top_1", [O.layer(O.latent(2, 8, 4, 8, 12, 10, base=20.0, scale=0.3), O.moe(9, 1, 12))]),
    # shapes of the matrix-instruction attention: sixteen tokens of one head per workgroup; two batches of sixteen heads on one key head; wide values;
    # a latent whose cache row serves as key (96 wide) and value (its first 64)
    ("one_head_per_key_head_chunk_9", [O.layer(O.attn(4, 4, 32, 16, 9, scale=0.4), None)]),
    ("thirty_two_heads_on_one_key_head", [O.layer(O.attn(32, 1, 32, 16, 11, scale=0.4), None)]),
    ("values_wider_than_keys", [O.layer(O.attn(8, 2, 32, 128, 0, scale=0.3), None)]),
    ("latent_on_the_matrix_path", [O.layer(O.latent(4, 16, 32, 16, 24, 64, base=100.0, scaling=(4.0, 128, 8.0, 1.0), scale=0.2), None)]),
    # cache rows as long as real models keep them: 512 + 64 under sixteen heads, 256 + 64 under four, 128 + 64 under two
    ("latent_row_576", [O.layer(O.latent(16, 8, 64, 8, 16, 512, base=1e4, scaling=(8.0, 64, 8.0, 1.0), scale=0.2), None)]),
    ("latent_row_320", [O.layer(O.latent(4, 24, 64, 8, 16, 256, base=1e4, scale=0.15), None)]),
    ("latent_row_192", [O.layer(O.latent(2, 8, 64, 24, 16, 128, base=1e3, scale=0.2), None)]),
])
def test_each_mechanism_alone(name, layers):
    cfg = small_model(layers)
    W = O.random_weights(cfg, 5)
    toks = tokens(cfg, 40, 6)
    ref_logits, ref_streams = O.forward(cfg, W, toks)
    eng = engine(cfg, W)
    eng.store.set_capture(True)
    logits, _ = eng.step([("a", toks, list(range(40)))])
    got = eng.store.read_capture(40)
    for li in range(len(layers)):
        assert rel(got[li], ref_streams[li]) < 2e-4, (name, li)
    assert rel(logits, ref_logits) < 2e-4, name


def test_the_oracle_feels_every_mechanism(monkeypatch):
    """the oracle itself: leaving out the one in the denominator, the distance bias, the value mixing, the router bias, the frequency scaling or the
    norm on the sublayer output moves its result far beyond the tolerance the store is held to -- so the store tests do see these mechanisms"""
    cfg = small_model([O.layer(O.attn(4, 2, 16, 12, 6, v_mix=True, scale=0.4), O.moe(6, 2, 12)), O.layer(O.attn(2, 1, 8, 24, 0, v_mix=True, scale=0.4), None),
                       O.layer(O.latent(4, 8, 12, 12, 20, 16, base=300.0, scaling=YARN, scale=0.3), None)])
    W = O.random_weights(cfg, 5); toks = tokens(cfg, 30, 6)
    base, _ = O.forward(cfg, W, toks)

    def changed(**patch):
        with monkeypatch.context() as m:
            for k, v in patch.items():
                m.setattr(O, k, v)
            return O.forward(cfg, W, toks)[0]
    no_bias = changed(head_slopes=lambda H: np.zeros(H))
    assert rel(no_bias, base) > 2e-2
    no_mix = changed(mix_values=lambda v, vf, lam: v)
    assert rel(no_mix, base) > 2e-2
    plain = changed(yarn_table=lambda dims, base_, factor, original, fast, slow: O.plain_table(dims, base_))
    assert rel(plain, base) > 1e-2
    rms_out = changed(centered_norm=lambda y, w, eps: O.rms_norm(y, w, eps))
    assert rel(rms_out, base) > 1e-2
    W2 = dict(W); W2["l0.mlp.router.b"] = np.zeros_like(W["l0.mlp.router.b"])
    assert rel(O.forward(cfg, W2, toks)[0], base) > 2e-2
    # the one in the denominator: with it, scores far below zero give weights that do not sum to one
    q = np.random.default_rng(1).standard_normal((5, 2, 8)); k = np.random.default_rng(2).standard_normal((5, 1, 8)); v = np.ones((5, 1, 3))
    out = O.chunked_bias_attention(q, k, v, 0.3, 0)
    assert (out[:, :, 0] < 0.95).all() and (out[:, :, 0] > 0.05).all()


# ---------------------------------------------------------------------------------------------------------------- one key that decides
def peaked_attention_model(chunk, dim=32, width=64, vocab=40):
    """chunked attention that finds ONE key: the query projection is steered so that the query of token 1 equals the key of token 0; with a score scale
    of 1.5 that key scores about 1.5 * dim against O(sqrt(dim)) for any other, the query's own included -- whether token 0 is inside the query's chunk
    decides the output at a token 1.  Two heads: slopes 1 / 16 and 1 / 256, so the second head still sees the key hundreds of positions back."""
    cfg = small_model([O.layer(O.attn(2, 1, dim, 16, chunk, scale=1.5), None)], width=width, vocab=vocab, mult=1.0)
    W = O.random_weights(cfg, 11)
    e = W["embed"].astype(np.float64)
    steer = (W["l0.mix.k"].astype(np.float64) @ np.outer(e[0], e[1])) / (e[1] @ e[1])
    W["l0.mix.q"] = (0.3 * W["l0.mix.q"] + np.concatenate([steer, steer], 0)).astype(np.float32)
    W["l0.mix.q.norm"] = W["l0.mix.k.norm"] = np.ones(dim, np.float32)
    return cfg, W


def peaked_latent_model(width=64, vocab=40):
    """the same through latents: W_uq is steered so that the plain query part of token 1, in every head, equals the plain key part of token 0"""
    H, d, r, R, Q = 2, 16, 8, 24, 20
    cfg = small_model([O.layer(O.latent(H, d, r, 12, Q, R, base=1e4, scaling=(4.0, 512, 16.0, 1.0), scale=1.0), None)], width=width, vocab=vocab, mult=1.0)
    W = O.random_weights(cfg, 12)
    e = W["embed"].astype(np.float64)
    c0 = O.rms_norm((e[0] @ W["l0.mix.dkv"].astype(np.float64).T)[:R], W["l0.mix.dkv.norm"].astype(np.float64), 1e-5)
    k0 = (c0 @ W["l0.mix.uk"].astype(np.float64).T).reshape(H, d)
    k0 *= np.sqrt(40.0 / (k0 ** 2).sum(-1, keepdims=True))          # every head's key scores 40 against itself
    cq1 = O.rms_norm(e[1] @ W["l0.mix.dq"].astype(np.float64).T, W["l0.mix.dq.norm"].astype(np.float64), 1e-5)
    uq = 0.2 * W["l0.mix.uq"].astype(np.float64).reshape(H, d + r, Q)
    uq[:, :d] += k0[:, :, None] * cq1[None, None, :] / (cq1 @ cq1)
    W["l0.mix.uq"] = uq.reshape(H * (d + r), Q).astype(np.float32)
    # the keys of token 0 have to BE k0: scale W_uk's rows per head accordingly
    uk = W["l0.mix.uk"].astype(np.float64).reshape(H, d, R)
    raw = (c0 @ uk.reshape(H * d, R).T).reshape(H, d)
    uk *= np.sqrt(40.0 / (raw ** 2).sum(-1))[:, None, None]
    W["l0.mix.uk"] = uk.reshape(H * d, R).astype(np.float32)
    return cfg, W


def needle_sequence(vocab, n, needle_at, query_at, seed):
    """random tokens 2.., token 0 (the needle) once, token 1 (the query) once"""
    t = [int(x) for x in np.random.default_rng(seed).integers(2, vocab, n)]
    t[needle_at] = 0; t[query_at] = 1
    return t


def whole_then_decoded(eng, toks, ref, qpos, n):
    want = [qpos - 1, qpos, qpos + 1]
    whole, _ = eng.step([("w", toks, want)])
    assert rel(whole, ref[want]) < 2e-4
    eng.finish("w")
    cut = qpos - 2          # the same positions decoded one token at a time after a prompt that ends before the query
    eng.step([("d", toks[:cut], [])])
    got = []
    for p in range(cut, n):
        lg, _ = eng.step([("d", [toks[p]], [0])])
        got.append(lg[0])
    assert rel(np.stack(got), ref[cut:]) < 2e-4


@pytest.mark.parametrize("chunk,qpos,inside", [(40, 119, True), (40, 119, False), (64, 191, True), (64, 191, False), (65, 129, True), (65, 129, False),
                                               (300, 599, True), (300, 599, False), (50, 100, False), (50, 101, True)])
def test_key_at_the_start_of_the_chunk_and_just_before_it_prompt_and_decode(chunk, qpos, inside):
    """the needle sits on the first position of the query's chunk, or one position earlier; queries at a chunk's last and first positions"""
    cfg, W = peaked_attention_model(chunk)
    n = qpos + 3
    start = qpos - qpos % chunk
    needle = start if inside else start - 1
    if needle == qpos:
        needle -= 1
    toks = needle_sequence(cfg["vocab"], n, needle, qpos, 13)
    ref, _ = O.forward(cfg, W, toks)
    # the oracle's own sensitivity: the needle on the other side of the edge changes the query's logits by tens of percent
    ref2, _ = O.forward(cfg, W, needle_sequence(cfg["vocab"], n, start - 1 if inside else start, qpos, 13))
    if needle != start - 1 or start != qpos:
        assert rel(ref2[qpos:qpos + 1], ref[qpos:qpos + 1]) > 0.2
    whole_then_decoded(engine(cfg, W, max_tokens=1408), toks, ref, qpos, n)


@pytest.mark.parametrize("make", [lambda: peaked_attention_model(0), peaked_latent_model])
def test_far_key_among_hundreds_across_pages(make):
    """no mask: the one matching key sits 700 positions back, eleven pages away"""
    cfg, W = make()
    n = 780
    toks = needle_sequence(cfg["vocab"], n, 40, 740, 17)
    ref, _ = O.forward(cfg, W, toks)
    toks_moved = list(toks); toks_moved[40] = 5
    ref_moved, _ = O.forward(cfg, W, toks_moved)
    assert rel(ref_moved[740:741], ref[740:741]) > 0.2           # the far key carries the answer
    eng = engine(cfg, W, max_tokens=832)
    eng.step([("a", toks[:700], [])])
    lg, _ = eng.step([("a", toks[700:], [40])])
    assert rel(lg, ref[740:741]) < 2e-4
    eng.finish("a")
    eng.step([("b", toks[:739], [])])
    eng.step([("b", toks[739:740], [])])
    lg, _ = eng.step([("b", toks[740:741], [0])])
    assert rel(lg, ref[740:741]) < 2e-4


@pytest.mark.parametrize("make", [lambda: peaked_attention_model(0), peaked_latent_model])
@pytest.mark.parametrize("needle,query", [(63, 64), (63, 127), (64, 128), (0, 1), (0, 63), (127, 128)])
def test_keys_at_page_borders(make, needle, query):
    cfg, W = make()
    n = 140
    toks = needle_sequence(cfg["vocab"], n, needle, query, 19)
    ref, _ = O.forward(cfg, W, toks)
    eng = engine(cfg, W)
    # the prompt cut exactly at the page border before the query, then decoded
    cut = (query // 64) * 64 if query % 64 else query - 1
    cut = max(cut, 1)
    eng.step([("a", toks[:cut], [])])
    got = []
    for p in range(cut, query + 1):
        lg, _ = eng.step([("a", [toks[p]], [0])])
        got.append(lg[0])
    assert rel(np.stack(got), ref[cut:query + 1]) < 2e-4


def test_first_tokens_of_a_sequence():
    cfg = cfg_varied(); W = O.random_weights(cfg, 21); toks = tokens(cfg, 4, 22)
    ref, _ = O.forward(cfg, W, toks)
    eng = engine(cfg, W)
    one, _ = eng.step([("one", toks[:1], [0])])
    assert rel(one, ref[:1]) < 2e-4
    two, _ = eng.step([("two", toks[:2], [0, 1])])
    assert rel(two, ref[:2]) < 2e-4
    nxt, _ = eng.step([("one", toks[1:2], [0])])
    assert rel(nxt, ref[1:2]) < 2e-4


@pytest.mark.parametrize("dtype,tol", [("float32", 2e-4), ("bfloat16", 4e-2)])
def test_prefill_equals_token_by_token_decode(dtype, tol):
    cfg = cfg_varied(); W = O.random_weights(cfg, 23); n = 90; toks = tokens(cfg, n, 24)
    ref, _ = O.forward(cfg, W, toks)
    eng = engine(cfg, W, dtype)
    whole, _ = eng.step([("w", toks, list(range(n)))])
    rows = []
    for p in range(n):
        lg, _ = eng.step([("d", [toks[p]], [0])])
        rows.append(lg[0])
    dec = np.stack(rows)
    if dtype == "float32":
        assert rel(whole, ref) < tol and rel(dec, ref) < tol
    else:       # bf16: a close call of the router may fall the other way for a few tokens (see test_bf16_store_close_to_oracle)
        for got in (whole, dec):
            e = np.sqrt(((got - ref) ** 2).mean(-1)) / np.sqrt((ref ** 2).mean())
            assert np.median(e) < 3e-2 and (e < tol + 2e-2).mean() >= 0.85


@pytest.mark.parametrize("sizes", [[2] * 30, [3, 2, 7, 2, 64, 5, 65, 2, 31, 2, 9], [37, 3, 3, 37, 37, 5, 11, 25, 24, 2], [1, 128, 2, 60]])
def test_portions_of_several_sizes(sizes):
    cfg = cfg_wide(); W = O.random_weights(cfg, 25); n = sum(sizes); toks = tokens(cfg, n, 26)
    ref, _ = O.forward(cfg, W, toks)
    eng = engine(cfg, W)
    at, rows = 0, []
    for s in sizes:
        lg, _ = eng.step([("c", toks[at:at + s], list(range(s)))])
        rows.append(lg); at += s
    assert rel(np.concatenate(rows), ref) < 2e-4


@pytest.mark.parametrize("make", [cfg_varied, cfg_wide])
def test_unequal_requests_in_one_batch_equal_each_alone(make):
    cfg = make(); W = O.random_weights(cfg, 27)
    lens = {"a": 70, "b": 9, "c": 131, "d": 33}
    toks = {k: tokens(cfg, n, 30 + i) for i, (k, n) in enumerate(lens.items())}
    refs = {k: O.forward(cfg, W, t)[0] for k, t in toks.items()}
    eng = engine(cfg, W, max_tokens=512)
    # a schedule that mixes portions with single tokens: every request advances by its own stride
    stride = {"a": [17, 1, 1, 30, 1, 20], "b": [2, 1, 1, 1, 4], "c": [64, 1, 65, 1], "d": [1, 1, 31]}
    at = {k: 0 for k in lens}
    got = {k: [] for k in lens}
    step = 0
    while any(at[k] < lens[k] for k in lens):
        entries, owners = [], []
        for k in lens:
            if at[k] >= lens[k]:
                continue
            s = stride[k][step] if step < len(stride[k]) else 1
            s = min(s, lens[k] - at[k])
            entries.append((k, toks[k][at[k]:at[k] + s], list(range(s)))); owners.append((k, s)); at[k] += s
        lg, _ = eng.step(entries)
        o = 0
        for k, s in owners:
            got[k].append(lg[o:o + s]); o += s
        step += 1
    for k in lens:
        assert rel(np.concatenate(got[k]), refs[k]) < 2e-4, k


def test_pages_and_slots_are_used_again():
    """a pool of five pages and four slots: requests come and go; the later ones run in pages and slots the earlier ones gave back"""
    cfg = cfg_varied(); W = O.random_weights(cfg, 31)
    eng = engine(cfg, W, max_tokens=320, max_slots=4)
    assert eng.store.free_pages() == 5
    seqs = [tokens(cfg, n, 40 + i) for i, n in enumerate([130, 60, 64, 100, 65, 190, 20, 129])]
    refs = [O.forward(cfg, W, t)[0] for t in seqs]
    a, _ = eng.step([(0, seqs[0], [129]), (1, seqs[1], [59]), (2, seqs[2], [63])])      # 3 + 1 + 1 pages: the pool is full
    assert eng.store.free_pages() == 0
    with pytest.raises(RuntimeError):
        eng.step([(3, seqs[3], [0])])                        # no page left: refused, nothing changed
    assert rel(a, np.stack([refs[0][129], refs[1][59], refs[2][63]])) < 2e-4
    eng.finish(0); eng.finish(3)                            # request 3 was admitted (slot) but holds no page
    assert eng.store.free_pages() == 3
    b, _ = eng.step([(3, seqs[3], [99]), (4, seqs[4][:40], [39])])          # 2 + 1 pages, out of request 0's
    assert rel(b, np.stack([refs[3][99], refs[4][39]])) < 2e-4
    eng.finish(1); eng.finish(2)
    c, _ = eng.step([(4, seqs[4][40:], [24]), (3, [seqs[3][0]], [])])      # request 4 crosses into a second page (one that request 1 or 2 held)
    assert rel(c, refs[4][64:65]) < 2e-4
    eng.finish(3); eng.finish(4)
    assert eng.store.free_pages() == 5
    d, _ = eng.step([(5, seqs[5], [0, 189]), (6, seqs[6], [19])])
    assert rel(d, np.stack([refs[5][0], refs[5][189], refs[6][19]])) < 2e-4
    eng.finish(5)
    e, _ = eng.step([(7, seqs[7], [128]), (6, [3], [0])])
    assert rel(e[:1], refs[7][128:129]) < 2e-4


def test_long_decoding_through_pages_and_chunks():
    cfg = cfg_wide(); W = O.random_weights(cfg, 33); n = 330; toks = tokens(cfg, n, 34)
    ref, _ = O.forward(cfg, W, toks)
    eng = engine(cfg, W)
    eng.step([("a", toks[:20], [])])
    rows = []
    for p in range(20, n):
        lg, _ = eng.step([("a", [toks[p]], [0])])
        rows.append(lg[0])
    assert rel(np.stack(rows), ref[20:]) < 2e-4


@pytest.mark.parametrize("mixer", [O.latent(16, 8, 64, 8, 16, 512, base=1e4, scaling=(8.0, 64, 8.0, 1.0), scale=0.2), O.latent(4, 24, 64, 8, 16, 256, base=1e4, scale=0.15),
                                   O.latent(2, 8, 64, 24, 16, 128, base=1e3, scale=0.2), O.attn(8, 2, 64, 64, 0, scale=0.12)])
def test_decoding_over_a_long_cache_on_the_matrix_path(mixer):
    """decode steps whose keys are split over several workgroups (partial states merged by a second launch), for the long cache rows of latent layers"""
    cfg = small_model([O.layer(mixer, O.moe(4, 2, 16))]); W = O.random_weights(cfg, 45); n = 600; toks = tokens(cfg, n, 46)
    ref, _ = O.forward(cfg, W, toks)
    eng = engine(cfg, W)
    eng.step([("a", toks[:570], [])])
    rows = []
    for p in range(570, n):
        lg, _ = eng.step([("a", [toks[p]], [0])])
        rows.append(lg[0])
    assert rel(np.stack(rows), ref[570:]) < 2e-4


def greedy_oracle(cfg, W, prompt, n_new):
    seq, out, margins = list(prompt), [], []
    for _ in range(n_new):
        lg = O.forward(cfg, W, seq)[0][-1]
        top = np.sort(lg)[-2:]
        margins.append(float(top[1] - top[0]))
        out.append(int(lg.argmax())); seq.append(out[-1])
    return out, min(margins)


def test_greedy_generation_through_the_scheduler():
    """five prompts, four slots, a pool that cannot hold all at once, a step budget that cuts prompts into portions"""
    cfg = cfg_varied(); W = O.random_weights(cfg, 35)
    prompts = [tokens(cfg, n, 50 + i) for i, n in enumerate([45, 3, 70, 18, 29])]
    eng = engine(cfg, W, max_tokens=256, max_slots=4)
    outs = eng.generate(prompts, 6, token_budget=32)
    assert eng.store.free_pages() == 4 and not eng.live()
    for p, o in zip(prompts, outs):
        want, margin = greedy_oracle(cfg, W, p, 6)
        if margin > 1e-3:                                   # a near-tie of the two best logits may fall either way in f32
            assert o == want
        else:
            assert o[0] == want[0] or margin < 1e-3


def test_sampling_uses_the_frameworks_sampler():
    cfg = cfg_varied(); W = O.random_weights(cfg, 37); p = tokens(cfg, 12, 38)
    eng = engine(cfg, W)
    a = eng.generate([p], 8, temperature=0.8, top_k=5, top_p=0.9, seed=7)
    b = eng.generate([p], 8, temperature=0.8, top_k=5, top_p=0.9, seed=7)
    assert a == b and len(a[0]) == 8
    g = eng.generate([p], 8)
    k1 = eng.generate([p], 8, temperature=1.3, top_k=1, seed=3)      # top_k = 1 is greedy whatever the temperature
    assert g == k1


def test_checkpoint_directory_command_line_and_trace_replay(tmp_path):
    cfg = cfg_varied(); W = O.random_weights(cfg, 39)
    model = str(tmp_path / "model"); O.write_checkpoint(model, cfg, W)
    from krasis_amd import model_registry as R
    assert R.model_family(R.read_config(model)) == "serve:Pamulix"
    p1, p2 = tokens(cfg, 20, 60), tokens(cfg, 7, 61)
    env = dict(os.environ, PYTHONPATH=ROOT)
    out = subprocess.run([sys.executable, "-m", "krasis_amd", "generate", "--model", model, "--dtype", "float32", "--max-new-tokens", "4",
                          "--prompt", ",".join(map(str, p1)), "--prompt", ",".join(map(str, p2))], env=env, capture_output=True, text=True, timeout=300)
    assert out.returncode == 0, out.stderr[-2000:]
    lines = [json.loads(x) for x in out.stdout.splitlines() if x.startswith("{")]
    for p, line in zip((p1, p2), lines):
        want, margin = greedy_oracle(cfg, W, p, 4)
        assert line["prompt"] == p and (line["tokens"] == want or margin < 1e-3)
    # trace replay: two requests, portions beside single tokens, one ends early and its slot is used again
    steps = [{"step": 0, "entries": [{"id": "x", "tokens": p1[:11], "want": [10]}, {"id": "y", "tokens": p2[:2], "want": []}], "end": []},
             {"step": 1, "entries": [{"id": "x", "tokens": p1[11:12], "want": [0]}, {"id": "y", "tokens": p2[2:], "want": [0, 4]}], "end": ["y"]},
             {"step": 2, "entries": [{"id": "x", "tokens": p1[12:], "want": []}], "end": []},
             {"step": 3, "entries": [{"id": "z", "tokens": p2, "want": [6]}], "end": ["x", "z"]}]
    outdir = str(tmp_path / "out")
    r = subprocess.run([os.path.join(ROOT, "bin", "trace_run"), "--model", model, "--dtype", "float32", "--out", outdir, "--max-tokens", "128"],
                       input="\n".join(json.dumps(s) for s in steps) + "\n", env=env, capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    assert [x for x in r.stdout.splitlines() if x.startswith("done")] == ["done 0", "done 1", "done 2", "done 3"]
    r1, r2 = O.forward(cfg, W, p1)[0], O.forward(cfg, W, p2)[0]
    V = cfg["vocab"]
    g0 = np.fromfile(os.path.join(outdir, "0.f32"), "<f4").reshape(-1, V)
    g1 = np.fromfile(os.path.join(outdir, "1.f32"), "<f4").reshape(-1, V)
    g3 = np.fromfile(os.path.join(outdir, "3.f32"), "<f4").reshape(-1, V)
    assert not os.path.exists(os.path.join(outdir, "2.f32"))
    assert rel(g0, r1[10:11]) < 2e-4 and rel(g1, np.stack([r1[11], r2[2], r2[6]])) < 2e-4 and rel(g3, r2[6:7]) < 2e-4


def test_store_refuses_what_it_cannot_run():
    from krasis_amd import serve_store as S
    with pytest.raises(ValueError):          # a window and a chunk on one layer
        S.ServeStore(50, 32, [S.LayerSpec(heads=4, kv_heads=2, dim=8, vdim=8, window=5, chunk=4)])
    with pytest.raises(ValueError):          # values to blend, but no earlier layer keeps its own
        S.ServeStore(50, 32, [S.LayerSpec(heads=4, kv_heads=2, dim=8, vdim=8, v_mix=S.VMIX_BLEND)])
    with pytest.raises(ValueError):          # the kept values have another size
        S.ServeStore(50, 32, [S.LayerSpec(heads=4, kv_heads=2, dim=8, vdim=8, v_mix=S.VMIX_FIRST), S.LayerSpec(heads=4, kv_heads=2, dim=8, vdim=12, v_mix=S.VMIX_BLEND)])
    with pytest.raises(ValueError):          # a latent mixer without ranks
        S.ServeStore(50, 32, [S.LayerSpec(heads=4, kv_heads=1, dim=8, vdim=8, mixer_kind=S.MIX_LATENT)])
    with pytest.raises(ValueError):          # norms on sublayer outputs in a parallel block
        S.ServeStore(50, 32, [S.LayerSpec(heads=4, kv_heads=2, dim=8, vdim=8)], post_norm=1)
    st = S.ServeStore(50, 32, [S.LayerSpec(heads=4, kv_heads=1, dim=8, vdim=8, mixer_kind=S.MIX_LATENT, q_rank=6, kv_rank=10, rot_dims=4)],
                      block_kind=S.BLOCK_SEQUENTIAL, pre_norm=0, post_norm=1, norm_bias=0)
    with pytest.raises(RuntimeError):
        st.finalize()                                         # tensors missing
    with pytest.raises(ValueError):
        st.set_tensor(0, "q", np.zeros((32, 32), np.float32))  # a latent mixer has no q matrix
    with pytest.raises(ValueError):
        st.set_tensor(0, "uk", np.zeros((32, 9), np.float32))  # wrong shape


def test_graph_replays_equal_eager_steps():
    """decode steps replay a captured graph from their second visit on; every replay is compared with a store that runs eagerly, with eager steps of
    other shapes (a prompt portion of a third request) and host synchronisation between the replays"""
    cfg = cfg_wide(); W = O.random_weights(cfg, 41)
    a, b = tokens(cfg, 150, 42), tokens(cfg, 150, 43)
    c = tokens(cfg, 60, 44)
    eng_g, eng_e = engine(cfg, W, "bfloat16"), engine(cfg, W, "bfloat16")
    eng_e.store.set_use_graph(False)
    for eng in (eng_g, eng_e):
        eng.step([("a", a[:30], []), ("b", b[:7], [])])
    for i in range(100):
        entries = [("a", [a[30 + i]], [0]), ("b", [b[7 + i]], [0])]
        lg, am = eng_g.step(entries)
        le, ae = eng_e.step(entries)
        assert np.array_equal(lg, le) and np.array_equal(am, ae), i
        if i % 25 == 10:                                    # an eager step of another shape in between
            part = c[(i // 25) * 15:(i // 25) * 15 + 15]
            lg, _ = eng_g.step([("c", part, [14])]); le, _ = eng_e.step([("c", part, [14])])
            assert np.array_equal(lg, le)
    assert eng_g.store.graph_replays() >= 60 and eng_e.store.graph_replays() == 0
    lg, _ = eng_g.step([("a", [a[130]], [0])])
    ref = O.forward(cfg, W, a[:131])[0]
    e = np.sqrt(((lg[0] - ref[130]) ** 2).mean()) / np.sqrt((ref ** 2).mean())
    assert e < 4e-2
