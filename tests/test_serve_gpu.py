"""The batched serving store (kr_serve_*) with the Lomutar design against the plain float64 restatement in tests/oracle_serve.py.

Small random models of several shapes; every comparison is between what the store's step function returns (logits, or the residual stream after each
layer) and the oracle run on the whole sequence.  The f32 store is held to 2e-4 of the stream's scale, the bf16 store to 4e-2."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest

from tests import oracle_serve as O

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def engine(cfg, W, dtype="float32", max_tokens=1024, max_slots=4):
    from krasis_amd import model_registry as R
    from krasis_amd.scheduler import BatchEngine
    eng = BatchEngine(R.lomutar_spec(cfg), dtype=dtype, max_tokens=max_tokens, max_slots=max_slots)
    eng.load_arrays(W)
    return eng


def rel(got, ref):
    """largest row error, relative to the root mean square of the reference rows"""
    d = np.asarray(got, np.float64) - ref
    return float(np.sqrt((d ** 2).mean(-1)).max() / np.sqrt((ref ** 2).mean()))


# head counts, head sizes, windows, rotation, router and expert sizes all differ from layer to layer and are never equal to one another or 1 by accident
def cfg_varied():
    return O.make_config(width=96, vocab=101, eps=1e-5, layers=[
        {"type": "attention", "mixer": O.attn(6, 3, 24, 16, 7, 10, base=5000.0, factor=1.5, scale=0.31), "mlp": O.dense(80)},
        {"type": "attention", "mixer": O.attn(6, 2, 16, 40, 19, 16, base=300.0, factor=4.0, scale=0.2), "mlp": O.moe(12, 3, 3, 2, 24, 1.25, 40, 0.75)},
        {"type": "attention", "mixer": O.attn(6, 2, 16, 40, 5, 16, base=300.0, factor=4.0, scale=0.45, kv_from=1), "mlp": None},
        {"type": "attention", "mixer": O.attn(4, 4, 12, 20, 0, 0, scale=0.3), "mlp": O.moe(6, 2, 1, 1, 20, 2.5)},
        {"type": "attention", "mixer": O.attn(12, 3, 24, 16, 33, 24, base=5000.0, factor=1.0, scale=0.25, kv_from=0), "mlp": O.moe(8, 2, 4, 2, 16, 0.9, 24, 3.0)},
    ])


def cfg_wide():
    """sizes whose rows are multiples of 16 bytes (the vector paths) with a long window and 16 query heads per key head"""
    return O.make_config(width=128, vocab=260, eps=1e-6, layers=[
        {"type": "attention", "mixer": O.attn(16, 1, 32, 64, 150, 8, base=1e5, factor=2.5, scale=0.22), "mlp": O.moe(16, 4, 4, 2, 32, 1.5, 64, 2.0)},
        {"type": "attention", "mixer": O.attn(8, 2, 64, 128, 70, 64, base=1e4, factor=1.0, scale=0.11), "mlp": O.dense(160)},
        {"type": "attention", "mixer": O.attn(8, 4, 32, 256, 0, 32, base=777.0, factor=3.0, scale=0.2), "mlp": O.moe(4, 1, 2, 1, 48, 1.1)},
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
    # one, and nineteen in twenty have to be close
    d = logits - ref_logits
    e = np.sqrt((d ** 2).mean(-1)) / np.sqrt((ref_logits ** 2).mean())
    assert np.median(e) < 2e-2 and (e < 4e-2).mean() >= 0.95


def single_mechanism_model(mixer, mlp, width=64, vocab=50):
    return O.make_config(width=width, vocab=vocab, eps=1e-5, layers=[{"type": "attention", "mixer": mixer, "mlp": mlp}])


@pytest.mark.parametrize("name,mixer,mlp", [
    ("rotation_full_head", O.attn(4, 2, 16, 16, 0, 16, base=50.0, factor=1.0, scale=0.25), None),
    ("rotation_part_scaled", O.attn(4, 2, 16, 16, 0, 6, base=9.0, factor=7.0, scale=0.25), None),
    ("no_rotation", O.attn(4, 2, 16, 16, 0, 0, scale=0.25), None),
    ("window_3", O.attn(4, 4, 16, 8, 3, 4, scale=0.6), None),
    ("window_1_sees_itself_only", O.attn(2, 1, 8, 8, 1, 4, scale=0.6), None),
    ("dense_ffn", O.attn(2, 1, 8, 8, 0, 4, scale=0.3), O.dense(24)),
    ("experts_no_groups_no_shared", O.attn(2, 1, 8, 8, 0, 4, scale=0.3), O.moe(5, 2, 1, 1, 12, 0.8)),
    ("experts_groups_keep2_of_5", O.attn(2, 1, 8, 8, 0, 4, scale=0.3), O.moe(20, 3, 5, 2, 12, 1.7, 20, 0.6)),
    ("experts_top_equals_kept", O.attn(2, 1, 8, 8, 0, 4, scale=0.3), O.moe(8, 4, 2, 1, 12, 5.0, 8, 5.0)),
    # shapes of the matrix-instruction attention: sixteen tokens of one head per workgroup; two batches of sixteen heads on one key head; wide values
    ("one_head_per_key_head_window_9", O.attn(4, 4, 32, 16, 9, 8, scale=0.4), None),
    ("thirty_two_heads_on_one_key_head", O.attn(32, 1, 32, 16, 11, 32, base=77.0, scale=0.4), None),
    ("values_wider_than_keys", O.attn(8, 2, 32, 128, 0, 16, scale=0.3), None),
])
def test_each_mechanism_alone(name, mixer, mlp):
    cfg = single_mechanism_model(mixer, mlp)
    W = O.random_weights(cfg, 5, sink_range=(0.5, 3.0))      # sinks large enough that leaving them out moves the output by tens of percent
    toks = tokens(cfg, 40, 6)
    ref_logits, ref_streams = O.forward(cfg, W, toks)
    eng = engine(cfg, W)
    eng.store.set_capture(True)
    logits, _ = eng.step([("a", toks, list(range(40)))])
    assert rel(eng.store.read_capture(40)[0], ref_streams[0]) < 2e-4, name
    assert rel(logits, ref_logits) < 2e-4, name


def test_sink_matters_and_clamps_bite():
    """the oracle itself: dropping the sink, or the expert clamps, changes its output far beyond the tolerance the store is held to -- so the store
    tests above do see these mechanisms"""
    cfg = single_mechanism_model(O.attn(2, 1, 8, 8, 0, 4, scale=0.3), O.moe(5, 2, 1, 1, 12, 0.8))
    W = O.random_weights(cfg, 5, sink_range=(0.5, 3.0)); toks = tokens(cfg, 20, 6)
    a, _ = O.forward(cfg, W, toks)
    W2 = dict(W); W2["l0.mix.sink"] = np.full_like(W["l0.mix.sink"], -60.0)
    b, _ = O.forward(cfg, W2, toks)
    assert rel(b, a) > 5e-2
    cfg2 = json.loads(json.dumps(cfg)); cfg2["layers"][0]["mlp"]["expert"]["limit"] = 50.0
    c, _ = O.forward(cfg2, W, toks)
    assert rel(c, a) > 1e-2


def peaked_model(window, dim=32, width=64, vocab=40):
    """attention that finds ONE key: the query projection is steered so that the query of token 1 equals the key of token 0 (before the rotation of
    four coordinates); with a score scale of 1.5 that key scores about 1.5 * dim against O(sqrt(dim)) for any other, the query's own included --
    whether token 0 is inside the window decides the output at a token 1"""
    cfg = O.make_config(width=width, vocab=vocab, eps=1e-5, layers=[
        {"type": "attention", "mixer": O.attn(2, 1, dim, 16, window, 4, base=1e4, factor=1.0, scale=1.5), "mlp": None}])
    W = O.random_weights(cfg, 11, sink_range=(0.0, 0.1))
    h = O.layer_norm(W["embed"].astype(np.float64), W["l0.norm1"], W["l0.norm1.b"], 1e-5)
    steer = (W["l0.mix.k"].astype(np.float64) @ np.outer(h[0], h[1])) / (h[1] @ h[1])
    W["l0.mix.q"] = (0.3 * W["l0.mix.q"] + np.concatenate([steer, steer], 0)).astype(np.float32)
    return cfg, W


def needle_sequence(vocab, n, needle_at, query_at, seed):
    """random tokens 2.., token 0 (the needle) once, token 1 (the query) once"""
    t = [int(x) for x in np.random.default_rng(seed).integers(2, vocab, n)]
    t[needle_at] = 0; t[query_at] = 1
    return t


@pytest.mark.parametrize("window,dist", [(40, 39), (40, 40), (65, 64), (65, 65), (300, 299), (300, 300), (0, 500)])
def test_key_just_inside_and_just_outside_the_window_prompt_and_decode(window, dist):
    cfg, W = peaked_model(window)
    n = 520 if dist >= 299 else 200
    qpos = n - 3
    toks = needle_sequence(cfg["vocab"], n, qpos - dist, qpos, 13)
    ref, _ = O.forward(cfg, W, toks)
    if window:       # the oracle's own sensitivity: the needle one step across the edge changes the query's logits by tens of percent
        other = dist + 1 if dist < window else dist - 1
        ref2, _ = O.forward(cfg, W, needle_sequence(cfg["vocab"], n, qpos - other, qpos, 13))
        assert rel(ref2[qpos:qpos + 1], ref[qpos:qpos + 1]) > 0.2
    eng = engine(cfg, W, max_tokens=1088)
    want = [qpos - 1, qpos, qpos + 1]
    whole, _ = eng.step([("w", toks, want)])
    assert rel(whole, ref[want]) < 2e-4
    eng.finish("w")
    # the same positions decoded one token at a time after a prompt that ends before the query
    cut = qpos - 2
    eng.step([("d", toks[:cut], [])])
    got = []
    for p in range(cut, n):
        lg, _ = eng.step([("d", [toks[p]], [0])])
        got.append(lg[0])
    assert rel(np.stack(got), ref[cut:]) < 2e-4


def test_far_key_among_hundreds_across_pages():
    """full attention (no window): the one matching key sits 700 positions back, eleven pages away"""
    cfg, W = peaked_model(0)
    n = 780
    toks = needle_sequence(cfg["vocab"], n, 40, 740, 17)
    ref, _ = O.forward(cfg, W, toks)
    toks_moved = list(toks); toks_moved[40] = 5
    ref_moved, _ = O.forward(cfg, W, toks_moved)
    assert rel(ref_moved[740:741], ref[740:741]) > 0.2           # the far key carries the answer
    eng = engine(cfg, W, max_tokens=832)
    lg, _ = eng.step([("a", toks[:700], [])])
    lg, _ = eng.step([("a", toks[700:], [40])])
    assert rel(lg, ref[740:741]) < 2e-4


@pytest.mark.parametrize("needle,query", [(63, 64), (63, 127), (64, 128), (0, 1), (0, 63), (127, 128)])
def test_keys_at_page_borders(needle, query):
    cfg, W = peaked_model(0)
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
            assert np.median(e) < 2e-2 and (e < tol).mean() >= 0.95


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
    # 130 + 60 + 64 -> 3 + 1 + 1 pages: the pool is full
    a, _ = eng.step([(0, seqs[0], [129]), (1, seqs[1], [59]), (2, seqs[2], [63])])
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
    with pytest.raises(RuntimeError):                       # five requests need five slots
        for r in (10, 11, 12):
            eng.admit(r)


def test_long_decoding_through_pages_and_the_window():
    cfg = cfg_wide(); W = O.random_weights(cfg, 33); n = 330; toks = tokens(cfg, n, 34)
    ref, _ = O.forward(cfg, W, toks)
    eng = engine(cfg, W)
    eng.step([("a", toks[:20], [])])
    rows = []
    for p in range(20, n):
        lg, _ = eng.step([("a", [toks[p]], [0])])
        rows.append(lg[0])
    assert rel(np.stack(rows), ref[20:]) < 2e-4


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
    # top_k = 1 is greedy whatever the temperature
    g = eng.generate([p], 8)
    k1 = eng.generate([p], 8, temperature=1.3, top_k=1, seed=3)
    assert g == k1


def test_checkpoint_directory_command_line_and_trace_replay(tmp_path):
    cfg = cfg_varied(); W = O.random_weights(cfg, 39)
    model = str(tmp_path / "model"); O.write_checkpoint(model, cfg, W)
    from krasis_amd import model_registry as R
    assert R.model_family(R.read_config(model)) == "serve:Lomutar"
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
    with pytest.raises(ValueError):
        S.ServeStore(50, 32, [S.LayerSpec(heads=4, kv_heads=3, dim=8, vdim=8)])
    with pytest.raises(ValueError):
        S.ServeStore(50, 32, [S.LayerSpec(heads=4, kv_heads=2, dim=8, vdim=8, kv_from=0)])
    with pytest.raises(ValueError):
        S.ServeStore(50, 32, [S.LayerSpec(heads=4, kv_heads=2, dim=8, vdim=8, mlp_kind=S.MLP_MOE, experts=8, top=5, groups=4, keep=2, expert_ff=8)])
    st = S.ServeStore(50, 32, [S.LayerSpec(heads=4, kv_heads=2, dim=8, vdim=8)])
    with pytest.raises(RuntimeError):
        st.finalize()                                         # tensors missing
    with pytest.raises(ValueError):
        st.set_tensor(0, "q", np.zeros((5, 32), np.float32))  # wrong shape


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
    ref = O.forward(cfg, W, a[:130])[0]
    lg, _ = eng_g.step([("a", [a[130]], [0])])
    ref = O.forward(cfg, W, a[:131])[0]
    e = np.sqrt(((lg[0] - ref[130]) ** 2).mean()) / np.sqrt((ref ** 2).mean())
    assert e < 4e-2
