"""Host-side parts of the batched serving path that need no GPU: the config reader of the Lomutar design, the safetensors reader, the model
registry's choice by config.json, the scheduler's admission / portion / page accounting (against a stand-in engine), the trace replay loop."""
import json
import os

import numpy as np
import pytest

from krasis_amd import model_registry as R
from krasis_amd import serve_store as S
from tests import oracle_serve as O


def small_cfg():
    return O.make_config(width=48, vocab=37, eps=3e-6, layers=[
        {"type": "attention", "mixer": O.attn(6, 3, 8, 12, 9, 4, base=123.0, factor=3.0, scale=0.4), "mlp": O.dense(20)},
        {"type": "attention", "mixer": O.attn(6, 3, 8, 12, 0, 0, scale=0.2, kv_from=0), "mlp": O.moe(10, 3, 5, 2, 6, 1.5, 14, 0.5)},
        {"type": "attention", "mixer": O.attn(2, 2, 8, 8, 4, 8), "mlp": None},
    ])


def test_config_reader_takes_every_size_and_constant_from_config():
    spec = R.lomutar_spec(small_cfg())
    assert (spec.vocab, spec.width, spec.norm_kind, spec.norm_eps) == (37, 48, S.NORM_LAYER, 3e-6)
    a, b, c = spec.layers
    assert (a.heads, a.kv_heads, a.dim, a.vdim, a.window, a.rot_dims, a.rot_base, a.rot_factor, a.scale) == (6, 3, 8, 12, 9, 4, 123.0, 3.0, 0.4)
    assert a.rot_interleaved == 1 and a.qk_unit_norm == 1 and a.has_sink == 1 and a.kv_from == -1
    assert (a.mlp_kind, a.ff, a.dense_act) == (S.MLP_DENSE, 20, S.ACT_GELU_TANH)
    assert (b.kv_from, b.window, b.rot_dims) == (0, 0, 0)
    assert (b.mlp_kind, b.experts, b.top, b.groups, b.keep, b.renorm, b.expert_ff, b.expert_limit, b.shared_ff, b.shared_limit) == \
        (S.MLP_MOE, 10, 3, 5, 2, 0, 6, 1.5, 14, 0.5)
    assert b.expert_act == S.ACT_CLAMPED_SWIGLU and abs(b.expert_alpha - 1.702) < 1e-9
    assert c.mlp_kind == S.MLP_NONE and c.rot_factor == 1.0
    names = [n for _, _, _, n in spec.tensors(spec)]
    assert "l1.mix.k" not in names and "l1.mix.v" not in names and "l0.mix.k" in names          # a borrowed cache has no projections
    assert "l1.mlp.e9.down" in names and "l1.mlp.shared.up" in names and "l2.mlp.gate" not in names and "final.norm.b" in names
    with pytest.raises(ValueError):
        bad = small_cfg(); bad["layers"][0]["type"] = "recurrent"; R.lomutar_spec(bad)
    with pytest.raises(ValueError):
        bad = small_cfg(); bad["layers"][0]["mlp"]["kind"] = "other"; R.lomutar_spec(bad)


def test_registry_picks_the_family_by_config():
    assert "Lomutar" in R.architectures()
    assert R.model_family(small_cfg()) == "serve:Lomutar"
    assert R.model_family({"model_type": "qwen3_moe", "hidden_size": 8}) == "decode:qwen3_moe"
    with pytest.raises(ValueError):
        R.model_family({"architecture": "Unknown"})


def test_safetensors_reader_roundtrip(tmp_path):
    cfg = small_cfg(); W = O.random_weights(cfg, 0)
    O.write_checkpoint(str(tmp_path), cfg, W)
    f = R.SafetensorsFile(os.path.join(tmp_path, "model.safetensors"))
    assert sorted(f.names()) == sorted(W)
    for name in ("embed", "l1.mlp.router", "l0.mix.sink"):
        bits = f.get(name)
        assert bits.dtype == np.uint16 and bits.shape == W[name].shape
        assert np.array_equal((bits.astype(np.uint32) << 16).view(np.float32), W[name])       # the test weights are bf16 values
    with pytest.raises(IOError):
        f.get("missing")
    assert R.read_config(str(tmp_path))["width"] == 48


class FakeStore:
    page_tokens = 64

    def __init__(self, pool_tokens, max_slots):
        self.pool_tokens, self.max_slots = pool_tokens, max_slots


class FakeEngine:
    """stands in for BatchEngine: records the steps, answers argmax = (sum of the entry's tokens + cache length) % 11"""

    def __init__(self, pool_tokens=256, max_slots=2):
        self.store = FakeStore(pool_tokens, max_slots)
        self.len, self.steps, self.peak_live, self.peak_pages = {}, [], 0, 0

    def admit(self, rid):
        assert rid not in self.len and len(self.len) < self.store.max_slots
        self.len[rid] = 0

    def finish(self, rid):
        del self.len[rid]

    def step(self, entries, logits=True):
        out = []
        self.steps.append([(rid, len(t), list(w)) for rid, t, w in entries])
        for rid, toks, want in entries:
            self.len[rid] += len(toks)
            for _ in want:
                out.append((sum(toks) + self.len[rid]) % 11)
        self.peak_live = max(self.peak_live, len(self.len))
        self.peak_pages = max(self.peak_pages, sum((n + 63) // 64 for n in self.len.values()))
        assert self.peak_pages * 64 <= self.store.pool_tokens
        return None, np.asarray(out, np.int32)


def test_scheduler_batches_portions_and_respects_slots_pages_and_budget():
    from krasis_amd.scheduler import Scheduler
    eng = FakeEngine(pool_tokens=256, max_slots=2)
    sch = Scheduler(eng, token_budget=50)
    prompts = [list(range(1, 101)), [5, 6, 7], list(range(3, 70)), [9] * 120]
    ids = [sch.submit(p, 5) for p in prompts]
    sch.run()
    assert all(len(sch.result(i)) == 5 for i in ids) and not eng.len
    assert eng.peak_live <= 2
    for st in eng.steps:
        assert sum(n for _, n, _ in st) <= 50                                   # the token budget of a step
        assert len({rid for rid, _, _ in st}) == len(st)                       # a request appears once
    # a prompt longer than the budget was fed in portions, only the last portion asks for logits
    first = [(n, w) for st in eng.steps for rid, n, w in st if rid == ("sched", 0)][:2]
    assert first[0] == (50, []) and first[1][0] == 50 and first[1][1] == [49]
    # decoding requests ride along with another request's prompt portion
    assert any(len(st) == 2 and {n for _, n, _ in st} != {1} and 1 in {n for _, n, _ in st} for st in eng.steps)
    with pytest.raises(ValueError):
        sch.submit([1] * 300, 10)                                               # can never fit the pool
    # a stop id ends a request early
    eng2 = FakeEngine(); sch2 = Scheduler(eng2)
    r = sch2.submit([1, 2, 3], 20, stop_ids=[(6 + 3) % 11])
    sch2.run()
    assert sch2.result(r) == [(6 + 3) % 11]


def test_trace_replay_loop(tmp_path):
    from krasis_amd.__main__ import trace_replay

    class Eng(FakeEngine):
        def live(self):
            return list(self.len)

        def step(self, entries, logits=True):
            for rid, _, _ in entries:
                if rid not in self.len:
                    self.admit(rid)
            _, am = super().step(entries)
            return np.tile(am[:, None].astype(np.float32), (1, 3)), am
    eng = Eng(max_slots=4)
    lines = [json.dumps({"step": 0, "entries": [{"id": "a", "tokens": [1, 2, 3], "want": [0, 2]}, {"id": "b", "tokens": [4], "want": []}], "end": []}), "",
             json.dumps({"step": 1, "entries": [{"id": "b", "tokens": [5, 6], "want": []}], "end": ["a"]}),
             json.dumps({"step": 2, "entries": [{"id": "b", "tokens": [7], "want": [0]}], "end": ["b", "never-seen"]})]
    said = []
    trace_replay(eng, str(tmp_path), lines, said.append)
    assert said == ["done 0", "done 1", "done 2"] and not eng.len
    assert np.fromfile(os.path.join(tmp_path, "0.f32"), "<f4").shape == (6,) and not os.path.exists(os.path.join(tmp_path, "1.f32"))
    assert np.fromfile(os.path.join(tmp_path, "2.f32"), "<f4").shape == (3,)
