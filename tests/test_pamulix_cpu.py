"""Host-side parts of the Pamulix design that need no GPU: its config reader (every size and constant from config.json, the constants the design fixes
from the code), its tensor names, the registry's choice, a checkpoint round trip, and the oracle's own rotation table."""
import math
import os

import numpy as np
import pytest

from krasis_amd import model_registry as R
from krasis_amd import serve_store as S
from tests import oracle_pamulix as O


def small_cfg():
    return O.make_config(width=48, vocab=37, eps=3e-6, residual_mult=0.3, layers=[
        O.layer(O.latent(3, 10, 6, 14, 20, 18, base=123.0, scaling=(5.0, 96, 12.0, 2.0), scale=0.4), O.moe(10, 3, 6)),
        O.layer(O.attn(6, 3, 8, 12, 9, v_mix=True, scale=0.2), None),
        O.layer(O.attn(2, 2, 8, 8, 0, scale=0.3), O.moe(4, 1, 5)),
        O.layer(O.attn(4, 2, 8, 18, 21, v_mix=True, scale=0.25), O.moe(7, 7, 9)),
        O.layer(O.latent(2, 4, 8, 4, 5, 6, base=10.0, scale=0.5), None),
    ])


def test_config_reader_takes_every_size_and_constant_from_config():
    spec = R.pamulix_spec(small_cfg())
    assert (spec.vocab, spec.width, spec.norm_kind, spec.norm_eps) == (37, 48, S.NORM_LAYER, 3e-6)
    assert (spec.block_kind, spec.pre_norm, spec.post_norm, spec.norm_bias) == (S.BLOCK_SEQUENTIAL, 0, 1, 0) and abs(spec.residual_mult - 0.3) < 1e-12
    a, b, c, d, e = spec.layers
    assert (a.mixer_kind, a.heads, a.kv_heads, a.dim, a.rot_dims, a.vdim, a.q_rank, a.kv_rank, a.scale) == (S.MIX_LATENT, 3, 1, 10, 6, 14, 20, 18, 0.4)
    assert (a.rot_scaling, a.rot_base, a.rot_factor, a.rot_original, a.rot_fast, a.rot_slow, a.rot_interleaved) == (S.ROT_BY_PARTS, 123.0, 5.0, 96.0, 12.0, 2.0, 1)
    assert (a.has_sink, a.dist_bias, a.chunk, a.window, a.v_mix, a.qk_unit_norm) == (S.SINK_NONE, 0, 0, 0, S.VMIX_NONE, S.QKNORM_NONE)
    assert (a.mlp_kind, a.experts, a.top, a.groups, a.keep, a.renorm, a.router_bias, a.expert_ff, a.expert_act, a.shared_ff) == (S.MLP_MOE, 10, 3, 1, 1, 1, 1, 6, S.ACT_SILU, 0)
    assert (b.mixer_kind, b.heads, b.kv_heads, b.dim, b.vdim, b.chunk, b.scale, b.rot_dims) == (S.MIX_ATTENTION, 6, 3, 8, 12, 9, 0.2, 0)
    assert (b.has_sink, b.dist_bias, b.dist_bias_exp, b.qk_unit_norm, b.mlp_kind) == (S.SINK_ZERO, 1, 8.0, S.QKNORM_WEIGHTED, S.MLP_NONE)
    # the first layer that mixes values keeps its own, the later ones blend; a layer that does not say so does neither
    assert (b.v_mix, c.v_mix, d.v_mix) == (S.VMIX_FIRST, S.VMIX_NONE, S.VMIX_BLEND)
    assert c.chunk == 0 and (c.top, d.top, d.experts) == (1, 7, 7)
    assert (e.rot_scaling, e.rot_factor, e.mlp_kind) == (S.ROT_LINEAR, 1.0, S.MLP_NONE)
    names = [n for _, _, _, n in spec.tensors(spec)]
    assert {"l0.mix.dq", "l0.mix.dq.norm", "l0.mix.uq", "l0.mix.dkv", "l0.mix.dkv.norm", "l0.mix.uk", "l0.mix.uv", "l0.mix.o", "l0.norm1", "l0.norm2"} <= set(names)
    assert "l0.mix.q" not in names and "l1.mix.q.norm" in names and "l1.mix.k.norm" in names
    assert "l1.mix.vmix" not in names and "l3.mix.vmix" in names and "l2.mix.vmix" not in names      # the first mixing layer's scalar is not used
    assert "l1.norm2" not in names and "l4.norm2" not in names and "l3.norm2" in names
    assert "l0.mlp.router.b" in names and "l3.mlp.e6.down" in names and "l3.mlp.e7.down" not in names
    assert "final.norm" in names and "final.norm.b" not in names
    W = O.random_weights(small_cfg(), 0)
    assert set(names) <= set(W)                                                   # every tensor the store asks for is one the checkpoint layout has
    with pytest.raises(ValueError):
        bad = small_cfg(); bad["layers"][0]["type"] = "recurrent"; R.pamulix_spec(bad)
    with pytest.raises(ValueError):
        bad = small_cfg(); bad["layers"][0]["mlp"]["kind"] = "dense"; R.pamulix_spec(bad)
    with pytest.raises(ValueError):
        bad = small_cfg(); bad["layers"][0]["mixer"]["rot"]["dims"] = 4; R.pamulix_spec(bad)


def test_registry_and_checkpoint_roundtrip(tmp_path):
    assert "Pamulix" in R.architectures() and "Lomutar" in R.architectures()
    cfg = small_cfg(); W = O.random_weights(cfg, 0)
    assert R.model_family(cfg) == "serve:Pamulix"
    O.write_checkpoint(str(tmp_path), cfg, W)
    f = R.SafetensorsFile(os.path.join(tmp_path, "model.safetensors"))
    assert sorted(f.names()) == sorted(W)
    lam = f.get("l3.mix.vmix")
    assert lam.shape == () and lam.dtype == np.uint16                              # a scalar tensor comes back as one value
    assert R.read_config(str(tmp_path))["residual_mult"] == 0.3


def test_oracle_rotation_table():
    """by-parts scaling: pairs below the ramp keep base^(-2i/dims), pairs above it are divided by the factor, cos and sin are stretched"""
    f, mult = O.yarn_table(32, 10000.0, 6.0, 1024, 16.0, 2.0)
    plain, one = O.plain_table(32, 10000.0)
    assert one == 1.0 and abs(mult - (0.1 * math.log(6.0) + 1.0)) < 1e-15
    lo = math.floor(32 * math.log(1024 / (2 * math.pi * 16.0)) / (2 * math.log(10000.0)))
    hi = math.ceil(32 * math.log(1024 / (2 * math.pi * 2.0)) / (2 * math.log(10000.0)))
    assert 0 < lo < hi < 16
    assert np.allclose(f[:lo + 1], plain[:lo + 1]) and np.allclose(f[hi:], plain[hi:] / 6.0)
    mid = (lo + hi) // 2
    assert plain[mid] / 6.0 < f[mid] < plain[mid]
    x = np.random.default_rng(0).standard_normal((5, 2, 40))
    y = O.rotate_pairs(x, np.arange(5), f, mult)
    assert np.array_equal(y[:, :, 32:], x[:, :, 32:]) and np.allclose(y[0, :, :32], x[0, :, :32] * mult)     # the tail passes; position 0 only stretches
    n0 = np.hypot(x[:, :, 0], x[:, :, 1]); n1 = np.hypot(y[:, :, 0], y[:, :, 1])
    assert np.allclose(n1, n0 * mult)
