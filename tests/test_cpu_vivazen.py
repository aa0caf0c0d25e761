"""Host side of the Vivazen design, no GPU: config.json -> layer structs and weight slots (every size from the config or a tensor's
shape, layers that run on another layer's tensors, absent parts), the registry, and the oracle's own invariants (portions equal the
whole; the absorbed form of latent attention equals per-head keys and values; mixing softmax weights equals mixing per-head outputs;
window, sink and cap behave as written)."""
import ctypes
import math

import numpy as np
import pytest

from oracle import hybrid as H
from oracle import vivazen as V


def _cfg():
    rot = {"base": 3000.0, "dims": 8, "scaling": {"factor": 8.0, "fast": 6.0, "original": 40, "slow": 0.5}}
    lat = {"dim": 24, "heads": 3, "kv_rank": 20, "rot_dim": 12, "vdim": 10, "scale": 0.25, "mask": {"size": 37}, "rot": rot}
    att = {"conv": 4, "dim": 8, "heads": 6, "kv_heads": 2, "scale": 0.4, "softcap": 4.0, "vdim": 14}
    mlp = {"ff": 72, "kind": "dense"}
    return {"architecture": "Vivazen", "norm": {"eps": 1e-5, "groups": 7}, "postln_alpha": 2.5, "vocab": 97, "width": 56,
            "layers": [{"type": "attention", "mixer": att, "mlp": mlp},
                       {"type": "latent_attention", "mixer": lat, "mlp": None},
                       {"type": "attention", "mixer": att, "mlp": mlp, "weights_of": 0},
                       {"type": "latent_attention", "mixer": lat, "mlp": None, "weights_of": 1}]}


def test_spec_reads_every_size_from_config_and_shapes(lib):
    from candle_vllm_amd import hybrid_model as hm
    cfg = _cfg()
    W = V.random_vivazen(np.random.default_rng(0), cfg)
    assert not any(k.startswith(("l2.", "l3.")) for k in W)                  # borrowed layers have no tensors
    spec = hm.VivazenSpec(cfg, {k: v.shape for k, v in W.items()})
    a, l, a2, l2 = spec.layers
    assert (spec.residual_form, spec.norm_groups) == (1, 7) and abs(spec.resid_alpha - 2.5) < 1e-7
    assert (a.mixer, a.a_heads, a.a_kv_heads, a.a_dim, a.a_vdim, a.a_conv, a.a_qk_norm, a.a_norm_whole, a.a_v_unit, a.a_talk, a.a_window,
            a.a_rot_dims, a.a_has_sink, a.mlp_kind, a.mlp_ff, a.share_with) == (hm.MIX_CONV_ATTENTION, 6, 2, 8, 14, 4, 1, 1, 1, 1, 0, 0, 0, 2, 72, 0)
    assert abs(a.a_softcap - 4.0) < 1e-7 and abs(a.a_scale - 0.4) < 1e-7
    assert (l.mixer, l.a_heads, l.a_kv_heads, l.a_dim, l.a_rot_dim, l.a_kv_rank, l.a_vdim, l.a_window, l.a_rot_dims, l.a_rot_interleaved,
            l.a_has_sink, l.a_head_gate, l.mlp_kind, l.share_with) == (hm.MIX_LATENT, 3, 1, 24, 12, 20, 10, 37, 8, 1, 1, 1, 0, 0)
    assert (a2.share_with, l2.share_with) == (1, 2) and spec.slots[2] == {} and spec.slots[3] == {} and spec.rope[3] is None
    offs = (ctypes.c_int32 * 9)()
    assert lib.mi355_hybrid_in_proj_rows(ctypes.byref(l), offs) == 3 * 36 + 32 + 3
    assert list(offs) == [0, 108, -1, -1, -1, -1, -1, -1, 140]
    assert lib.mi355_hybrid_in_proj_rows(ctypes.byref(a), offs) == 48 + 16 + 28 and list(offs)[:4] == [0, 48, 64, -1]
    assert spec.slots[1][hm.HW_IN_PROJ] == ["l1.mix.q", "l1.mix.dkv", "l1.mix.g"]
    assert spec.slots[0][hm.HW_A_CONV] == ["l0.mix.q.conv", "l0.mix.k.conv", "l0.mix.v.conv"]
    rs = spec.rope_scaling(cfg["layers"][1]["mixer"]["rot"])
    assert (rs.type, rs.factor, rs.beta_fast, rs.beta_slow, rs.original_max_position_embeddings) == (hm.ROPE_YARN, 8.0, 6.0, 0.5, 40.0)
    with pytest.raises(ValueError):
        hm.VivazenSpec({**cfg, "layers": [{"type": "delta", "mixer": dict(cfg["layers"][0]["mixer"]), "mlp": None}]}, {})
    with pytest.raises(ValueError):
        hm.VivazenSpec({**cfg, "layers": [dict(cfg["layers"][0], weights_of=0)]}, {})


def test_absent_parts_and_the_transposed_key_projection(lib):
    from candle_vllm_amd import hybrid_model as hm
    cfg = _cfg()
    lat = cfg["layers"][1]["mixer"]
    del lat["mask"], lat["rot"]["scaling"]
    cfg["norm"] = {"eps": 1e-3}
    W = V.random_vivazen(np.random.default_rng(0), cfg)
    del W["l1.mix.sink"], W["l1.mix.g"]
    spec = hm.VivazenSpec(cfg, {k: v.shape for k, v in W.items()})
    l = spec.layers[1]
    assert (l.a_window, l.a_has_sink, l.a_head_gate, spec.norm_groups) == (0, 0, 0, 1)
    assert spec.rope_scaling(lat["rot"]).type == hm.ROPE_DEFAULT
    (ukt,) = spec.slots[1][hm.HW_L_UKT]
    bits = {"l1.mix.uk": hm._bf16_bits(W["l1.mix.uk"])}
    got = ukt.bits(bits, {"l1.mix.uk": W["l1.mix.uk"].shape}).reshape(3, 20, 24)
    want = hm._bf16_bits(W["l1.mix.uk"]).reshape(3, 24, 20)
    for h in range(3):
        assert np.array_equal(got[h], want[h].T)


def test_registry_knows_the_design_and_its_component(lib):
    from candle_vllm_amd import registry
    assert "Vivazen" in registry.registered()
    assert registry.component_of({"architecture": "Vivazen"}) == "hybrid"
    assert registry.component_of({"architectures": ["LlamaForCausalLM"]}) is None


def test_host_layer_refuses_what_it_cannot_run(lib):
    from candle_vllm_amd import hybrid_model as hm
    cfg = _cfg()
    W = V.random_vivazen(np.random.default_rng(0), cfg)
    spec = hm.VivazenSpec(cfg, {k: v.shape for k, v in W.items()})
    n = len(spec.layers)
    arr = (hm.HybridLayer * n)(*spec.layers)
    c = hm.HybridConfig(width=56, vocab=97, n_layers=n, dtype=hm.DT_F32, block_size=16, state_slots=2, norm_eps=1e-5, unit_eps=1e-6,
                        residual_form=1, resid_alpha=2.5, norm_groups=7)
    h = lib.mi355_hybrid_create(ctypes.byref(c), arr)
    assert h
    lib.mi355_hybrid_destroy(h)
    c.norm_groups = 5                                                        # 56 is not a multiple of 5
    assert not lib.mi355_hybrid_create(ctypes.byref(c), arr)
    c.norm_groups = 7
    arr[2].share_with = 4                                                    # a lender that itself borrows
    assert not lib.mi355_hybrid_create(ctypes.byref(c), arr)
    arr[2].share_with = 2                                                    # a lender of another shape
    assert not lib.mi355_hybrid_create(ctypes.byref(c), arr)


# ------------------------------------------------------------------------------------------------------------ the oracle itself
def test_oracle_portions_equal_the_whole():
    cfg = _cfg()
    W = V.random_vivazen(np.random.default_rng(1), cfg)
    toks = np.random.default_rng(2).integers(0, 97, 50).tolist()
    whole, tr = V.VivazenOracle(cfg, W).feed(toks)
    o = V.VivazenOracle(cfg, W)
    parts = [o.feed(toks[lo:hi])[0] for lo, hi in ((0, 1), (1, 3), (3, 20), (20, 21), (21, 50))]
    assert np.abs(np.concatenate(parts) - whole).max() < 1e-9
    assert tr.shape == (4, 50, 56)
    # borrowed layers run: without them the logits differ
    short = {**cfg, "layers": cfg["layers"][:2]}
    assert np.abs(V.VivazenOracle(short, W).feed(toks)[0] - whole).max() > 1e-3


def test_oracle_group_norm_window_sink_cap_and_mixing():
    rng = np.random.default_rng(3)
    x, w = rng.standard_normal((4, 12)), rng.standard_normal(12)
    assert np.allclose(V.group_rms_norm(x, w, 1e-5, 1), H.rms_norm(x, w, 1e-5))
    g = V.group_rms_norm(x, np.ones(12), 0.0, 3)
    assert np.allclose((g.reshape(4, 3, 4) ** 2).mean(-1), 1.0)
    assert abs(V.gelu_tanh(np.array([1.0]))[0] - 0.841192) < 1e-5
    # window: exactly `size` keys are seen, itself included; the sink takes weight and has no value
    vis = V.visible_mask([10], range(11), 4)
    assert vis.sum() == 4 and vis[0, 10] and vis[0, 7] and not vis[0, 6]
    wts = V.softmax_weights(np.zeros((1, 3)), np.ones((1, 3), bool), sink=0.0)
    assert np.allclose(wts, 0.25)
    # identity mixing = plain grouped attention; the cap bounds the scores
    T, Hh, G, d, vd = 9, 4, 2, 6, 5
    q, k, v = rng.standard_normal((T, Hh, d)), rng.standard_normal((T, G, d)), rng.standard_normal((T, G, vd))
    pos = list(range(T))
    plain = V.mixed_head_attention(q, k, v, pos, pos, 0.5, 0.0, np.eye(Hh))
    ref = H.window_sink_attention(q, k, v, pos, pos, 0.5)
    assert np.allclose(plain, ref)
    talk = rng.standard_normal((Hh, Hh))
    # mixing the weights = mixing, per key/value head, the outputs of the unmixed weights
    a = np.zeros((T, Hh, G, vd))
    for c in range(G):
        a[:, :, c] = V.mixed_head_attention(q, k, np.repeat(v[:, c:c + 1], G, axis=1), pos, pos, 0.5, 2.0, np.eye(Hh))
    via_outputs = np.stack([sum(talk[h, g] * a[:, g, h // (Hh // G)] for g in range(Hh)) for h in range(Hh)], axis=1)
    assert np.allclose(via_outputs, V.mixed_head_attention(q, k, v, pos, pos, 0.5, 2.0, talk))
    big = V.mixed_head_attention(100 * q, k, v, pos, pos, 0.5, 1.0, np.eye(Hh))
    assert np.all(np.isfinite(big))


def test_oracle_latent_attention_equals_its_absorbed_form():
    rng = np.random.default_rng(4)
    T, Hh, d, r, rank, vd = 12, 3, 5, 4, 7, 6
    qp, qr = rng.standard_normal((T, Hh, d)), rng.standard_normal((T, Hh, r))
    c, kr = rng.standard_normal((T, rank)), rng.standard_normal((T, r))
    uk, uv, sink = rng.standard_normal((Hh * d, rank)), rng.standard_normal((Hh * vd, rank)), rng.standard_normal(Hh)
    pos = list(range(T))
    want = V.latent_attention(qp, qr, c, kr, uk, uv, pos, pos, 0.3, 5, sink)
    vis = V.visible_mask(pos, pos, 5)
    for h in range(Hh):
        q_abs = qp[:, h] @ uk[h * d:(h + 1) * d]
        s = (q_abs @ c.T + qr[:, h] @ kr.T) * 0.3
        o = (V.softmax_weights(s, vis, sink[h]) @ c) @ uv[h * vd:(h + 1) * vd].T
        assert np.allclose(o, want[:, h])
    f, amp = V.yarn_frequencies(50000.0, 16, {"factor": 4.0, "fast": 32.0, "original": 2048, "slow": 1.0})
    assert abs(amp - (0.1 * math.log(4.0) + 1)) < 1e-12 and abs(f[0] - 1.0) < 1e-12 and abs(f[-1] - 50000.0 ** (-14 / 16) / 4.0) < 1e-12
    x = rng.standard_normal((3, 2, 6))
    y = V.rotate_pairs(x, [0, 5, 9], np.array([0.7, 0.1]), 1.0)
    assert np.allclose(y[0], x[0]) and np.allclose(y[..., 4:], x[..., 4:])
    assert np.allclose((y[..., :4] ** 2).sum(-1), (x[..., :4] ** 2).sum(-1))
    assert np.allclose(y[1, 0, 0], x[1, 0, 0] * math.cos(3.5) - x[1, 0, 1] * math.sin(3.5))
