"""Host side of the layer-list models, no GPU: config.json -> layer structs and weight slots, the safetensors reader, the registry,
the block engine's state slots and streamed prompts, and the oracle's own invariants (a recurrence fed in portions equals the
recurrence fed whole; the window and the sink behave as written)."""
import ctypes
import json
import struct

import numpy as np
import pytest

from oracle import hybrid as H


def _cfg():
    att = {"dim": 24, "heads": 4, "kv_heads": 2, "vdim": 40, "scale": 0.3, "mask": {"size": 37},
           "rot": {"base": 3000.0, "dims": 12, "scaling": {"factor": 8.0, "low": 1.0, "high": 2.0, "original": 64}}}
    right = {"conv": 3, "dim": 20, "heads": 4, "kv_heads": 2, "vdim": 24, "_a_rank": 5, "_g_rank": 3}
    mlp = {"ff": 72, "kind": "dense", "limit": 1.25}
    return {"architecture": "Sogodra", "norm": {"eps": 1e-5}, "vocab": 97, "width": 56,
            "layers": [{"type": "mingru", "mixer": {"width": 50}, "mlp": mlp},
                       {"type": "parallel", "mixer": {"left": att, "right": right, "left_scale": 0.7, "right_scale": 1.3}, "mlp": None},
                       {"type": "delta", "mixer": {"conv": 5, "dim": 16, "heads": 3, "kv_heads": 3, "vdim": 48}, "mlp": mlp}]}


def test_spec_reads_every_size_from_config_and_shapes(lib):
    from candle_vllm_amd import hybrid_model as hm
    cfg = _cfg()
    W = H.random_sogodra(np.random.default_rng(0), cfg)
    spec = hm.SogodraSpec(cfg, {k: v.shape for k, v in W.items()})
    g, p, d = spec.layers
    assert (g.mixer, g.g_width, g.mlp_kind, g.mlp_ff) == (hm.MIX_MINGRU, 50, 1, 72) and abs(g.mlp_limit - 1.25) < 1e-7
    assert (p.mixer, p.a_heads, p.a_kv_heads, p.a_dim, p.a_vdim, p.a_window, p.a_rot_dims, p.a_has_sink, p.a_qk_norm) == \
        (hm.MIX_PARALLEL, 4, 2, 24, 40, 37, 12, 1, 1)
    assert (p.d_heads, p.d_kv_heads, p.d_dim, p.d_vdim, p.d_conv, p.d_decay_channels, p.d_a_rank, p.d_gate, p.d_g_rank, p.mlp_kind) == \
        (4, 2, 20, 24, 3, 1, 5, hm.GATE_SIGMOID_LR, 3, 0)
    assert abs(p.a_out_scale - 0.7) < 1e-6 and abs(p.d_out_scale - 1.3) < 1e-6
    assert (d.mixer, d.d_heads, d.d_kv_heads, d.d_conv, d.d_decay_channels, d.d_gate) == (hm.MIX_DELTA, 3, 3, 5, 0, hm.GATE_SILU)
    offs = (ctypes.c_int32 * 9)()
    rows = lib.mi355_hybrid_in_proj_rows(ctypes.byref(p), offs)
    aq, ak, av = 4 * 24, 2 * 24, 2 * 40
    dq, dv = 2 * 20, 4 * 24
    assert list(offs) == [0, aq, aq + ak, aq + ak + av, aq + ak + av + dq, aq + ak + av + 2 * dq, aq + ak + av + 2 * dq + dv,
                          aq + ak + av + 2 * dq + dv + 4, aq + ak + av + 2 * dq + dv + 4 + 5]
    assert rows == offs[8] + 3
    assert lib.mi355_hybrid_in_proj_rows(ctypes.byref(g), offs) == 150 and list(offs)[:4] == [0, 50, 100, -1]
    # the tensors behind the concatenated slots, in the order of the rows
    assert spec.slots[1][hm.HW_IN_PROJ] == ["l1.mix.left.q", "l1.mix.left.k", "l1.mix.left.v", "l1.mix.right.q", "l1.mix.right.k",
                                            "l1.mix.right.v", "l1.mix.right.b", "l1.mix.right.a1", "l1.mix.right.g1"]
    assert spec.slots[2][hm.HW_IN_PROJ][-2:] == ["l2.mix.a", "l2.mix.g"]
    with pytest.raises(ValueError):
        hm.SogodraSpec({**cfg, "layers": [{"type": "conv", "mixer": {}, "mlp": None}]}, {})


def test_absent_parts_of_a_config_are_absent(lib):
    from candle_vllm_amd import hybrid_model as hm
    cfg = _cfg()
    left = cfg["layers"][1]["mixer"]["left"]
    del left["mask"], left["rot"]
    left["_sink"], left["_qk_norm"] = False, False
    W = H.random_sogodra(np.random.default_rng(0), cfg)
    p = hm.SogodraSpec(cfg, {k: v.shape for k, v in W.items()}).layers[1]
    assert (p.a_window, p.a_rot_dims, p.a_has_sink, p.a_qk_norm) == (0, 0, 0, 0)


def test_safetensors_reader(tmp_path, lib):
    from candle_vllm_amd.hybrid_model import read_safetensors
    a = np.arange(12, dtype=np.uint16).reshape(3, 4)
    b = np.array([1, -2, 3], np.int32)
    head = json.dumps({"__metadata__": {"x": "y"}, "a": {"dtype": "BF16", "shape": [3, 4], "data_offsets": [0, 24]},
                       "b": {"dtype": "I32", "shape": [3], "data_offsets": [24, 36]}}).encode()
    f = tmp_path / "m.safetensors"
    f.write_bytes(struct.pack("<Q", len(head)) + head + a.tobytes() + b.tobytes())
    t = read_safetensors(str(f))
    assert t["a"][1] == (3, 4) and np.array_equal(t["a"][0], a.reshape(-1)) and np.array_equal(t["b"][0], b)


def test_registry_picks_the_host_layer_by_config(tmp_path, lib):
    from candle_vllm_amd import registry
    assert "Sogodra" in registry.registered() and "LlamaForCausalLM" in registry.registered()
    assert registry.architectures_of({"architecture": "Sogodra"}) == ["Sogodra"]
    (tmp_path / "config.json").write_text(json.dumps({"architectures": ["NoSuchModel"]}))
    with pytest.raises(ValueError):
        registry.load_model(str(tmp_path))


def test_llama_checkpoint_names_map_to_dense_slots(lib):
    from candle_vllm_amd import dense_loader as dl
    assert dl.slot_of("model.layers.11.self_attn.k_proj.weight") == (11, "wk")
    assert dl.slot_of("model.layers.0.mlp.up_proj.weight") == (0, "w3") and dl.slot_of("lm_head.weight") == (-1, "output")
    assert dl.slot_of("model.layers.3.self_attn.rotary_emb.inv_freq") is None
    d = dl.dims_from_config({"hidden_size": 64, "num_hidden_layers": 2, "num_attention_heads": 4, "num_key_value_heads": 2,
                             "intermediate_size": 128, "vocab_size": 99, "rms_norm_eps": 1e-6, "architectures": ["Qwen2ForCausalLM"]})
    assert (d.head_dim, d.n_kv_heads, d.qkv_bias, d.rms_eps) == (16, 2, True, 1e-6)


def test_state_slots_follow_the_sequences(lib):
    from candle_vllm_amd.block_engine import BlockEngine
    be = BlockEngine(4, 8, 0)
    be.state_init(2)
    a, b, c = be.new_sequence(1, [1, 2, 3]), be.new_sequence(2, [4]), be.new_sequence(3, [5] * 9)
    be.allocate([a], chunk=3)
    be.allocate([b], chunk=1)
    assert (be.state_acquire(a), be.state_acquire(b), be.state_acquire(a)) == (0, 1, 0)
    assert be.state_free_slots() == 0 and be.state_slot(c) == -1
    with pytest.raises(RuntimeError):
        be.state_acquire(c)
    be.free_sequence(a)                                   # pages and slot come back together
    assert be.state_free_slots() == 1 and be.get_num_free_blocks() == 7
    be.allocate([c], chunk=9)
    assert be.state_acquire(c) == 0 and be.get_num_free_blocks() == 4
    with pytest.raises(ValueError):
        be.state_init(3)                                  # not while sequences hold slots


def test_prompt_in_portions_takes_pages_for_what_it_holds(lib):
    from candle_vllm_amd.block_engine import BlockEngine
    be = BlockEngine(4, 3, 0)
    s = be.new_sequence(7, [1, 2, 3, 4])
    be.allocate([s], chunk=4)
    assert be.get_num_free_blocks() == 2                  # four tokens: exactly one page of four
    m = be.prepare_prompt([s])
    assert list(m["input_ids"]) == [1, 2, 3, 4] and list(m["context_lens"]) == [4]
    s.set_num_cached_tokens(4)
    s.extend_prompt([5, 6, 7, 8, 9])
    assert be.can_append_prefill_chunk_to_seq_group([s], 0)
    be.append_prefill_chunk_slots_to_seq_group([s], 0)
    assert be.get_num_free_blocks() == 0
    m = be.prepare_prompt([s])
    assert list(m["input_ids"]) == [5, 6, 7, 8, 9] and list(m["positions"]) == [4, 5, 6, 7, 8] and list(m["context_lens"]) == [9]
    assert list(m["cu_seqlens_q"]) == [0, 5]
    bt = be.block_table(s)
    assert list(m["slot_mapping"]) == [bt[1] * 4 + i for i in range(4)] + [bt[2] * 4]
    s.set_num_cached_tokens(9)
    s.extend_prompt([1, 2, 3, 4])                          # 13 tokens need a fourth page, and the pool has three
    assert not be.can_append_prefill_chunk_to_seq_group([s], 0)


# ---- the oracle's own invariants
def test_oracle_recurrences_in_portions_equal_whole():
    rng = np.random.default_rng(3)
    T, G, Hh, d, vd = 19, 2, 4, 6, 5
    q, k = H.unit_heads(rng.standard_normal((T, G, d)), 1e-6), H.unit_heads(rng.standard_normal((T, G, d)), 1e-6)
    v, beta, g = rng.standard_normal((T, Hh, vd)), H.sigmoid(rng.standard_normal((T, Hh))), H.sigmoid(rng.standard_normal((T, Hh, d)))
    o, S = H.gated_delta_rule(q, k, v, beta, g)
    o1, S1 = H.gated_delta_rule(q[:7], k[:7], v[:7], beta[:7], g[:7])
    o2, S2 = H.gated_delta_rule(q[7:], k[7:], v[7:], beta[7:], g[7:], S1)
    assert np.allclose(np.concatenate([o1, o2]), o) and np.allclose(S2, S)
    x, w = rng.standard_normal((T, 3)), rng.standard_normal((3, 4))
    y, _ = H.causal_conv_silu(x, w)
    ya, tail = H.causal_conv_silu(x[:2], w)
    yb, _ = H.causal_conv_silu(x[2:], w, tail)
    assert np.allclose(np.concatenate([ya, yb]), y)
    zs, us = rng.standard_normal((T, 3)), rng.standard_normal((T, 3))
    s, _ = H.min_gru(zs, us)
    sa, st = H.min_gru(zs[:5], us[:5])
    sb, _ = H.min_gru(zs[5:], us[5:], st)
    assert np.allclose(np.concatenate([sa, sb]), s)
    # the candidate is continuous at 0: u + 1/2 from above, sigmoid(u) from below
    c, _ = H.min_gru(np.full((1, 2), 50.0), np.array([[0.0, -1e-9]]))
    assert np.allclose(c, 0.5)


def test_oracle_window_and_sink():
    rng = np.random.default_rng(4)
    q, k, v = rng.standard_normal((1, 1, 4)), rng.standard_normal((10, 1, 4)), rng.standard_normal((10, 1, 3))
    full = H.window_sink_attention(q, k, v, [9], list(range(10)), 1.0)
    w3 = H.window_sink_attention(q, k, v, [9], list(range(10)), 1.0, window=3)
    ref3 = H.window_sink_attention(q, k[7:], v[7:], [2], [0, 1, 2], 1.0)
    assert np.allclose(w3, ref3) and not np.allclose(w3, full)
    big = H.window_sink_attention(q, k, v, [9], list(range(10)), 1.0, sink=np.array([50.0]))
    assert np.abs(big).max() < 1e-6                        # a huge sink takes all the weight and has no value
    none = H.window_sink_attention(q, k, v, [9], list(range(10)), 1.0, sink=np.array([-50.0]))
    assert np.allclose(none, full)
    f = H.rotary_frequencies(100.0, 8, (4.0, 1.0, 4.0, 64.0))
    f0 = H.rotary_frequencies(100.0, 8)
    wl = 2 * np.pi / f0
    assert all((a == b) if l < 16 else (abs(a - b / 4) < 1e-15 if l > 64 else b / 4 < a < b) for a, b, l in zip(f, f0, wl))
