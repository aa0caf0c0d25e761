"""The Vivazen mechanisms of the layer-list host layer (include/mi355_hybrid.h) against the float64 oracle of oracle/vivazen.py:
every new mechanism alone through its C entry point (group norm behind the residual sum, gelu gate/up, per-head batched products,
yarn tables and interleaved rotation, latent attention in its absorbed form over shared key/value page rows, the convolution in
front of attention, whole-projection norms, capped scores and mixed head weights), then whole models through the step engine --
whole prompts against token-by-token decoding, portions down to two tokens, unequal batches against each request alone, pages and
slots that are freed and used again, dominant keys just inside / outside the window and hundreds of tokens back, the first tokens,
long decoding, sizes that are 1 or equal, layers that run on another layer's weights -- and greedy generation through run_engine
and the scheduler.  Configurations and weights are made here."""
import ctypes
import math

import numpy as np
import pytest

torch = pytest.importorskip("torch")

from oracle import hybrid as H                          # noqa: E402
from oracle import vivazen as V                         # noqa: E402

pytestmark = pytest.mark.gpu
F32, BF16 = 0, 2


def _gpu():
    if not torch.cuda.is_available():
        pytest.fail("GPU tests need a visible MI355X")


def _st():
    return torch.cuda.current_stream().cuda_stream


def dev(a, dt=np.float32):
    return torch.from_numpy(np.ascontiguousarray(np.asarray(a).astype(dt))).cuda()


def bits(a):
    u = np.ascontiguousarray(a, np.float32).view(np.uint32)
    return ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)


def dev_dt(a, dtype):
    return dev(a) if dtype == F32 else torch.from_numpy(bits(a).view(np.int16)).cuda()


def host_dt(t, dtype):
    if dtype == F32:
        return t.cpu().numpy().astype(np.float64)
    u = t.cpu().numpy().view(np.uint16).astype(np.uint32) << 16
    return u.view(np.float32).astype(np.float64)


_KEEP = []


def P(a, dt=np.float32):
    t = dev(a, dt)
    _KEEP.append(t)
    return t.data_ptr()


def ok(rc):
    assert rc == 0, rc
    torch.cuda.synchronize()
    _KEEP.clear()


def f32(a):
    return np.asarray(a, np.float32).astype(np.float64)


# ------------------------------------------------------------------------------------------------------------ mechanisms alone
@pytest.mark.parametrize("T,W,groups,alpha", [(5, 200, 4, 3.0), (3, 63, 7, 0.5), (2, 1024, 1, 1.0), (1, 6, 6, 2.0)])
def test_resid_group_norm_gather_and_gelu_glu(lib, T, W, groups, alpha):
    _gpu()
    rng = np.random.default_rng(T + W)
    x, y, w = f32(rng.standard_normal((T, W))), f32(3 * rng.standard_normal((T, W + 4))), f32(rng.standard_normal(W))
    dx, dy, dw = dev(x), dev(y), dev(w)
    xc = torch.zeros((T, W), dtype=torch.int16, device="cuda")
    ok(lib.mi355_hyb_resid_norm(dx.data_ptr(), xc.data_ptr(), dy.data_ptr(), W + 4, dw.data_ptr(), T, W, groups, alpha, 1e-5, _st()))
    want = V.group_rms_norm(alpha * x + y[:, :W], w, 1e-5, groups)
    assert np.abs(dx.cpu().numpy() - want).max() < 1e-5 * max(1.0, np.abs(want).max())
    assert np.abs(host_dt(xc, BF16) - want).max() < 1e-2 * max(1.0, np.abs(want).max())
    rows = [T - 1, 0]
    for dt in (F32, BF16):
        out = torch.zeros((2, W), dtype=torch.float32 if dt == F32 else torch.int16, device="cuda")
        ok(lib.mi355_hyb_gather_group_norm(out.data_ptr(), dt, dx.data_ptr(), P(rows, np.int32), dw.data_ptr(), 2, W, groups, 1e-5, _st()))
        w2 = V.group_rms_norm(f32(dx.cpu().numpy())[rows], w, 1e-5, groups)
        assert np.abs(host_dt(out, dt) - w2).max() < (1e-5 if dt == F32 else 1e-2) * max(1.0, np.abs(w2).max())
    ff = 77
    gu = f32(2 * rng.standard_normal((T, 2 * ff)))
    out = torch.zeros((T, ff), device="cuda")
    ok(lib.mi355_hyb_gelu_glu(out.data_ptr(), F32, P(gu), T, ff, _st()))
    assert np.abs(out.cpu().numpy() - V.gelu_glu(gu[:, :ff], gu[:, ff:])).max() < 3e-6


@pytest.mark.parametrize("dtype,a_f32", [(F32, True), (BF16, True), (BF16, False)])
@pytest.mark.parametrize("T,n,k,heads", [(1, 24, 16, 3), (9, 64, 48, 2), (20, 40, 64, 5), (70, 33, 24, 4), (150, 128, 64, 2)])
def test_linear_batched_per_head(lib, dtype, a_f32, T, n, k, heads):
    """head h: out[:, h] = a[:, h] . w[h]^T with the operands' heads side by side in wider rows"""
    _gpu()
    rng = np.random.default_rng(T + n + k)
    pad = 8
    a = H.bf16_round(rng.standard_normal((T, heads * k + pad)))
    w = H.bf16_round(rng.standard_normal((heads, n, k)))
    a_dt = F32 if a_f32 else BF16
    out = torch.full((T, heads * n + 3), 7.0, device="cuda")
    da, dw = dev_dt(a, a_dt), dev_dt(w, dtype)
    ok(lib.mi355_hyb_linear_batched(out.data_ptr(), heads * n + 3, n, da.data_ptr(), a_dt, heads * k + pad, k, dw.data_ptr(), n * k, T, n, k,
                                    heads, dtype, _st()))
    got = out.cpu().numpy().astype(np.float64)
    for h in range(heads):
        want = a[:, h * k:(h + 1) * k] @ w[h].T
        assert np.abs(got[:, h * n:(h + 1) * n] - want).max() <= 2e-5 * math.sqrt(k) * max(1.0, np.abs(want).max())
    assert np.all(got[:, heads * n:] == 7.0)


def _tables(lib, dims, n_pos, base, scaling):
    """the framework's f64 table builder with the design's scaling"""
    from candle_vllm_amd.hybrid_model import VivazenSpec
    rs = VivazenSpec.rope_scaling({"dims": dims, "base": base, "scaling": scaling})
    cos, sin = np.zeros((n_pos, dims // 2), np.float32), np.zeros((n_pos, dims // 2), np.float32)
    assert lib.mi355_rope_tables_f64(cos.ctypes.data, sin.ctypes.data, dims, n_pos, float(base), ctypes.byref(rs), n_pos, n_pos) == 0
    return cos, sin


@pytest.mark.parametrize("dims,base,scaling", [(16, 20000.0, {"factor": 6.0, "fast": 16.0, "original": 1024, "slow": 1.5}),
                                               (10, 300.0, {"factor": 0.5, "fast": 3.0, "original": 48, "slow": 0.25}),       # a factor below 1: amplitude below 1
                                               (8, 100.0, {"factor": 2.5, "fast": 4.0, "original": 64, "slow": 0.5}),
                                               (32, 1e6, {"factor": 16.0, "fast": 8.0, "original": 512, "slow": 2.0}),
                                               (2, 10.0, {"factor": 3.0, "fast": 32.0, "original": 32, "slow": 1.0}),
                                               (12, 777.0, None)])
def test_yarn_tables(lib, dims, base, scaling):
    f, amp = V.yarn_frequencies(base, dims, scaling)
    cos, sin = _tables(lib, dims, 300, base, scaling)
    ang = np.arange(300)[:, None] * f[None]
    assert np.abs(cos - np.cos(ang) * amp).max() < 2e-7 * amp and np.abs(sin - np.sin(ang) * amp).max() < 2e-7 * amp
    if scaling:
        plain, _ = V.yarn_frequencies(base, dims, None)
        lo, hi = sorted((1.0, 1.0 / scaling["factor"]))
        assert (amp > 1.0) == (scaling["factor"] > 1.0) and np.all(f <= plain * hi + 1e-18) and np.all(f >= plain * lo - 1e-18)


@pytest.mark.parametrize("dtype", [F32, BF16])
@pytest.mark.parametrize("Hh,d,r,rank,rot", [(4, 24, 16, 40, 16), (2, 8, 12, 10, 8), (1, 16, 2, 3, 2), (3, 32, 8, 64, 0)])
def test_latent_prepare_norm_rotation_pages(lib, dtype, Hh, d, r, rank, rot):
    """the page row [normed latent | rotated shared key part] and the query rows [absorbed part | rotated part]; interleaved pairs,
    only the first `rot` of the r dimensions turn, positions far from 0"""
    _gpu()
    rng = np.random.default_rng(Hh + d + r)
    T, eps, n_slots = 7, 1e-3, 40
    ldp = Hh * (d + r) + rank + r + 5
    proj = f32(rng.standard_normal((T, ldp)))
    q_abs = f32(rng.standard_normal((T, Hh, rank)))
    cw = f32(1 + 0.2 * rng.standard_normal(rank))
    pos = np.array([0, 1, 2, 50, 51, 199, 7])
    slots = rng.permutation(n_slots)[:T]
    sc = {"factor": 3.0, "fast": 16.0, "original": 48, "slow": 1.0}
    q_off, c_off = 2, 2 + Hh * (d + r)
    q_out = torch.zeros((T, Hh, rank + r), dtype=torch.float32 if dtype == F32 else torch.int16, device="cuda")
    pages = torch.zeros((n_slots, rank + r), dtype=q_out.dtype, device="cuda")
    cos, sin = _tables(lib, rot, 256, 500.0, sc) if rot else (np.zeros((1, 1), np.float32),) * 2
    ok(lib.mi355_hyb_latent_prepare(q_out.data_ptr(), pages.data_ptr(), P(proj), ldp, q_off, c_off, P(q_abs), P(cw), P(cos), P(sin),
                                    P(pos, np.int64), P(slots, np.int64), T, Hh, d, r, rank, rot, 1, eps, dtype, _st()))
    f, amp = V.yarn_frequencies(500.0, rot, sc) if rot else (np.zeros(0), 1.0)
    dkv = proj[:, c_off:c_off + rank + r]
    lat = V.unit_rms(dkv[:, :rank], eps) * cw
    kr = V.rotate_pairs(dkv[:, rank:], pos, f, amp)
    q = proj[:, q_off:q_off + Hh * (d + r)].reshape(T, Hh, d + r)
    qr = V.rotate_pairs(q[:, :, d:], pos, f, amp)
    tol = 3e-6 if dtype == F32 else 1.2e-2
    got_p, got_q = host_dt(pages, dtype), host_dt(q_out, dtype)
    assert np.abs(got_p[slots, :rank] - lat).max() < tol * max(1, np.abs(lat).max())
    assert np.abs(got_p[slots, rank:] - kr).max() < tol * max(1, np.abs(kr).max())
    assert np.abs(got_q[:, :, :rank] - q_abs).max() < tol * max(1, np.abs(q_abs).max())
    assert np.abs(got_q[:, :, rank:] - qr).max() < tol * max(1, np.abs(qr).max())
    untouched = np.setdiff1d(np.arange(n_slots), slots)
    assert np.all(got_p[untouched] == 0)


@pytest.mark.parametrize("dtype", [F32, BF16])
@pytest.mark.parametrize("Hh,G,d,vd", [(4, 2, 24, 40), (2, 2, 8, 8), (3, 1, 16, 130), (1, 1, 4, 2)])
def test_attn_prepare_whole_projection_norms(lib, dtype, Hh, G, d, vd):
    _gpu()
    rng = np.random.default_rng(Hh + d)
    T, eps, n_slots = 6, 1e-3, 30
    C = (Hh + G) * d + G * vd
    src = f32(2 * rng.standard_normal((T, C + 3)))
    qw, kw = f32(1 + 0.3 * rng.standard_normal(Hh * d)), f32(1 + 0.3 * rng.standard_normal(G * d))
    slots = rng.permutation(n_slots)[:T]
    tdt = torch.float32 if dtype == F32 else torch.int16
    q_out = torch.zeros((T, Hh * d), dtype=tdt, device="cuda")
    kp, vp = torch.zeros((n_slots, G * d), dtype=tdt, device="cuda"), torch.zeros((n_slots, G, vd), dtype=tdt, device="cuda")
    ok(lib.mi355_hyb_attn_prepare_whole(q_out.data_ptr(), kp.data_ptr(), vp.data_ptr(), P(src), C + 3, 1, 1 + Hh * d, 1 + (Hh + G) * d, P(qw), P(kw),
                                        P(slots, np.int64), T, Hh, G, d, vd, 1, eps, dtype, _st()))
    q = V.unit_rms(src[:, 1:1 + Hh * d], eps) * qw
    k = V.unit_rms(src[:, 1 + Hh * d:1 + (Hh + G) * d], eps) * kw
    v = V.unit_rms(src[:, 1 + (Hh + G) * d:1 + C].reshape(T, G, vd), eps)
    tol = 3e-6 if dtype == F32 else 1.2e-2
    assert np.abs(host_dt(q_out, dtype) - q).max() < tol * max(1, np.abs(q).max())
    assert np.abs(host_dt(kp, dtype)[slots] - k).max() < tol * max(1, np.abs(k).max())
    assert np.abs(host_dt(vp, dtype)[slots] - v).max() < tol * max(1, np.abs(v).max())


@pytest.mark.parametrize("taps", [1, 3, 4])
def test_conv_without_activation_portions_and_state(lib, taps):
    """the convolution in portions of 1, 2, ... tokens continues from the slot's tail; a sequence that starts at 0 ignores stale state"""
    _gpu()
    rng = np.random.default_rng(taps)
    T, C, ldp, off, n_slots = 23, 37, 50, 6, 3
    proj, w = f32(rng.standard_normal((T, ldp))), f32(rng.standard_normal((C, taps)))
    want, _ = V.causal_conv(proj[:, off:off + C], w)
    stride = C * max(taps - 1, 1) + 5
    state = dev(rng.standard_normal((n_slots, stride)))                    # stale values everywhere
    lo, got = 0, []
    for n in (1, 2, 1, 7, 12):
        seq = torch.zeros(n, dtype=torch.int32, device="cuda")
        out = torch.zeros((n, C), device="cuda")
        def args():                                                         # fresh uploads for every launch: ok() lets the last ones go
            return P([lo + n], np.int32), P([0, n], np.int32), P([1], np.int32)
        ok(lib.mi355_hyb_conv(out.data_ptr(), P(proj[lo:lo + n]), ldp, off, P(w), state.data_ptr(), stride, *args(), seq.data_ptr(), 1, n, C,
                              taps, 0, _st()))
        ok(lib.mi355_hyb_conv_state_update(state.data_ptr(), stride, P(proj[lo:lo + n]), ldp, off, *args(), 1, C, taps, _st()))
        got.append(out.cpu().numpy())
        lo += n
    assert np.abs(np.concatenate(got) - want).max() < 1e-5


def _scatter(rows, bs, rng, n_blocks, free):
    """rows [Tk, width] of one sequence -> (block table, slots); takes pages from `free`"""
    nb = -(-rows.shape[0] // bs)
    table = [free.pop() for _ in range(nb)]
    slots = np.array([table[j // bs] * bs + j % bs for j in range(rows.shape[0])])
    return table, slots


@pytest.mark.parametrize("dtype", [F32, BF16])
@pytest.mark.parametrize("Hh,d,r,rank,vd,window,bs,big", [(4, 24, 16, 40, 32, 20, 16, False), (2, 8, 4, 10, 6, 0, 8, False),
                                                          (1, 16, 8, 24, 16, 1, 4, False), (3, 16, 2, 3, 5, 50, 32, False),
                                                          # prompt-sized steps; bf16 pages with a 64-wide row: the matrix-core kernel
                                                          (4, 32, 16, 48, 24, 100, 16, True), (2, 16, 32, 96, 64, 0, 64, True)])
def test_latent_attention_absorbed_over_shared_rows(lib, dtype, Hh, d, r, rank, vd, window, bs, big):
    """query [W_uk^T q | rotated part] against page rows [latent | rotated key part] that also serve as the values, then W_uv per
    head: equals the oracle that builds every head's keys and values from the latents.  Two unequal sequences in shuffled pages; a
    dominant key is placed just inside the window of the last query and just outside the window of the one before it"""
    _gpu()
    rng = np.random.default_rng(Hh * 100 + d + window)
    lens, news = ([300, 213], [170, 213]) if big else ([150, 37], [9, 37])
    n_blocks, dq = 64, rank + r
    pages = H.bf16_round(rng.standard_normal((n_blocks * bs, dq)))
    free = list(rng.permutation(n_blocks))
    uk, uv = H.bf16_round(rng.standard_normal((Hh * d, rank)) / math.sqrt(rank)), H.bf16_round(rng.standard_normal((Hh * vd, rank)) / math.sqrt(rank))
    sink = f32(rng.standard_normal(Hh))
    scale = 1.0 / math.sqrt(d + r)
    want, qs, tabs = [], [], []
    for L, n_new in zip(lens, news):
        c, kr = H.bf16_round(rng.standard_normal((L, rank))), H.bf16_round(rng.standard_normal((L, r)))
        qp, qr = H.bf16_round(rng.standard_normal((n_new, Hh, d))), H.bf16_round(rng.standard_normal((n_new, Hh, r)))
        q_pos = list(range(L - n_new, L))
        if window > 1 and L > window + 2:
            for a, off in ((n_new - 1, window - 1), (n_new - 2, window)):
                kr[q_pos[a] - off] = H.bf16_round(6.0 * qr[a, 0] * math.sqrt(d + r) / max(1e-6, np.dot(qr[a, 0], qr[a, 0]) ** 0.5))
        q_abs = np.stack([qp[:, h] @ uk[h * d:(h + 1) * d] for h in range(Hh)], axis=1)          # [n_new, H, rank]
        table, slots = _scatter(c, bs, rng, n_blocks, free)
        pages[slots] = np.concatenate([c, kr], axis=1)
        tabs.append(table)
        if dtype == BF16:
            # 16-bit operands: the reference is taken on the rounded absorbed query itself (scores q_abs . c + qr . kr, values = the
            # latents, then W_uv); that this form equals the per-head keys and values is what the f32 run shows
            q_abs = H.bf16_round(q_abs)
            vis = V.visible_mask(q_pos, range(L), window)
            o = np.zeros((n_new, Hh, vd))
            for h in range(Hh):
                s = (q_abs[:, h] @ c.T + qr[:, h] @ kr.T) * scale
                o[:, h] = (V.softmax_weights(s, vis, sink[h]) @ c) @ uv[h * vd:(h + 1) * vd].T
            want.append(o)
        else:
            want.append(V.latent_attention(qp, qr, c, kr, uk, uv, q_pos, list(range(L)), scale, window, sink))
        qs.append(np.concatenate([q_abs, qr], axis=2))
    T = sum(news)
    mb = max(len(t) for t in tabs)
    bt = np.zeros((2, mb), np.uint32)
    for i, t in enumerate(tabs):
        bt[i, :len(t)] = t
    cu = np.array([0, news[0], T], np.uint32)
    seq = torch.zeros(T, dtype=torch.int32, device="cuda")
    ok(lib.mi355_hyb_token_seq(seq.data_ptr(), P(cu, np.uint32), 2, _st()))
    dq_t, dp = dev_dt(np.concatenate(qs), dtype), dev_dt(pages, dtype)
    att = torch.zeros((T, Hh * rank), dtype=torch.float32 if dtype == F32 else torch.int16, device="cuda")
    ok(lib.mi355_hyb_window_attention_ex(att.data_ptr(), dtype, Hh * rank, 0, dq_t.data_ptr(), dp.data_ptr(), dp.data_ptr(), P(bt, np.uint32),
                                         P(lens, np.uint32), P(cu, np.uint32), seq.data_ptr(), P(sink), 2, T, Hh, 1, dq, rank, bs, mb, window,
                                         scale, 1.0, dq, dq, 0.0, 0, dtype, _st()))
    out = torch.zeros((T, Hh * vd), device="cuda")
    duv = dev_dt(uv, dtype)
    ok(lib.mi355_hyb_linear_batched(out.data_ptr(), Hh * vd, vd, att.data_ptr(), dtype, Hh * rank, rank, duv.data_ptr(), vd * rank, T, vd, rank,
                                    Hh, dtype, _st()))
    got = out.cpu().numpy().reshape(T, Hh, vd)
    wantc = np.concatenate(want)
    assert np.abs(got - wantc).max() < (2e-5 if dtype == F32 else 3e-2) * max(1.0, np.abs(wantc).max())


@pytest.mark.parametrize("dtype", [F32, BF16])
@pytest.mark.parametrize("Hh,G,d,vd,cap,bs,big", [(4, 2, 24, 40, 5.0, 16, False), (3, 3, 8, 8, 0.0, 8, False), (2, 1, 16, 130, 1.0, 32, False),
                                                  (1, 1, 4, 2, 50.0, 4, False),
                                                  (4, 2, 64, 48, 3.0, 16, True), (6, 3, 32, 16, 30.0, 64, True)])
def test_capped_scores_and_mixed_head_weights(lib, dtype, Hh, G, d, vd, cap, bs, big):
    """every head's weights against the values of every key/value head, then the mix of those outputs = the oracle that mixes the
    heads' softmax weights before the value product; the cap changes the scores (the first query is scaled so that tanh saturates)"""
    _gpu()
    rng = np.random.default_rng(Hh * 10 + d + int(cap))
    lens, news = ([300, 213], [170, 213]) if big else ([90, 37], [9, 37])
    n_blocks = 64
    kp, vp = H.bf16_round(rng.standard_normal((n_blocks * bs, G, d))), H.bf16_round(rng.standard_normal((n_blocks * bs, G, vd)))
    free = list(rng.permutation(n_blocks))
    talk = f32(np.eye(Hh) * 0.6 + 0.4 * rng.standard_normal((Hh, Hh)))
    scale = 1.3 / math.sqrt(d)
    want, qs, tabs = [], [], []
    for L, n_new in zip(lens, news):
        k, v = H.bf16_round(rng.standard_normal((L, G, d))), H.bf16_round(rng.standard_normal((L, G, vd)))
        q = H.bf16_round(rng.standard_normal((n_new, Hh, d)) * np.where(np.arange(n_new) % 3 == 0, 4.0, 1.0)[:, None, None])
        table, slots = _scatter(k, bs, rng, n_blocks, free)
        kp[slots], vp[slots] = k, v
        qs.append(q); tabs.append(table)
        want.append(V.mixed_head_attention(q, k, v, list(range(L - n_new, L)), list(range(L)), scale, cap, talk))
        if 0 < cap <= 5:
            assert np.abs(want[-1] - V.mixed_head_attention(q, k, v, list(range(L - n_new, L)), list(range(L)), scale, 0.0, talk)).max() > 1e-2
    T = sum(news)
    mb = max(len(t) for t in tabs)
    bt = np.zeros((2, mb), np.uint32)
    for i, t in enumerate(tabs):
        bt[i, :len(t)] = t
    cu = np.array([0, news[0], T], np.uint32)
    seq = torch.zeros(T, dtype=torch.int32, device="cuda")
    ok(lib.mi355_hyb_token_seq(seq.data_ptr(), P(cu, np.uint32), 2, _st()))
    dq_t, dk, dv = dev_dt(np.concatenate(qs), dtype), dev_dt(kp, dtype), dev_dt(vp, dtype)
    a = torch.zeros((T, Hh * G * vd), device="cuda")
    ok(lib.mi355_hyb_window_attention_ex(a.data_ptr(), F32, Hh * G * vd, 0, dq_t.data_ptr(), dk.data_ptr(), dv.data_ptr(), P(bt, np.uint32),
                                         P(lens, np.uint32), P(cu, np.uint32), seq.data_ptr(), None, 2, T, Hh, G, d, vd, bs, mb, 0, scale, 1.0,
                                         0, 0, cap, 1, dtype, _st()))
    out = torch.zeros((T, Hh * vd), device="cuda")
    ok(lib.mi355_hyb_head_mix(out.data_ptr(), F32, a.data_ptr(), P(talk), T, Hh, G, vd, _st()))
    wantc = np.concatenate(want).reshape(T, Hh * vd)
    assert np.abs(out.cpu().numpy() - wantc).max() < (2e-5 if dtype == F32 else 2e-2) * max(1.0, np.abs(wantc).max())


def test_head_gate(lib):
    _gpu()
    rng = np.random.default_rng(3)
    T, Hh, vd, ldg = 5, 3, 10, 9
    x, g = f32(rng.standard_normal((T, Hh * vd))), f32(2 * rng.standard_normal((T, ldg)))
    out = torch.zeros((T, Hh * vd), device="cuda")
    ok(lib.mi355_hyb_head_gate(out.data_ptr(), F32, P(x), P(g), ldg, T, Hh, vd, _st()))
    want = x.reshape(T, Hh, vd) * H.sigmoid(g[:, :Hh])[:, :, None]
    assert np.abs(out.cpu().numpy().reshape(T, Hh, vd) - want).max() < 2e-6


# ------------------------------------------------------------------------------------------------------------ whole models
def small_config(variant=0):
    rot = {"base": 3000.0, "dims": 12, "scaling": {"factor": 8.0, "fast": 6.0, "original": 40, "slow": 0.5}}
    lat = {"dim": 24, "heads": 3, "kv_rank": 20, "rot_dim": 12, "vdim": 10, "scale": 0.25, "mask": {"size": 37}, "rot": rot}
    att = {"conv": 4, "dim": 8, "heads": 6, "kv_heads": 2, "scale": 0.4, "softcap": 4.0, "vdim": 14}
    mlp = {"ff": 72, "kind": "dense"}
    layers = [{"type": "attention", "mixer": att, "mlp": mlp},
              {"type": "latent_attention", "mixer": lat, "mlp": mlp, "weights_of": 3},       # runs on a LATER layer's tensors
              {"type": "attention", "mixer": dict(att, conv=2, heads=2, softcap=30.0), "mlp": None},
              {"type": "latent_attention", "mixer": lat, "mlp": mlp},
              {"type": "latent_attention", "mixer": dict(lat, mask={"size": 9}, rot=dict(rot, dims=4)), "mlp": None},
              {"type": "attention", "mixer": att, "mlp": mlp, "weights_of": 0}]
    cfg = {"architecture": "Vivazen", "layers": layers, "norm": {"eps": 1e-5, "groups": 7}, "postln_alpha": 2.0, "vocab": 97, "width": 56}
    if variant == 1:                # values that may hide a fault when they are 1 or equal: one head, one tap, window 1, one group
        lat1 = {"dim": 8, "heads": 1, "kv_rank": 8, "rot_dim": 8, "vdim": 8, "scale": 0.5, "mask": {"size": 1}, "rot": {"base": 100.0, "dims": 8}}
        att1 = {"conv": 1, "dim": 8, "heads": 1, "kv_heads": 1, "scale": 1.0, "softcap": 1.0, "vdim": 8}
        layers = [{"type": "latent_attention", "mixer": lat1, "mlp": None},
                  {"type": "attention", "mixer": att1, "mlp": {"ff": 8, "kind": "dense"}},
                  {"type": "latent_attention", "mixer": dict(lat1, heads=2, mask=None, rot_dim=2, rot={"base": 10.0, "dims": 2}), "mlp": None},
                  {"type": "attention", "mixer": dict(att1, heads=4, kv_heads=4, conv=3, vdim=1), "mlp": None}]
        cfg = {"architecture": "Vivazen", "layers": layers, "norm": {"eps": 1e-3, "groups": 1}, "postln_alpha": 1.0, "vocab": 33, "width": 40}
    if variant == 2:                # sizes that take the matrix-core attention in bf16 prompts: 64-wide latent rows, 32-wide heads
        lat2 = {"dim": 16, "heads": 4, "kv_rank": 48, "rot_dim": 16, "vdim": 24, "scale": 0.2, "mask": {"size": 70},
                "rot": {"base": 2e4, "dims": 16, "scaling": {"factor": 5.0, "fast": 20.0, "original": 128, "slow": 2.0}}}
        att2 = {"conv": 3, "dim": 32, "heads": 4, "kv_heads": 2, "scale": 0.2, "softcap": 20.0, "vdim": 16}
        layers = [{"type": "latent_attention", "mixer": lat2, "mlp": mlp}, {"type": "attention", "mixer": att2, "mlp": mlp},
                  {"type": "latent_attention", "mixer": lat2, "mlp": mlp, "weights_of": 0}]
        cfg = {"architecture": "Vivazen", "layers": layers, "norm": {"eps": 1e-5, "groups": 2}, "postln_alpha": 1.5, "vocab": 120, "width": 64}
    return cfg


def build(cfg, dtype, seed=0, block_size=16, state_slots=4):
    from candle_vllm_amd.hybrid_model import HybridModel, VivazenSpec
    rng = np.random.default_rng(seed)
    W = V.random_vivazen(rng, cfg)
    spec = VivazenSpec(cfg, {k: v.shape for k, v in W.items()})
    m = HybridModel(spec, dtype=dtype, block_size=block_size, state_slots=state_slots)
    m.load_state_dict_f32(W)
    return m, W


def row_err(a, b):
    d = a - b
    d = d - d.mean(-1, keepdims=True)
    return np.sqrt((d * d).mean(-1)).max() / max(1e-9, np.sqrt((b * b).mean()))


TOL = {"float32": 3e-5, "bfloat16": 4e-2}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("variant", [0, 1, 2])
def test_model_whole_portions_decode_against_oracle(lib, dtype, variant):
    """one request whole, with the residual stream behind every layer; then the same tokens in portions of 2, 1, 17, ... tokens and
    token by token: every way must give the oracle's logits at every position (windows of 9, 37 and 70 pass over page borders of 16
    in the prompt and in decoding; the convolution's tail crosses every cut)"""
    _gpu()
    from candle_vllm_amd.step_engine import StepEngine
    cfg = small_config(variant)
    m, W = build(cfg, dtype, seed=variant)
    rng = np.random.default_rng(11)
    n = 150 if variant == 2 else 75
    toks = rng.integers(0, cfg["vocab"], n).tolist()
    want, want_trace = V.VivazenOracle(cfg, W).feed(toks)
    eng = StepEngine(m, 3 * 160)
    eng.feed("a", toks)
    got, tr = eng.step(["a"], [list(range(n))], trace=True)
    eng.finish("a")
    if dtype == "float32":
        assert np.abs(tr.cpu().numpy() - want_trace).max() < 1e-4 * np.abs(want_trace).max()
    tol = TOL[dtype]
    assert row_err(got.cpu().numpy(), want) < tol
    for cuts in ([2, 1, 17, 1, 1, 2, 30, 3, 18], [40] + [1] * 35, [1] * 20 + [55]):
        cuts = cuts + ([n - 75] if n > 75 else [])
        assert sum(cuts) == n
        lo, rows = 0, []
        for c in cuts:
            eng.feed("b", toks[lo:lo + c])
            rows.append(eng.step(["b"], [list(range(c))]).cpu().numpy())
            lo += c
        eng.finish("b")
        assert row_err(np.concatenate(rows), want) < tol, cuts
        assert eng.free_pages() == eng.num_blocks and eng.be.state_free_slots() == 4


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_unequal_batches_pages_and_slots_reused(lib, dtype):
    """five requests of unequal length through four slots and a pool that only fits them because pages come back: portions of some
    beside single tokens of others, a request that sits steps out, a late one that takes over a freed slot and freed pages --
    every logit must equal the request run alone in the oracle"""
    _gpu()
    from candle_vllm_amd.step_engine import StepEngine
    cfg = small_config(0)
    m, W = build(cfg, dtype, seed=3)
    rng = np.random.default_rng(21)
    lens = {"a": 70, "b": 33, "c": 5, "d": 48, "e": 41}
    toks = {r: rng.integers(0, cfg["vocab"], n).tolist() for r, n in lens.items()}
    want = {r: V.VivazenOracle(cfg, W).feed(toks[r])[0] for r in toks}
    eng = StepEngine(m, 80 + 48 + 16 + 48 + 0)                            # "e" (48 rounded) only fits after "b" and "c" have gone
    sched = [[("a", 2), ("b", 30)], [("a", 16), ("b", 1), ("c", 3)], [("a", 1), ("b", 1), ("c", 1), ("d", 47)], [("a", 30), ("c", 1), ("b", 1)],
             [("a", 1), ("d", 1), ("e", 2)], [("e", 38), ("a", 1)], [("a", 19), ("e", 1)]]
    at, got = {r: 0 for r in toks}, {r: [] for r in toks}
    for step in sched:
        ids, w = [], []
        for r, n in step:
            eng.feed(r, toks[r][at[r]:at[r] + n])
            at[r] += n
            ids.append(r); w.append(list(range(n)))
        out = eng.step(ids, w).cpu().numpy()
        lo = 0
        for r, n in step:
            got[r].append(out[lo:lo + n]); lo += n
        for r, _ in step:
            if at[r] == lens[r]:
                eng.finish(r)
    assert at == lens
    for r in toks:
        assert row_err(np.concatenate(got[r]), want[r]) < TOL[dtype], r
    assert eng.free_pages() == eng.num_blocks and eng.be.state_free_slots() == 4


def _sharp_latent_config(window):
    lat = {"dim": 4, "heads": 2, "kv_rank": 8, "rot_dim": 8, "vdim": 16, "scale": 8.0, "mask": {"size": window}, "rot": {"base": 10.0, "dims": 2}}
    return {"architecture": "Vivazen", "layers": [{"type": "latent_attention", "mixer": lat, "mlp": None}], "norm": {"eps": 1e-5, "groups": 2},
            "postln_alpha": 0.3, "vocab": 50, "width": 32}


def test_window_edge_and_sink_show_in_the_logits(lib):
    """a latent-attention model made sharp (large scale): the oracle's logits with the window one token shorter or longer, or with
    the sink left out, differ by far more than the tolerance, and the engine matches the right one, in the prompt and in decoding"""
    _gpu()
    from candle_vllm_amd.step_engine import StepEngine
    cfg = _sharp_latent_config(21)
    m, W = build(cfg, "float32", seed=8)
    W["l0.mix.sink"] = H.bf16_round(np.array([3.0, 4.0]))
    m.load_state_dict_f32(W)
    rng = np.random.default_rng(2)
    toks = rng.integers(0, 50, 60).tolist()
    want, _ = V.VivazenOracle(cfg, W).feed(toks)
    for delta in (-1, 1):
        other, _ = V.VivazenOracle(_sharp_latent_config(21 + delta), W).feed(toks)
        assert row_err(other[25:], want[25:]) > 100 * TOL["float32"]
    no_sink = {k: v for k, v in W.items() if not k.endswith("sink")}
    assert row_err(V.VivazenOracle(cfg, no_sink).feed(toks)[0], want) > 100 * TOL["float32"]
    eng = StepEngine(m, 64)
    eng.feed("a", toks[:40])
    rows = [eng.step(["a"], [list(range(40))]).cpu().numpy()]
    for t in toks[40:]:
        eng.feed("a", [t])
        rows.append(eng.step(["a"]).cpu().numpy())
    assert row_err(np.concatenate(rows), want) < TOL["float32"]


def test_far_key_hundreds_back_decides_a_late_token(lib):
    """causal attention without a window: one key 400 tokens back is made to match a late query (the token there is unique and the late
    token repeats it; keys are the queries' first head; the values differ because their convolution also reads the token before), so
    losing far pages changes the logits by far more than the tolerance.  Prompt in portions over many pages, then decoding"""
    _gpu()
    from candle_vllm_amd.step_engine import StepEngine
    att = {"conv": 2, "dim": 16, "heads": 2, "kv_heads": 1, "scale": 4.0, "softcap": 60.0, "vdim": 16}
    cfg = {"architecture": "Vivazen", "layers": [{"type": "attention", "mixer": att, "mlp": None}], "norm": {"eps": 1e-5, "groups": 1},
           "postln_alpha": 0.2, "vocab": 60, "width": 32}
    m, W = build(cfg, "float32", seed=9)
    W["l0.mix.k"] = W["l0.mix.q"][:16].copy()                              # key of a token = query of the same token (head 0)
    for n in ("q", "k"):                                                   # q and k read the current token only; the values also the one before
        W["l0.mix.%s.conv" % n][:, 0], W["l0.mix.%s.conv" % n][:, 1] = 0.0, 1.0
    W["l0.mix.q.norm"][:], W["l0.mix.k.norm"][:] = 1.0, 1.0
    m.load_state_dict_f32(W)
    rng = np.random.default_rng(5)
    toks = rng.integers(0, 59, 470).tolist()
    toks[30] = 59                                                          # the only 59 of the prompt ...
    toks[440] = 59                                                         # ... until position 440 asks for it again
    want, _ = V.VivazenOracle(cfg, W).feed(toks)
    cut = [t for i, t in enumerate(toks) if i != 30]                       # the same sequence without the far token
    other, _ = V.VivazenOracle(cfg, W).feed(cut)
    assert row_err(other[439:440], want[440:441]) > 100 * TOL["float32"]
    eng = StepEngine(m, 480)
    rows, lo = [], 0
    for c in [100, 3, 157, 2, 178]:
        eng.feed("a", toks[lo:lo + c])
        rows.append(eng.step(["a"], [list(range(c))]).cpu().numpy())
        lo += c
    for t in toks[440:]:
        eng.feed("a", [t])
        rows.append(eng.step(["a"]).cpu().numpy())
    assert row_err(np.concatenate(rows), want) < TOL["float32"]


def test_long_decoding_and_first_tokens(lib):
    _gpu()
    from candle_vllm_amd.step_engine import StepEngine
    cfg = small_config(0)
    m, W = build(cfg, "float32", seed=5)
    rng = np.random.default_rng(4)
    toks = rng.integers(0, cfg["vocab"], 200).tolist()
    want, _ = V.VivazenOracle(cfg, W).feed(toks)
    eng = StepEngine(m, 208)
    rows = []
    for t in toks:                                                          # from the very first token on, one at a time
        eng.feed("a", [t])
        rows.append(eng.step(["a"]).cpu().numpy())
    assert row_err(np.concatenate(rows)[:4], want[:4]) < TOL["float32"]
    assert row_err(np.concatenate(rows), want) < TOL["float32"]


def test_graph_replays_equal_eager_steps(lib):
    """decoding batches replay a captured hipGraph: every replay, with eager prompt portions of other requests between them, gives the
    eager step's logits bit for bit"""
    _gpu()
    from candle_vllm_amd.step_engine import StepEngine
    cfg = small_config(0)
    m, W = build(cfg, "bfloat16", seed=12)
    rng = np.random.default_rng(13)
    toks = {r: rng.integers(0, cfg["vocab"], 60).tolist() for r in "ab"}
    outs = {}
    for use_graph in (False, True):
        eng = StepEngine(m, 256)
        eng.use_graph = use_graph
        rows = []
        eng.feed("a", toks["a"][:20]); eng.feed("b", toks["b"][:33])
        rows.append(eng.step(["a", "b"]).cpu().numpy())
        for i in range(20):
            eng.feed("a", toks["a"][20 + i:21 + i]); eng.feed("b", toks["b"][33 + i:34 + i])
            rows.append(eng.step(["a", "b"]).cpu().numpy())
            if i == 7:
                eng.feed("c", toks["a"][:25]); rows.append(eng.step(["c"]).cpu().numpy()); eng.finish("c")
        eng.finish("a"); eng.finish("b")
        outs[use_graph] = np.concatenate(rows)
    assert np.array_equal(outs[False], outs[True])
    cap, rep = m.graph_stats()
    assert cap >= 1 and rep >= 15


@pytest.mark.parametrize("chunk", [0, 7])
def test_greedy_generation_through_scheduler(lib, chunk):
    """run_engine + the C++ scheduler (continuous batching, staggered arrivals, chunked prefill): every request generates exactly the
    tokens the oracle generates for it alone"""
    _gpu()
    from candle_vllm_amd import block_engine as be
    from candle_vllm_amd.engine import Request, run_engine
    cfg = small_config(0)
    m, W = build(cfg, "float32", seed=6)
    rng = np.random.default_rng(6)
    prompts = [rng.integers(0, cfg["vocab"], n).tolist() for n in (19, 3, 40, 11, 26)]
    n_new = 12
    want = []
    for p in prompts:
        o = V.VivazenOracle(cfg, W)
        lg, _ = o.feed(p)
        out = []
        for _ in range(n_new):
            t = int(lg[-1].argmax())
            out.append(t)
            lg, _ = o.feed([t])
        want.append(out)
    nblk = 24
    sched = be.Scheduler(16, nblk, 0, 4, 64, prefill_chunk_size=chunk)
    sched.block_engine.state_init(4)
    m.alloc_cache(nblk)
    reqs = [Request(i, p, n_new, arrival_step=2 * i) for i, p in enumerate(prompts)]
    stats = run_engine(m, sched, reqs, chunk=chunk)
    assert stats["finished"] == len(prompts)
    for r, w in zip(reqs, want):
        assert r.tokens == w, (r.id, r.tokens, w)
    assert sched.block_engine.state_free_slots() == 4


# ------------------------------------------------------------------------------------------------------------ random configurations
def random_config(rng):
    """sizes, head counts, layer order, windows and constants drawn at random (sizes of 8 .. 192 that are not all multiples of 16 or 32,
    one to eight heads, two to five taps, one to eight norm groups, layers that borrow an earlier layer's weights, layers without a
    feed-forward, rotation with and without scaling)"""
    width = int(rng.choice([96, 128, 192, 256, 320, 384]))
    groups = int(rng.choice([g for g in (1, 2, 3, 4, 6, 8) if width % g == 0]))

    def lat():
        d, r = int(rng.choice([16, 24, 32, 48, 64, 96, 128])), int(rng.choice([4, 8, 16, 32, 64]))
        m = {"dim": d, "heads": int(rng.choice([1, 2, 3, 4, 6, 8])), "kv_rank": int(rng.choice([16, 24, 32, 48, 64, 96, 128, 192])), "rot_dim": r,
             "vdim": int(rng.choice([8, 16, 24, 32, 48, 64, 96])), "scale": float((d + r) ** -0.5 * rng.uniform(0.7, 1.5)),
             "mask": {"size": int(rng.integers(5, 200))}, "rot": {"base": float(rng.choice([1e3, 1e4, 5e5, 123456.0])), "dims": r}}
        if rng.random() < 0.8:
            m["rot"]["scaling"] = {"factor": float(rng.choice([2.0, 3.5, 8.0, 16.0, 40.0])), "fast": float(rng.choice([8.0, 16.0, 32.0, 64.0])),
                                   "original": int(rng.choice([64, 256, 1024, 4096])), "slow": float(rng.choice([0.5, 1.0, 2.0]))}
        return m

    def att():
        G, d = int(rng.choice([1, 2, 3, 4])), int(rng.choice([16, 32, 40, 64, 80, 128]))
        return {"conv": int(rng.integers(2, 6)), "dim": d, "heads": G * int(rng.choice([1, 2, 3, 4])), "kv_heads": G,
                "scale": float(d ** -0.5 * rng.uniform(0.7, 1.5)), "softcap": float(rng.choice([5.0, 20.0, 50.0, 100.0])),
                "vdim": int(rng.choice([8, 16, 24, 48, 64, 80, 128]))}
    kinds = {"latent_attention": [lat() for _ in range(2)], "attention": [att() for _ in range(2)]}
    layers = []
    for _ in range(int(rng.integers(3, 9))):
        owners = [j for j, l in enumerate(layers) if "weights_of" not in l]
        if owners and rng.random() < 0.3:
            j = int(rng.choice(owners))
            layers.append(dict(layers[j], weights_of=j))
            continue
        t = str(rng.choice(["latent_attention", "attention"]))
        layers.append({"type": t, "mixer": kinds[t][int(rng.integers(0, 2))],
                       "mlp": {"ff": int(rng.choice([64, 160, 384, 512])), "kind": "dense"} if rng.random() < 0.85 else None})
    return {"architecture": "Vivazen", "layers": layers, "norm": {"eps": float(rng.choice([1e-5, 1e-6])), "groups": groups},
            "postln_alpha": float(rng.choice([2.0, 3.0, 4.0])), "vocab": int(rng.integers(50, 600)), "width": width}


@pytest.mark.gpu
@pytest.mark.parametrize("seed", [2, 11, 21])
def test_random_configurations_whole_and_mixed_schedules(lib, seed):
    """three unequal requests of a random configuration: each alone in one step, then together in a random schedule of portions (2, 3,
    17, 64, 65, 100 tokens; a request may sit a step out) that ends token by token -- on 64-token pages, in f32 and bf16"""
    _gpu()
    from candle_vllm_amd.step_engine import StepEngine
    rng = np.random.default_rng(seed)
    cfg = random_config(rng)
    W = V.random_vivazen(rng, cfg)
    lens = [int(rng.integers(150, 420)), int(rng.integers(1, 40)), int(rng.integers(60, 130))]
    toks = [rng.integers(0, cfg["vocab"], n).tolist() for n in lens]
    want = [V.VivazenOracle(cfg, W).feed(t)[0] for t in toks]
    from candle_vllm_amd.hybrid_model import HybridModel, VivazenSpec
    for dtype in ("float32", "bfloat16"):
        m = HybridModel(VivazenSpec(cfg, {k: v.shape for k, v in W.items()}), dtype=dtype, block_size=64, state_slots=4)
        m.load_state_dict_f32(W)
        eng = StepEngine(m, 64 * 12)
        for i, t in enumerate(toks):
            eng.feed("w", t)
            assert row_err(eng.step(["w"], [list(range(len(t)))]).cpu().numpy(), want[i]) < TOL[dtype], (dtype, "whole", i)
            eng.finish("w")
        at, got = [0, 0, 0], [[], [], []]
        while any(a < n for a, n in zip(at, lens)):
            ids, w, take = [], [], []
            for i in range(3):
                if at[i] >= lens[i] or rng.random() < 0.2:
                    continue
                left = lens[i] - at[i]
                c = 1 if left <= 20 else int(min(left - 20, rng.choice([2, 3, 17, 64, 65, 100])))
                eng.feed("r%d" % i, toks[i][at[i]:at[i] + c])
                ids.append("r%d" % i); w.append(list(range(c))); take.append((i, c))
                at[i] += c
            if not ids:
                continue
            out, lo = eng.step(ids, w).cpu().numpy(), 0
            for i, c in take:
                got[i].append(out[lo:lo + c]); lo += c
                if at[i] == lens[i]:
                    eng.finish("r%d" % i)
        for i in range(3):
            assert row_err(np.concatenate(got[i]), want[i]) < TOL[dtype], (dtype, "schedule", i)
        assert eng.free_pages() == eng.num_blocks and eng.be.state_free_slots() == 4
