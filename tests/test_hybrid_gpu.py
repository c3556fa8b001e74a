"""Hybrid decoders (the Lozupel design) on the GPU against the plain float32 restatement in
oracle/lozupel_ref.py: every mechanism alone, then the whole model through the engine -- whole
prompts, token-by-token decoding, portions down to two tokens, mixed batches, reused pages and
state slots, window and page edges, other sizes -- and greedy generation through LLM.generate.
Small seeded configurations made here; float32 runs carry the sharp bars, bfloat16 a loose one."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

from oracle import lozupel_ref as R  # noqa: E402


def _left(heads, kv, dim, vdim, window, rot, base=10000.0, scale=0.2):
    return {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "mask": {"size": window},
            "rot": {"dims": rot, "base": base}, "scale": scale}


def _delta(heads, kv, dim, vdim, conv):
    return {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "conv": conv}


CONFIGS = {
    # loop from layer 0, three passes, grouped heads everywhere, partial rotation, vdim != dim
    "loop0": {"architecture": "Lozupel", "embedding": {"scale": 1.5}, "width": 96, "vocab": 160,
              "norm": {"eps": 1e-5}, "logit_softcap": 12.0, "loop": {"start": 0, "stop": 2, "times": 3},
              "layers": [{"type": "delta", "mixer": _delta(4, 2, 48, 40, 2), "mlp": {"kind": "dense", "ff": 136}},
                         {"type": "parallel", "mixer": {"left": _left(6, 2, 32, 48, 20, 16), "right": _delta(2, 1, 32, 24, 4)},
                          "mlp": None},
                         {"type": "parallel", "mixer": {"left": _left(4, 4, 16, 16, 7, 16, base=500.0, scale=0.25),
                                                        "right": _delta(3, 3, 64, 72, 3)},
                          "mlp": {"kind": "dense", "ff": 64}}]},
    # no loop, no soft cap, a window of one token, a convolution of one tap, wide heads
    "plain": {"architecture": "Lozupel", "embedding": {"scale": 1.0}, "width": 64, "vocab": 97,
              "norm": {"eps": 1e-6},
              "layers": [{"type": "parallel", "mixer": {"left": _left(2, 1, 128, 96, 1, 64), "right": _delta(1, 1, 128, 128, 1)},
                          "mlp": {"kind": "dense", "ff": 80}},
                         {"type": "delta", "mixer": _delta(2, 2, 16, 8, 5), "mlp": None},
                         {"type": "parallel", "mixer": {"left": _left(3, 3, 24, 40, 33, 8), "right": _delta(4, 2, 24, 16, 2)},
                          "mlp": None}]},
    # a loop in the middle that runs once, tail layers after it
    "tail": {"architecture": "Lozupel", "embedding": {"scale": 0.25}, "width": 128, "vocab": 200,
             "norm": {"eps": 1e-5}, "logit_softcap": 5.0, "loop": {"start": 1, "stop": 2, "times": 1},
             "layers": [{"type": "delta", "mixer": _delta(2, 2, 32, 32, 3), "mlp": None},
                        {"type": "parallel", "mixer": {"left": _left(4, 2, 32, 32, 17, 32), "right": _delta(2, 2, 32, 64, 3)},
                         "mlp": {"kind": "dense", "ff": 96}},
                        {"type": "delta", "mixer": _delta(4, 1, 64, 32, 4), "mlp": {"kind": "dense", "ff": 160}}]},
    # a width the weight-streaming GEMM's tiled form covers (decode-sized steps in 16 bits take it)
    "wide": {"architecture": "Lozupel", "embedding": {"scale": 1.0}, "width": 512, "vocab": 384,
             "norm": {"eps": 1e-6}, "logit_softcap": 20.0, "loop": {"start": 0, "stop": 2, "times": 2},
             "layers": [{"type": "parallel", "mixer": {"left": _left(8, 2, 64, 64, 24, 32), "right": _delta(4, 2, 64, 128, 4)},
                         "mlp": {"kind": "dense", "ff": 1024}},
                        {"type": "delta", "mixer": _delta(8, 4, 64, 64, 3), "mlp": {"kind": "dense", "ff": 512}}]},
}
_cache = {}


def _weights(name):
    if ("w", name) not in _cache:
        _cache[("w", name)] = R.random_state(CONFIGS[name], seed=len(name))
    return _cache[("w", name)]


def _engine(name, dtype="float32", pages=40, max_model_len=320):
    from mi355_decode.config import EngineArgs, ModelConfig
    from mi355_decode.llm import build_engine
    key = (name, dtype, pages, max_model_len)
    if key not in _cache:
        torch.backends.cuda.matmul.allow_tf32 = False
        _cache[key] = build_engine(EngineArgs(model=name, dtype=dtype, max_num_seqs=4, max_model_len=max_model_len,
                                              num_gpu_blocks_override=pages, gpu_memory_utilization=0.0,
                                              max_num_batched_tokens=1 << 20),
                                   state_dict=_weights(name), model_config=ModelConfig.from_dict(CONFIGS[name]))
    eng = _cache[key]
    assert not eng.seqs and eng.alloc.num_free == pages and eng.slots.num_free == 4
    return eng


def _tokens(name, n, seed):
    return np.random.default_rng(seed).integers(0, CONFIGS[name]["vocab"], n).tolist()


def _ref(name, toks):
    key = ("ref", name, tuple(toks))
    if key not in _cache:
        with torch.no_grad():
            _cache[key] = R.forward(_weights(name), CONFIGS[name], toks).numpy()
    return _cache[key]


def _close(got, want, tol=3e-4):
    scale = float(np.abs(want).max())
    err = float(np.abs(got - want).max())
    assert err <= tol * scale, f"max |diff| {err:.3e} on a scale of {scale:.3f}"


def _run_cuts(eng, rid, toks, cuts):
    """Feeds toks in portions `cuts` (the last portion takes the rest), all positions wanted."""
    rows, at = [], 0
    sizes = list(cuts)
    while at < len(toks):
        n = min(sizes.pop(0) if sizes else len(toks) - at, len(toks) - at)
        rows.append(eng.forced_step([(rid, toks[at:at + n], list(range(n)))], [rid] if at + n == len(toks) else []))
        at += n
    return np.concatenate(rows)


# ------------------------------------------------------------------------------------------ #
# mechanisms alone
# ------------------------------------------------------------------------------------------ #
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_norms_and_pointwise(dtype):
    from mi355_decode import ops
    g = torch.Generator().manual_seed(3)
    T, W = 7, 200
    tol = 1e-5 if dtype == torch.float32 else 1.2e-2
    x = torch.randn(T, W, generator=g) * 3
    add = torch.randn(T, W, generator=g).to(dtype)
    for wt in (torch.tensor([1.3]), torch.randn(W, generator=g)):
        wt = wt.to(dtype)
        resid = x.clone().cuda()
        out = ops.add_rms_norm_f32(resid, wt.cuda(), 1e-5, add=add.cuda())
        want = x + add.float()
        assert torch.equal(resid.cpu(), want)
        ref = R.vector_rms_norm(want, wt.float(), 1e-5)
        assert (out.float().cpu() - ref).abs().max() <= tol * ref.abs().max()
    xa, xb = torch.randn(T, W, generator=g).to(dtype), (torch.randn(T, W, generator=g) * 5).to(dtype)
    wa, wb = torch.randn(W, generator=g).to(dtype), torch.randn(W, generator=g).to(dtype)
    resid = x.clone().cuda()
    ops.rms_norm_mix_f32(resid, xa.cuda(), wa.cuda(), xb.cuda(), wb.cuda(), 1e-6, 0.5)
    ref = x + 0.5 * (R.vector_rms_norm(xa.float(), wa.float(), 1e-6) + R.vector_rms_norm(xb.float(), wb.float(), 1e-6))
    assert (resid.cpu() - ref).abs().max() <= 1e-5 * ref.abs().max()
    gu = (torch.randn(T, 2 * 72, generator=g) * 2).to(dtype)
    out = ops.gelu_tanh_and_mul(gu.cuda())
    ref = R.gelu_tanh(gu.float()[:, :72]) * gu.float()[:, 72:]
    assert (out.float().cpu() - ref).abs().max() <= tol * ref.abs().max()
    z = (torch.randn(5, 33, generator=g) * 20).to(dtype)
    ref = 7.0 * torch.tanh(z.float() / 7.0)
    assert (ops.softcap(z.clone().cuda(), 7.0).float().cpu() - ref).abs().max() <= tol * 7.0
    emb = torch.randn(50, 24, generator=g).to(dtype)
    ids = torch.tensor([3, 49, 0, 3])
    assert torch.equal(ops.embed_scale_f32(emb.cuda(), ids.cuda(), 0.75).cpu(), emb.float()[ids] * 0.75)
    resid = x.clone().cuda()
    ops.resid_add_f32(resid, other=x.cuda(), rows=add.cuda(), vec=wb[:W].cuda())
    assert torch.allclose(resid.cpu(), x + x + add.float() + wb.float(), atol=1e-5)
    for act, fn in ((ops.ACT_SILU, torch.nn.functional.silu), (ops.ACT_SIGMOID, torch.sigmoid)):
        o = torch.randn(T, 3, 40, generator=g)
        gate = torch.randn(T, 3 * 40 + 8, generator=g).to(dtype)
        hw = torch.randn(40, generator=g)
        out = ops.gated_head_rms_norm(o.cuda(), gate.cuda()[:, 8:], hw.cuda(), 1e-5, act)
        ref = (R.vector_rms_norm(o, hw, 1e-5) * fn(gate.float()[:, 8:]).view(T, 3, 40)).reshape(T, -1)
        assert (out.float().cpu() - ref).abs().max() <= tol * ref.abs().max()


def _paged(T, num_pages, seed):
    """A shuffled block table for one sequence of T tokens and its slot mapping."""
    order = np.random.default_rng(seed).permutation(num_pages)[: (T + 15) // 16].astype(np.int32)
    pos = np.arange(T)
    return order, order[pos // 16].astype(np.int64) * 16 + pos % 16


def _attend_in_cuts(q, k, v, cuts, H, G, d, dv, window, rot, temp, bias, gate, scale=0.3, base=100.0, tiled=False):
    """rope + store + attention over one sequence fed in portions; returns [T, H * dv] float32."""
    from mi355_decode import ops
    from mi355_decode.hybrid_runner import rotary_table
    T = q.shape[0]
    dt = q.dtype
    pages = 12
    table, slots = _paged(T, pages, 5)
    kc = torch.full((pages, G, 16, d), float("nan"), dtype=dt, device="cuda")
    vc = torch.full((pages, G, dv, 16), float("nan"), dtype=dt, device="cuda")
    bt = torch.zeros(1, pages, dtype=torch.int32)
    bt[0, : len(table)] = torch.from_numpy(table)
    cs = rotary_table(rot, base, pages * 16, "cuda")
    outs, at = [], 0
    for n in cuts:
        sl = slice(at, at + n)
        qq = q[sl].clone().cuda()
        pos = torch.arange(at, at + n, dtype=torch.int64, device="cuda")
        ops.rope_partial_kv_write(qq, k[sl].cuda(), v[sl].cuda(), cs, pos, torch.from_numpy(slots[sl]).cuda(), kc, vc,
                                  H, G, d, dv)
        outs.append(ops.sigmoid_window_attn(qq, kc, vc, bt.cuda(), torch.zeros(n, dtype=torch.int32, device="cuda"), pos,
                                            temp.cuda(), bias.cuda(), None if gate is None else gate[sl].cuda(), H,
                                            window, scale,
                                            tiles=torch.from_numpy(ops.query_tiles([0, n])).cuda() if tiled else None,
                                            # single rows: the window's keys spread over three workgroups
                                            partial=torch.empty(3 * H * dv, device="cuda") if tiled and n == 1 else None,
                                            num_splits=3 if tiled and n == 1 else 1).float().cpu())
        at += n
    assert at == T
    return torch.cat(outs)


@pytest.mark.parametrize("H,G,d,dv,window,rot", [(4, 2, 32, 48, 20, 16), (3, 3, 24, 130, 1, 0), (2, 1, 128, 64, 33, 128),
                                                 (8, 2, 64, 64, 200, 32)])
def test_window_attention_whole_portions_and_single_tokens(H, G, d, dv, window, rot):
    g = torch.Generator().manual_seed(H * 100 + d)
    T = 75
    q, k, v = torch.randn(T, H * d, generator=g), torch.randn(T, G * d, generator=g), torch.randn(T, G * dv, generator=g)
    temp, bias, gate = torch.rand(H, generator=g) + 0.5, torch.randn(H, generator=g) - 1.0, torch.randn(T, H, generator=g)
    pos = torch.arange(T)
    ref = R.sigmoid_window_attention(R.rotate_partial(q.view(T, H, d), pos, rot, 100.0),
                                     R.rotate_partial(k.view(T, G, d), pos, rot, 100.0), v.view(T, G, dv), window, 0.3,
                                     temp, bias) * torch.sigmoid(gate)[:, :, None]
    ref = ref.reshape(T, H * dv)
    for cuts in ([T], [1] * T, [2, 14, 1, 16, 17, 2, 23]):
        got = _attend_in_cuts(q, k, v, cuts, H, G, d, dv, window, rot, temp, bias, gate)
        assert (got - ref).abs().max() <= 2e-5 * ref.abs().max(), cuts


@pytest.mark.parametrize("H,G,d,dv,window,rot", [(4, 2, 32, 48, 20, 16), (2, 1, 128, 64, 33, 128), (8, 2, 64, 64, 200, 32),
                                                 (16, 1, 96, 16, 7, 64), (2, 1, 256, 256, 40, 64), (2, 2, 160, 144, 20, 32)])
def test_window_attention_on_the_matrix_cores(H, G, d, dv, window, rot):
    """The 16-row tile form (16-bit storage) against the restatement run on the same rounded inputs:
    whole prompt, uneven portions, single rows; unused page slots hold NaN and must not leak."""
    g = torch.Generator().manual_seed(H + d)
    T = 75
    bf = lambda t: t.to(torch.bfloat16)                                      # noqa: E731
    q, k, v = bf(torch.randn(T, H * d, generator=g)), bf(torch.randn(T, G * d, generator=g)), bf(torch.randn(T, G * dv, generator=g))
    temp, bias, gate = torch.rand(H, generator=g) + 0.5, torch.randn(H, generator=g) - 1.0, bf(torch.randn(T, H, generator=g))
    pos = torch.arange(T)
    qr = bf(R.rotate_partial(q.float().view(T, H, d), pos, rot, 100.0)).float()
    kr = bf(R.rotate_partial(k.float().view(T, G, d), pos, rot, 100.0)).float()
    ref = R.sigmoid_window_attention(qr, kr, v.float().view(T, G, dv), window, 0.3, temp, bias) \
        * torch.sigmoid(gate.float())[:, :, None]
    ref = ref.reshape(T, H * dv)
    for cuts in ([T], [5, 16, 1, 17, 33, 3], [1] * 20 + [55]):
        got = _attend_in_cuts(q, k, v, cuts, H, G, d, dv, window, rot, temp, bias, gate, tiled=True)
        assert torch.isfinite(got).all()
        assert (got - ref).abs().max() <= 1.5e-2 * ref.abs().max(), cuts


@pytest.mark.parametrize("window", [16, 17, 31, 48])
def test_window_edge_shows_with_one_loud_key(window):
    """One key far louder than the rest: the token window - 1 after it still hears it, the next one
    does not -- in a whole prompt and when the late tokens arrive one by one."""
    H = G = 1
    d = dv = 32
    T, j0 = 70, 5
    q = torch.zeros(T, d)
    q[:, 0] = 8.0
    k = torch.zeros(T, d)
    k[j0, 0] = 8.0
    v = torch.zeros(T, dv)
    v[j0, 3] = 1.0
    temp, bias = torch.ones(1), torch.full((1,), -30.0)          # every other key weighs sigmoid(-30)
    for cuts, dt in (([T], torch.float32), ([j0 + 2] + [1] * (T - j0 - 2), torch.float32), ([T], torch.bfloat16),
                     ([3, 40, T - 43], torch.bfloat16)):
        got = _attend_in_cuts(q.to(dt), k.to(dt), v.to(dt), cuts, H, G, d, dv, window, 0, temp, bias, None, scale=1.0,
                              tiled=dt == torch.bfloat16)
        inside, outside = j0 + window - 1, j0 + window
        assert got[inside, 3] > 0.99 and abs(got[outside, 3]) < 1e-6 and got[j0, 3] > 0.99 and got[j0 - 1, 3] == 0


def _delta_in_cuts(qkv, beta, decay, a_log, dt_bias, cuts, H, G, d, dv, per_channel, slot=2, slots=4, long_chunks=False):
    from mi355_decode import ops
    T = qkv.shape[0]
    state = torch.full((slots, H, d, dv), float("nan"), device="cuda")
    qk = G * d
    outs, at = [], 0
    for n in cuts:
        sl = slice(at, at + n)
        outs.append(ops.gated_delta_rule(qkv[sl].contiguous().cuda(), 0, qk, 2 * qk, beta[sl].cuda(), decay[sl].cuda(),
                                         a_log.cuda(), dt_bias.cuda(), state,
                                         torch.tensor([0, n], dtype=torch.int32, device="cuda"),
                                         torch.arange(at, at + n, dtype=torch.int64, device="cuda"),
                                         torch.tensor([slot], dtype=torch.int32, device="cuda"), H, G, d, dv,
                                         per_channel=per_channel, long_chunks=long_chunks and n > 1).cpu())
        at += n
    return torch.cat(outs)


def _delta_ref(qkv, beta, decay, a_log, dt_bias, H, G, d, dv, per_channel):
    T, qk = qkv.shape[0], G * d
    rep = H // G
    q = (R.unit(qkv[:, :qk].view(T, G, d)) * d ** -0.5).repeat_interleave(rep, dim=1)
    k = R.unit(qkv[:, qk:2 * qk].view(T, G, d)).repeat_interleave(rep, dim=1)
    v = qkv[:, 2 * qk:].view(T, H, dv)
    z = torch.nn.functional.softplus(decay + dt_bias)
    a = torch.exp(-torch.exp(a_log)[None, :, None] * z.view(T, H, d)) if per_channel else torch.exp(-torch.exp(a_log) * z)
    return R.gated_delta_rule(q, k, v, torch.sigmoid(beta), a)


@pytest.mark.parametrize("H,G,d,dv,per_channel", [(4, 2, 48, 40, False), (2, 1, 32, 24, True), (3, 3, 64, 72, True),
                                                  (1, 1, 128, 128, False), (2, 2, 16, 8, False), (2, 1, 200, 130, True)])
def test_delta_rule_whole_portions_and_single_tokens(H, G, d, dv, per_channel):
    g = torch.Generator().manual_seed(d + dv)
    T = 41
    qkv = torch.randn(T, 2 * G * d + H * dv, generator=g)
    beta = torch.randn(T, H, generator=g)
    decay = torch.randn(T, H * d if per_channel else H, generator=g)
    a_log, dt_bias = torch.randn(H, generator=g) * 0.5 - 1, torch.randn(decay.shape[1], generator=g) * 0.5
    ref = _delta_ref(qkv, beta, decay, a_log, dt_bias, H, G, d, dv, per_channel)
    for cuts in ([T], [1] * T, [2, 3, 1, 17, 2, 16]):
        for long_chunks in (False, True):             # one column per lane; rows split over lanes (single tokens: always the former)
            got = _delta_in_cuts(qkv, beta, decay, a_log, dt_bias, cuts, H, G, d, dv, per_channel, long_chunks=long_chunks)
            assert (got - ref).abs().max() <= 3e-5 * ref.abs().max(), (cuts, long_chunks)


def test_delta_rule_keeps_a_far_write_and_loses_it_with_decay():
    """A value written at token 0 under key e0 is read back 300 tokens later when nothing decays
    (all other keys orthogonal to e0), and is gone when the head decays."""
    H = G = 1
    d, dv, T = 32, 16, 300
    qkv = torch.zeros(T, 2 * d + dv)
    qkv[0, d + 0] = 1.0                      # key e0 ...
    qkv[0, 2 * d + 7] = 1.0                  # ... stores value e7
    qkv[1:, d + 1] = 1.0                     # later keys: e1
    qkv[-1, 0] = 1.0                         # the last query asks for e0
    qkv[:-1, 1] = 1.0
    beta = torch.full((T, 1), 30.0)          # sigmoid -> 1
    for z, want in ((-40.0, 1.0), (1.0, 0.0)):
        decay = torch.full((T, 1), z)
        got = _delta_in_cuts(qkv, beta, decay, torch.zeros(1), torch.zeros(1), [250] + [1] * 50, H, G, d, dv, False,
                             long_chunks=True)
        ref = _delta_ref(qkv, beta, decay, torch.zeros(1), torch.zeros(1), H, G, d, dv, False)
        assert (got - ref).abs().max() <= 1e-5
        assert abs(float(got[-1, 0, 7]) * d ** 0.5 - want) < 1e-3


@pytest.mark.parametrize("taps,dtype,C", [(1, torch.float32, 70), (2, torch.float32, 70), (3, torch.float32, 70),
                                          (5, torch.float32, 70), (2, torch.bfloat16, 72), (4, torch.bfloat16, 136),
                                          (3, torch.bfloat16, 70), (5, torch.bfloat16, 72)])
def test_short_convolution_across_portions_and_reused_slots(taps, dtype, C):
    """Scalar form (float32, odd widths, many taps) and the 8-channel form (16-bit, 2-4 taps)."""
    from mi355_decode import ops
    g = torch.Generator().manual_seed(taps)
    w = torch.randn(C, taps, generator=g).to(dtype)
    tol = 1e-5 if dtype == torch.float32 else 1e-2
    state = torch.full((3, taps - 1, C), float("nan"), device="cuda") if taps > 1 else torch.zeros(3, 0, C, device="cuda")
    for T, slot in ((23, 1), (9, 1), (40, 0)):                     # slot 1 is used twice: its old state must not leak
        x = torch.randn(T, C + 8, generator=g).to(dtype)[:, 8:]
        ref = R.short_conv_silu(x.float(), w.float())
        for cuts in ([T], [1] * T, [2, 1, 3] + [T - 6]):
            outs, at = [], 0
            for n in cuts:
                xs = x[at:at + n].cuda()
                outs.append(ops.causal_conv_silu(xs, w.cuda(), state, torch.zeros(n, dtype=torch.int32, device="cuda"),
                                                 torch.arange(at, at + n, dtype=torch.int64, device="cuda"),
                                                 torch.tensor([0, n], dtype=torch.int32, device="cuda"),
                                                 torch.tensor([slot], dtype=torch.int32, device="cuda")).float().cpu())
                at += n
            assert (torch.cat(outs) - ref).abs().max() <= tol * ref.abs().max(), (T, cuts)


# ------------------------------------------------------------------------------------------ #
# the whole model through the engine
# ------------------------------------------------------------------------------------------ #
@pytest.mark.parametrize("name", list(CONFIGS))
def test_whole_prompt_and_every_layer(name):
    eng = _engine(name)
    toks = _tokens(name, 90, 1)
    eng.runner.layer_trace = []
    try:
        got = eng.forced_step([("a", toks, list(range(len(toks))))], ["a"])
        trace = [t.cpu().numpy() for t in eng.runner.layer_trace]
    finally:
        eng.runner.layer_trace = None
    want = []
    with torch.no_grad():
        R.forward(_weights(name), CONFIGS[name], toks, want)
    assert len(trace) == len(want)
    for i, (a, b) in enumerate(zip(trace, want)):
        assert np.abs(a - b.numpy()).max() <= 1e-4 * np.abs(b.numpy()).max(), f"layer run {i}"
    _close(got, _ref(name, toks))


@pytest.mark.parametrize("name", list(CONFIGS))
def test_portions_and_token_by_token_equal_the_whole_prompt(name):
    eng = _engine(name)
    toks = _tokens(name, 70, 2)
    want = _ref(name, toks)
    for cuts in ([1] * 70, [2, 2, 3, 16, 1, 17, 2], [33, 2] + [1] * 35, [5] * 14):
        _close(_run_cuts(eng, "p", toks, cuts), want)


def test_first_tokens_and_one_token_requests():
    eng = _engine("loop0")
    for n in (1, 2, 3):
        toks = _tokens("loop0", n, 10 + n)
        _close(_run_cuts(eng, "s", toks, [1] * n), _ref("loop0", toks))
        _close(_run_cuts(eng, "s", toks, [n]), _ref("loop0", toks))


@pytest.mark.parametrize("name", ["loop0", "tail"])
def test_mixed_batches_equal_each_request_alone(name):
    """Four requests of unequal length advance together, portions beside single tokens; requests end and new
    ones take their pages and state slots."""
    eng = _engine(name, pages=24)
    lens = {"a": 60, "b": 23, "c": 91, "d": 2, "e": 47, "f": 35}
    toks = {r: _tokens(name, n, ord(r)) for r, n in lens.items()}
    plan = {"a": [30, 1, 1, 2, 26], "b": [2, 1, 20], "c": [16, 17, 1, 1, 1, 55], "d": [1, 1], "e": [2, 45], "f": [34, 1]}
    at = {r: 0 for r in lens}
    got = {r: [] for r in lens}
    live, waiting = ["a", "b", "c", "d"], ["e", "f"]
    step = 0
    while live:
        entries, end = [], []
        for r in list(live):
            if r == "b" and step % 2 == 1:
                continue                                            # b sits out every other step
            n = plan[r].pop(0)
            entries.append((r, toks[r][at[r]:at[r] + n], list(range(n))))
            at[r] += n
            if at[r] == lens[r]:
                end.append(r)
        out = eng.forced_step(entries, end)
        row = 0
        for r, t, _ in entries:
            got[r].append(out[row:row + len(t)])
            row += len(t)
        for r in end:
            live.remove(r)
            if waiting:
                live.append(waiting.pop(0))
        step += 1
    for r in lens:
        _close(np.concatenate(got[r]), _ref(name, toks[r]))


def test_pages_and_slots_are_reused_without_leaking():
    eng = _engine("plain", pages=8, max_model_len=128)              # one 100-token request nearly fills the pool
    for i in range(6):
        toks = _tokens("plain", 100 - 7 * i, 50 + i)
        _close(_run_cuts(eng, f"r{i}", toks, [40, 3] + [1] * 10), _ref("plain", toks))


def test_long_decoding_past_windows_and_pages():
    eng = _engine("loop0")
    toks = _tokens("loop0", 300, 9)
    _close(_run_cuts(eng, "long", toks, [10] + [1] * 290), _ref("loop0", toks), tol=6e-4)


def test_bfloat16_tracks_the_float32_restatement():
    eng = _engine("loop0", dtype="bfloat16")
    toks = _tokens("loop0", 64, 4)
    want = _ref("loop0", toks)
    for cuts in ([64], [30, 2] + [1] * 32):
        got = _run_cuts(eng, "h", toks, cuts)
        d = got - want
        d = d - d.mean(1, keepdims=True)
        rel = np.sqrt((d ** 2).mean(1)) / np.abs(want).max()
        assert rel.max() < 0.06, rel.max()


def test_decode_sized_steps_on_the_tiled_weight_stream():
    """bfloat16 at a width whose matrices have fragment-tiled copies: single tokens and short portions
    (the tiled GEMM, K split into slabs for the narrow outputs) against whole prompts (library GEMMs)
    and against the float32 restatement."""
    eng = _engine("wide", dtype="bfloat16")
    assert eng.runner._tiled_w, "no tiled weight copies at width 512"
    toks = _tokens("wide", 48, 3)
    want = _ref("wide", toks)
    whole = _run_cuts(eng, "w", toks, [48])
    for cuts in ([1] * 48, [20, 3, 1, 7] + [1] * 17):
        got = _run_cuts(eng, "w", toks, cuts)
        for a, b in ((got, want), (got, whole)):
            d = a - b
            d = d - d.mean(1, keepdims=True)
            assert (np.sqrt((d ** 2).mean(1)) / np.abs(want).std()).max() < 0.08


@pytest.mark.parametrize("name,dtype", [("loop0", "float32"), ("tail", "float32"), ("plain", "bfloat16"), ("wide", "bfloat16")])
def test_greedy_generation_through_the_engine(name, dtype):
    """LLM.generate: scheduler admission, prefill, then decode steps replayed from HIP graphs with
    run-ahead.  A token may leave the restatement's only where its own margin is inside the error."""
    from mi355_decode.llm import LLM
    from mi355_decode.sampling_params import SamplingParams
    eng = _engine(name, dtype=dtype)
    prompts = [_tokens(name, n, 70 + n) for n in (5, 33, 18, 1, 26)]     # five requests on four slots: one waits
    steps = 24
    outs = LLM(eng).generate(prompts, SamplingParams(max_tokens=steps, temperature=0.0, ignore_eos=True))
    assert eng.runner.use_graphs and eng.runner.graphs, "the decode steps did not run as HIP graphs"
    tol = 2e-3 if dtype == "float32" else 0.25
    for p, o in zip(prompts, outs):
        assert len(o) == steps
        with torch.no_grad():
            z = R.forward(_weights(name), CONFIGS[name], p + o)[len(p) - 1: -1]
        for t in range(steps):
            best = int(torch.argmax(z[t]))
            assert o[t] == best or float(z[t, best] - z[t, o[t]]) <= tol, f"token {t}: {o[t]} vs {best}"


def test_served_from_a_model_directory(tmp_path):
    """The OpenAI server started on a directory with config.json + model.safetensors of this family:
    weights from the checkpoint names, greedy completions by token id against the restatement (margin
    rule), and a seeded sampled completion through the framework's sampler."""
    import json
    import os
    import socket
    import subprocess
    import sys
    import time
    from safetensors.torch import save_file
    from conftest import PKG, ROOT
    from mi355_decode.harness import BenchClient
    name = "tail"
    cfg, w = CONFIGS[name], _weights(name)
    model_dir = tmp_path / "model"
    model_dir.mkdir()
    json.dump(cfg, open(model_dir / "config.json", "w"))
    save_file({k: (v.reshape(()) if v.numel() == 1 and "norm" in k else v).to(torch.bfloat16).contiguous() for k, v in w.items()},
              str(model_dir / "model.safetensors"))
    with socket.socket() as s:
        s.bind(("127.0.0.1", 0))
        port = s.getsockname()[1]
    args = ["--model", str(model_dir), "--served-model-name", "hybrid", "--host", "127.0.0.1", "--port", str(port),
            "--dtype", "float32", "--max-num-seqs", "4", "--max-model-len", "128"]
    env = dict(os.environ, PYTHONPATH=PKG + os.pathsep + ROOT)
    log = open(tmp_path / "server.log", "w")
    proc = subprocess.Popen([sys.executable, "-m", "mi355_decode.entrypoints.openai.api_server"] + args, env=env, stdout=log,
                            stderr=subprocess.STDOUT, start_new_session=True)
    url = f"http://127.0.0.1:{port}"
    try:
        client = BenchClient(url)
        t0 = time.time()
        while True:
            assert proc.poll() is None, open(tmp_path / "server.log").read()[-3000:]
            try:
                if client.health() == 200:
                    break
            except Exception:
                pass
            assert time.time() - t0 < 240, "server did not become healthy"
            time.sleep(0.2)
        post = lambda **body: client.http.post(f"{url}/v1/completions", json={"model": "hybrid", **body})   # noqa: E731
        prompt, steps = _tokens(name, 21, 5), 12
        r = post(prompt=prompt, max_tokens=steps, temperature=0, ignore_eos=True, logprobs=0, return_tokens_as_token_ids=True)
        assert r.status_code == 200, r.text
        got = [int(t.split(":")[1]) for t in r.json()["choices"][0]["logprobs"]["tokens"]]
        assert len(got) == steps
        with torch.no_grad():
            z = R.forward(w, cfg, prompt + got)[len(prompt) - 1: -1]
        for t in range(steps):
            best = int(torch.argmax(z[t]))
            assert got[t] == best or float(z[t, best] - z[t, got[t]]) <= 2e-3, f"token {t}"
        draws = [post(prompt=prompt, max_tokens=8, temperature=0.9, top_k=20, seed=7, ignore_eos=True, logprobs=0,
                      return_tokens_as_token_ids=True).json()["choices"][0]["logprobs"]["tokens"] for _ in range(2)]
        assert draws[0] == draws[1] and len(draws[0]) == 8
        assert "synthetic" not in open(tmp_path / "server.log").read()
    finally:
        import signal
        os.killpg(proc.pid, signal.SIGTERM)
        try:
            proc.wait(timeout=20)
        except subprocess.TimeoutExpired:
            os.killpg(proc.pid, signal.SIGKILL)
