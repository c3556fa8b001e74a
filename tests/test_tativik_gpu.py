"""Hybrid decoders in the sandwich arrangement (the Tativik design) on the GPU against the plain
float32 restatement in oracle/tativik_ref.py: every mechanism alone -- norms in groups and the gated
residual, the general delta rule, the latent attention with its window and sink, routing and the
expert products -- then the whole model through the engine: whole prompts, token-by-token decoding,
portions down to two tokens, mixed batches, reused pages and state slots, window and page edges,
other sizes, and greedy generation through LLM.generate.  Small seeded configurations made here;
float32 runs carry the sharp bars, bfloat16 a loose one."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

from oracle import tativik_ref as R  # noqa: E402


def _latent(heads, dim, rot_dim, vdim, kv_rank, q_rank, window, dims=None, base=10000.0, scale=0.2, kv_from=None):
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "q_rank": q_rank,
         "mask": {"size": window}, "rot": {"dims": rot_dim if dims is None else dims, "base": base}, "scale": scale}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return m


def _moe(experts, top, count, keep, ff):
    return {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top, "groups": {"count": count, "keep": keep}}}


CONFIGS = {
    # three norm groups, a shared latent two layers back, partial rotation, vdim != dim, a layer without
    # a feed-forward, two of three expert groups kept
    "mix": {"architecture": "Tativik", "width": 96, "vocab": 160, "norm": {"eps": 1e-5, "groups": 3}, "residual_mult": 0.5,
            "layers": [{"type": "latent_attention", "mixer": _latent(3, 16, 8, 24, 40, 24, 20, dims=4), "mlp": _moe(6, 3, 3, 2, 40)},
                       {"type": "general_delta", "mixer": {"heads": 2, "dim": 32}, "mlp": _moe(6, 2, 2, 1, 24)},
                       {"type": "latent_attention", "mixer": _latent(2, 24, 8, 8, 40, 16, 7, dims=4, scale=0.3, kv_from=0),
                        "mlp": None},
                       {"type": "general_delta", "mixer": {"heads": 1, "dim": 64}, "mlp": _moe(4, 1, 4, 3, 56)}]},
    # one norm group, multiplier 1, one expert chosen from one group, a window of one token and one
    # longer than any prompt here, a head wider than 128
    "plain": {"architecture": "Tativik", "width": 64, "vocab": 97, "norm": {"eps": 1e-6, "groups": 1}, "residual_mult": 1.0,
              "layers": [{"type": "general_delta", "mixer": {"heads": 4, "dim": 16}, "mlp": _moe(4, 1, 1, 1, 24)},
                         {"type": "latent_attention", "mixer": _latent(2, 32, 16, 32, 64, 32, 1, base=500.0), "mlp": None},
                         {"type": "latent_attention", "mixer": _latent(4, 8, 4, 16, 72, 40, 1000, scale=0.4), "mlp": _moe(5, 2, 1, 1, 16)},
                         {"type": "general_delta", "mixer": {"heads": 1, "dim": 136}, "mlp": None}]},
    # a width the weight-streaming GEMM's tiled form covers (decode-sized steps in 16 bits take it)
    "wide": {"architecture": "Tativik", "width": 512, "vocab": 384, "norm": {"eps": 1e-6, "groups": 4}, "residual_mult": 0.8,
             "layers": [{"type": "general_delta", "mixer": {"heads": 8, "dim": 64}, "mlp": _moe(8, 2, 4, 2, 256)},
                        {"type": "latent_attention", "mixer": _latent(8, 64, 32, 64, 128, 192, 48, scale=0.1), "mlp": _moe(8, 2, 4, 2, 256)},
                        {"type": "latent_attention", "mixer": _latent(4, 32, 32, 128, 128, 64, 24, scale=0.12, kv_from=1),
                         "mlp": _moe(16, 4, 2, 1, 128)}]},
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
@pytest.mark.parametrize("groups", [1, 2, 5])
def test_group_norms_and_the_gated_residual(dtype, groups):
    from mi355_decode import ops
    g = torch.Generator().manual_seed(groups)
    T, W = 6, 5 * 2 * 23
    tol = 1e-5 if dtype == torch.float32 else 1.2e-2
    x = torch.randn(T, W, generator=g) * 3
    x[:, : W // groups] *= 30.0                            # one part far louder than the rest: one norm over the row would show
    wt = torch.randn(W, generator=g)
    ref = R.group_rms_norm(x, wt, groups, 1e-5)
    out = ops.group_rms_norm_f32(x.cuda(), wt.cuda(), groups, 1e-5, dtype=dtype)
    assert out.dtype == dtype and (out.float().cpu() - ref).abs().max() <= tol * ref.abs().max()
    inplace = x.clone().cuda()
    assert ops.group_rms_norm_f32(inplace, wt.cuda(), groups, 1e-5, out=inplace) is inplace
    assert (inplace.cpu() - ref).abs().max() <= 1e-5 * ref.abs().max()
    y = (torch.randn(T, W, generator=g) * 2).to(dtype)
    gate = torch.randn(T, W + 16, generator=g).to(dtype)
    bias = torch.randn(W, generator=g)
    resid = x.clone().cuda()
    ops.gated_norm_resid_f32(resid, y.cuda(), gate.cuda()[:, 16:], bias.cuda(), wt.cuda(), groups, 1e-6, 0.7)
    ref = x + 0.7 * R.group_rms_norm(y.float() * torch.sigmoid(gate.float()[:, 16:] + bias), wt, groups, 1e-6)
    assert (resid.cpu() - ref).abs().max() <= 2e-5 * ref.abs().max()
    rows = (torch.randn(T, 50 + 8, generator=g) * 4).to(dtype)
    rw = torch.randn(50, generator=g)
    out = ops.rms_norm_rows(rows.cuda()[:, 8:], rw.cuda(), 1e-5)
    ref = R.plain_rms_norm(rows.float()[:, 8:], rw, 1e-5)
    assert (out.float().cpu() - ref).abs().max() <= tol * ref.abs().max()
    assert (ops.tanh_rows(rows.cuda()[:, 8:]).float().cpu() - torch.tanh(rows.float()[:, 8:])).abs().max() <= tol
    o = torch.randn(T, 3, 40, generator=g)
    hg = torch.randn(T, 3 * 40, generator=g).to(dtype)
    hw = torch.randn(3 * 40, generator=g)                   # one weight per head and channel
    out = ops.gated_head_rms_norm(o.cuda(), hg.cuda(), hw.cuda(), 1e-5, ops.ACT_SIGMOID)
    ref = (o / torch.sqrt((o * o).mean(-1, keepdim=True) + 1e-5)).reshape(T, -1) * hw * torch.sigmoid(hg.float())
    assert (out.float().cpu() - ref).abs().max() <= tol * ref.abs().max()


def _gdelta_in_cuts(x, w0, ab, cuts, H, d, slot=2, slots=4, long_chunks=True):
    """x [T, 5, H * d] = r | k | v | decay | rate inputs of one sequence fed in portions."""
    from mi355_decode import ops
    state = torch.full((slots, H, d, d), float("nan"), device="cuda")
    outs, at = [], 0
    for n in cuts:
        xs = x[at:at + n].reshape(n, -1).contiguous().cuda()      # column slices of one row-major matrix
        C = H * d
        outs.append(ops.general_delta_rule(xs[:, :C], xs[:, C:2 * C], xs[:, 2 * C:3 * C], xs[:, 3 * C:4 * C], w0.cuda(),
                                           xs[:, 4 * C:], ab.cuda(), state,
                                           torch.tensor([0, n], dtype=torch.int32, device="cuda"),
                                           torch.arange(at, at + n, dtype=torch.int64, device="cuda"),
                                           torch.tensor([slot], dtype=torch.int32, device="cuda"), H, d,
                                           long_chunks=long_chunks).cpu())
        at += n
    return torch.cat(outs), state


def _gdelta_ref(x, w0, ab, H, d):
    T = x.shape[0]
    w = torch.exp(-R.DECAY_RATE * torch.sigmoid(x[:, 3] + w0)).view(T, H, d)
    a = torch.sigmoid(x[:, 4] + ab).view(T, H, d)
    return R.general_delta_rule(x[:, 0].view(T, H, d), x[:, 1].view(T, H, d), x[:, 2].view(T, H, d), w, a)


@pytest.mark.parametrize("H,d", [(2, 48), (3, 32), (1, 64), (2, 20), (1, 128), (1, 200)])
def test_general_delta_rule_whole_portions_and_single_tokens(H, d):
    g = torch.Generator().manual_seed(H * 1000 + d)
    T = 41
    x = torch.randn(T, 5, H * d, generator=g)
    w0, ab = torch.randn(H * d, generator=g), torch.randn(H * d, generator=g) * 0.5
    ref = _gdelta_ref(x, w0, ab, H, d)
    x16 = x.to(torch.bfloat16)
    ref16 = _gdelta_ref(x16.float(), w0, ab, H, d)
    for cuts in ([T], [1] * T, [2, 3, 1, 17, 2, 16]):
        for long_chunks in (True, False):                   # state rows split over lanes; one state column per lane
            got, _ = _gdelta_in_cuts(x, w0, ab, cuts, H, d, long_chunks=long_chunks)
            assert (got - ref).abs().max() <= 3e-5 * ref.abs().max(), (cuts, long_chunks)
            got, _ = _gdelta_in_cuts(x16, w0, ab, cuts, H, d, long_chunks=long_chunks)     # 16-bit inputs, fp32 inside
            assert (got - ref16).abs().max() <= 3e-5 * ref16.abs().max(), (cuts, long_chunks, "bfloat16")


def test_general_delta_rule_keeps_a_far_write_removes_it_along_its_key_and_forgets_it_with_decay():
    """One loud key / value pair is written at token 3; 200 tokens later a query along that key still
    reads it when the decay is slow and the later keys are orthogonal to it; a later token with the
    same key and removal rate 1 takes it out; a fast decay loses it."""
    H, d, T = 1, 32, 220
    g = torch.Generator().manual_seed(11)
    x = torch.zeros(T, 5, d)
    x[:, 1, 1:] = torch.randn(T, d - 1, generator=g) * 0.1     # later keys live in channels 1.., orthogonal to channel 0
    x[:, 2] = torch.randn(T, d, generator=g) * 0.1
    x[3, 1] = 0.0
    x[3, 1, 0] = 4.0                                           # the loud key, channel 0
    x[3, 2] = 0.0
    x[3, 2, 5] = 7.0                                           # its value, channel 5
    x[-1, 0, 0] = 1.0                                          # the last token asks along the loud key
    x[:, 3] = -30.0                                            # decay exp(-e^-0.5 sigmoid(-30)) = 1
    x[:, 4] = -30.0                                            # removal rate 0
    zero = torch.zeros(d)
    ref = _gdelta_ref(x, zero, zero, H, d)
    assert abs(float(ref[-1, 0, 5]) - 28.0) < 0.1              # k v^T read along k: 4 * 7
    for cuts in ([T], [50, 2] + [1] * 168):
        got, _ = _gdelta_in_cuts(x, zero, zero, cuts, H, d)
        assert (got - ref).abs().max() <= 1e-4 * ref.abs().max()
    x[100, 1] = 0.0
    x[100, 1, 0] = 0.5                                         # the same direction again, removal rate 1, nothing written
    x[100, 2] = 0.0
    x[100, 4] = 30.0
    ref = _gdelta_ref(x, zero, zero, H, d)
    got, _ = _gdelta_in_cuts(x, zero, zero, [99, 2, 119], H, d)
    assert abs(float(got[-1, 0, 5])) < 1e-3 and (got - ref).abs().max() <= 1e-4 * ref.abs().max()
    x[100, 4] = -30.0
    x[:, 3] = 30.0                                             # the fastest decay: exp(-e^-0.5) per token
    ref = _gdelta_ref(x, zero, zero, H, d)
    got, _ = _gdelta_in_cuts(x, zero, zero, [T], H, d)
    assert abs(float(got[-1, 0, 5])) < 1e-6 and (got - ref).abs().max() <= 1e-4 * ref.abs().max() + 1e-9


def test_general_delta_state_slots_are_separate_and_reset_at_position_zero():
    H, d = 2, 32
    g = torch.Generator().manual_seed(5)
    xa, xb = torch.randn(30, 5, H * d, generator=g), torch.randn(20, 5, H * d, generator=g)
    w0, ab = torch.randn(H * d, generator=g), torch.randn(H * d, generator=g)
    from mi355_decode import ops
    state = torch.full((3, H, d, d), float("nan"), device="cuda")
    C = H * d

    def step(chunks):
        """chunks: [(x rows, first position, slot)] run as one packed batch."""
        rows = torch.cat([c[0].reshape(len(c[0]), -1) for c in chunks]).contiguous().cuda()
        cu = np.cumsum([0] + [len(c[0]) for c in chunks]).astype(np.int32)
        pos = np.concatenate([np.arange(c[1], c[1] + len(c[0])) for c in chunks]).astype(np.int64)
        out = ops.general_delta_rule(rows[:, :C], rows[:, C:2 * C], rows[:, 2 * C:3 * C], rows[:, 3 * C:4 * C], w0.cuda(),
                                     rows[:, 4 * C:], ab.cuda(), state, torch.from_numpy(cu).cuda(),
                                     torch.from_numpy(pos).cuda(),
                                     torch.tensor([c[2] for c in chunks], dtype=torch.int32, device="cuda"), H, d).cpu()
        return [out[cu[i]:cu[i + 1]] for i in range(len(chunks))]

    ra, rb = _gdelta_ref(xa, w0, ab, H, d), _gdelta_ref(xb, w0, ab, H, d)
    a1, b1 = step([(xa[:17], 0, 2), (xb[:1], 0, 0)])             # a portion beside a single first token
    a2, b2 = step([(xa[17:18], 17, 2), (xb[1:], 1, 0)])          # a single token beside a portion
    (a3,) = step([(xa[18:], 18, 2)])
    (b3,) = step([(xb, 0, 2)])                                   # b again on the slot a used: position 0 resets it
    for got, want in ((torch.cat([a1, a2, a3]), ra), (torch.cat([b1, b2]), rb), (b3, rb)):
        assert (got - want).abs().max() <= 3e-5 * want.abs().max()


def _paged(T, num_pages, seed):
    """A shuffled block table for one sequence of T tokens and its slot mapping."""
    order = np.random.default_rng(seed).permutation(num_pages)[: (T + 15) // 16].astype(np.int32)
    pos = np.arange(T)
    return order, order[pos // 16].astype(np.int64) * 16 + pos % 16


def _latent_in_cuts(x, nw, ql, q, hw, off, sink, gate, cuts, H, R_, rot, dims, window, scale, base=100.0, pages=12,
                    tiled=False):
    """Latent write + attention over one sequence fed in portions (a last portion takes what `cuts`
    leaves); returns [T, H, R_] float32."""
    from mi355_decode import ops
    from mi355_decode.hybrid_runner import rotary_table
    T, dt = x.shape[0], x.dtype
    cuts = list(cuts) + [T]
    table, slots = _paged(T, pages, 5)
    cache = torch.full((pages, 16, R_ + rot), float("nan"), dtype=dt, device="cuda")
    cache_t = torch.full((pages, R_, 16), float("nan"), dtype=dt, device="cuda") if tiled else None
    bt = torch.zeros(1, pages, dtype=torch.int32)
    bt[0, : len(table)] = torch.from_numpy(table)
    cs = rotary_table(dims, base, pages * 16, "cuda")
    outs, at = [], 0
    for n in cuts:
        n = min(n, T - at)
        if n == 0:
            break
        sl = slice(at, at + n)
        pos = torch.arange(at, at + n, dtype=torch.int64, device="cuda")
        ops.latent_kv_write(x[sl].cuda(), nw.cuda(), cs, pos, torch.from_numpy(slots[sl]).cuda(), cache, R_, rot, 1e-5,
                            cache_t=cache_t)
        qlh = ql[sl].transpose(0, 1).contiguous().cuda()
        if tiled:                                             # the matrix cores; single rows spread their keys over three workgroups
            out = ops.latent_window_attn_tiles(ops.latent_q_pack(qlh, q[sl].cuda(), hw, off, rot, cs, pos), cache, cache_t,
                                               bt.cuda(), torch.from_numpy(ops.pair_tiles([0, n], H)).cuda(), pos, sink.cuda(),
                                               None if gate is None else gate[sl].cuda(), window, scale,
                                               num_splits=3 if n == 1 else 1)
        else:
            out = ops.latent_window_attn(qlh, q[sl].cuda(), hw, off, cache, bt.cuda(),
                                         torch.zeros(n, dtype=torch.int32, device="cuda"), pos, sink.cuda(),
                                         None if gate is None else gate[sl].cuda(), cs, window, scale)
        outs.append(out.float().cpu().transpose(0, 1))
        at += n
    assert at == T
    return torch.cat(outs)


def _latent_ref(x, nw, ql, q, hw, off, sink, gate, H, R_, rot, dims, window, scale, base=100.0):
    T = x.shape[0]
    x, ql, q = x.float(), ql.float(), q.float()
    pos = torch.arange(T)
    c = R.plain_rms_norm(x[:, :R_], nw, 1e-5)
    kr = R.rotate_half(x[:, R_:], pos, dims, base)
    qr = R.rotate_half(q.view(T, H, hw)[:, :, off:off + rot], pos, dims, base)
    out = torch.zeros(T, H, R_)
    for h in range(H):
        s = (ql[:, h] @ c.T + qr[:, h] @ kr.T) * scale
        out[:, h] = R.window_softmax_with_sink(s, window, sink[h]) @ c
    if gate is not None:
        out = out * torch.sigmoid(gate.float())[:, :, None]
    return out


@pytest.mark.parametrize("H,R_,rot,dims,window", [(3, 40, 8, 4, 20), (2, 64, 16, 16, 1), (4, 96, 32, 32, 33), (1, 130, 6, 0, 200),
                                                  (8, 128, 64, 64, 48), (2, 512, 64, 32, 17)])
def test_latent_attention_whole_portions_and_single_tokens(H, R_, rot, dims, window):
    g = torch.Generator().manual_seed(H * 100 + R_)
    T, hw, off = 75, rot + 5, 5
    x = torch.randn(T, R_ + rot, generator=g)
    nw, sink = torch.randn(R_, generator=g) * 0.2 + 1, torch.randn(H, generator=g)
    ql, q = torch.randn(T, H, R_, generator=g) * 0.5, torch.randn(T, H * hw, generator=g)
    gate = torch.randn(T, H, generator=g)
    args = (H, R_, rot, dims, window, 0.3)
    ref = _latent_ref(x, nw, ql, q, hw, off, sink, gate, *args)
    for cuts in ([T], [1] * T, [2, 3, 1, 30, 2, 16, 21]):
        got = _latent_in_cuts(x, nw, ql, q, hw, off, sink, gate, cuts, *args)
        assert (got - ref).abs().max() <= 3e-5 * ref.abs().max(), cuts
    b16 = lambda t: t.to(torch.bfloat16)                      # noqa: E731
    got = _latent_in_cuts(b16(x), nw, b16(ql), b16(q), hw, off, sink, b16(gate), [40, 2, 1, 32], *args)
    ref = _latent_ref(b16(x), nw, b16(ql), b16(q), hw, off, sink, b16(gate), *args)
    assert (got - ref).abs().max() <= 3e-2 * ref.abs().max()


@pytest.mark.parametrize("H,R_,rot,dims,window", [(3, 48, 8, 4, 20), (2, 64, 16, 16, 1), (4, 96, 32, 32, 33), (1, 128, 8, 0, 200),
                                                  (16, 128, 64, 64, 48), (20, 512, 64, 32, 17), (5, 208, 24, 24, 40)])
def test_latent_attention_on_the_matrix_cores(H, R_, rot, dims, window):
    """bfloat16 inputs; the restatement sees the same rounded inputs, so what is left is the rounding of
    the stored latent, of the packed query and of the weights in the second product."""
    g = torch.Generator().manual_seed(H * 100 + R_)
    T, hw, off = 75, rot + 8, 8
    b16 = lambda t: t.to(torch.bfloat16)                      # noqa: E731
    x = b16(torch.randn(T, R_ + rot, generator=g))
    nw, sink = torch.randn(R_, generator=g) * 0.2 + 1, torch.randn(H, generator=g)
    ql, q = b16(torch.randn(T, H, R_, generator=g) * 0.5), b16(torch.randn(T, H * hw, generator=g))
    gate = b16(torch.randn(T, H, generator=g))
    args = (H, R_, rot, dims, window, 0.3)
    ref = _latent_ref(x, nw, ql, q, hw, off, sink, gate, *args)
    for cuts in ([T], [1] * T, [2, 3, 1, 30, 2, 16, 21]):
        got = _latent_in_cuts(x, nw, ql, q, hw, off, sink, gate, cuts, *args, tiled=True)
        assert (got - ref).abs().max() <= 3e-2 * ref.abs().max(), cuts


@pytest.mark.parametrize("window", [16, 17, 31, 48, 64, 65, 200])
def test_latent_window_edge_and_sink_show_with_one_loud_key(window):
    """Token 9 holds a latent that every query scores far above all others: a query sees it exactly
    while 0 <= i - 9 < window (for the widest window: one key among two hundred, a dozen pages back);
    once it is gone the sink, set high, takes most of the weight."""
    H, R_, rot, T = 2, 32, 8, 9 + max(70, window + 5)
    g = torch.Generator().manual_seed(window)
    x = torch.randn(T, R_ + rot, generator=g) * 0.1
    x[9, :R_] = 0.0
    x[9, 3] = 1.0                                              # normed: sqrt(32) on channel 3
    nw = torch.ones(R_)
    ql = torch.zeros(T, H, R_)
    ql[:, :, 3] = 3.0
    q = torch.zeros(T, H * rot)
    sink = torch.tensor([12.0, -50.0])
    args = (H, R_, rot, rot, window, 1.0)
    ref = _latent_ref(x, nw, ql, q, rot, 0, sink, None, *args)
    inside, outside = 9 + window - 1, 9 + window
    assert float(ref[inside, 0, 3]) > 5.0 and abs(float(ref[outside, 0, 3])) < 2.5     # the edge, in the restatement
    assert float(ref[outside, 0].abs().max()) < 0.3 * float(ref[outside, 1].abs().max())   # the sink takes head 0's weight
    for cuts in ([T], [9 + window - 1, 1, 1] + [1] * 5, [5, 2] + [1] * (T - 7)):
        got = _latent_in_cuts(x, nw, ql, q, rot, 0, sink, None, cuts, *args, pages=16)
        assert (got - ref).abs().max() <= 1e-4 * ref.abs().max(), cuts
        b16 = lambda t: t.to(torch.bfloat16)                  # noqa: E731
        got = _latent_in_cuts(b16(x), nw, b16(ql), b16(q), rot, 0, sink, None, cuts, *args, pages=16, tiled=True)
        r16 = _latent_ref(b16(x), nw, b16(ql), b16(q), rot, 0, sink, None, *args)
        assert (got - r16).abs().max() <= 3e-2 * r16.abs().max(), cuts


def test_routing_groups_corrections_and_negative_choice_scores():
    from mi355_decode import ops
    g = torch.Generator().manual_seed(2)
    for E, top, count, keep in ((8, 2, 2, 1), (12, 3, 4, 2), (6, 1, 6, 2), (16, 4, 1, 1), (9, 9, 3, 3), (64, 8, 8, 4), (160, 20, 5, 3)):
        z = torch.randn(300, E, generator=g) * 2
        # corrections that push every choice score below zero: a barred expert must not beat them as a "0"
        for corr in (torch.randn(E, generator=g) * 0.3, torch.randn(E, generator=g) * 0.3 - 3.0):
            ids, wts = ops.moe_route(z.cuda(), corr.cuda(), top, count, keep)
            rid, rw = R.route(z, corr, top, count, keep)
            assert torch.equal(ids.cpu().long().sort(-1).values, rid.sort(-1).values), (E, top, count, keep)
            got = torch.zeros(300, E).scatter_(1, ids.cpu().long(), wts.cpu())
            want = torch.zeros(300, E).scatter_(1, rid, rw)
            assert (got - want).abs().max() < 1e-6
        z[::7, 1] = float("nan")                              # a NaN logit must not turn into an index outside the experts
        ids, _ = ops.moe_route(z.cuda(), torch.zeros(E).cuda(), top, count, keep)
        ids = ids.cpu()
        assert int(ids.min()) >= 0 and int(ids.max()) < E and all(len(set(r.tolist())) == top for r in ids)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("T", [1, 5, 300])
@pytest.mark.parametrize("W,F", [(72, 40), (96, 64)])           # the second: sizes that the matrix-core row kernels cover in 16 bits
def test_expert_products_by_rows_and_by_expert_matrices(dtype, T, W, F):
    """The mixture through the runner's feed-forward object: few rows take the per-row kernels, many
    rows one library product per expert; both against the restatement."""
    from types import SimpleNamespace
    from mi355_decode.config import MoESpec
    from mi355_decode.hybrid_runner import MoEFeedForward
    g = torch.Generator().manual_seed(T)
    E, top = 6, 3
    wt = {"router": torch.randn(E, W, generator=g) * W ** -0.5, "correction": torch.randn(E, generator=g) * 0.3}
    for e in range(E):
        wt[f"e{e}.gate"], wt[f"e{e}.up"] = torch.randn(F, W, generator=g) * W ** -0.5, torch.randn(F, W, generator=g) * W ** -0.5
        wt[f"e{e}.down"] = torch.randn(W, F, generator=g) * F ** -0.5
    wt = {k: v.to(torch.bfloat16).float() for k, v in wt.items()}
    h = torch.randn(T, W, generator=g).to(dtype)
    mlp = {"router": {"top": top, "groups": {"count": 3, "keep": 2}}}
    ref = R.moe_ff(wt, "", mlp, h.float())
    lw = SimpleNamespace(router_w=wt["router"].cuda(), correction=wt["correction"].cuda(),
                         gate_up_w=torch.stack([torch.cat([wt[f"e{e}.gate"], wt[f"e{e}.up"]]) for e in range(E)]).to(dtype).cuda(),
                         down_w=torch.stack([wt[f"e{e}.down"] for e in range(E)]).to(dtype).cuda())
    ff = MoEFeedForward(MoESpec(E, top, 3, 2, F), lw, None)
    tol = 2e-5 if dtype == torch.float32 else 3e-2
    for min_rows, max_tokens in ((1, 2048), (1 << 30, 2048), (1, 64)):   # products per expert; the per-row kernels; in slices
        ff.GROUPED_MIN_ROWS, ff.GROUPED_MAX_TOKENS = min_rows, max_tokens
        got = ff(h.cuda()).float().cpu()
        assert (got - ref).abs().max() <= tol * ref.abs().max(), (min_rows, max_tokens)


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
        assert np.abs(a - b.numpy()).max() <= 1e-4 * np.abs(b.numpy()).max(), f"layer {i}"
    _close(got, _ref(name, toks))


@pytest.mark.parametrize("name", list(CONFIGS))
def test_portions_and_token_by_token_equal_the_whole_prompt(name):
    eng = _engine(name)
    toks = _tokens(name, 70, 2)
    want = _ref(name, toks)
    for cuts in ([1] * 70, [2, 2, 3, 16, 1, 17, 2], [33, 2] + [1] * 35, [5] * 14):
        _close(_run_cuts(eng, "p", toks, cuts), want)


def test_first_tokens_and_one_token_requests():
    eng = _engine("mix")
    for n in (1, 2, 3):
        toks = _tokens("mix", n, 10 + n)
        _close(_run_cuts(eng, "s", toks, [1] * n), _ref("mix", toks))
        _close(_run_cuts(eng, "s", toks, [n]), _ref("mix", toks))


@pytest.mark.parametrize("name", ["mix", "plain"])
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
    eng = _engine("mix")
    toks = _tokens("mix", 300, 9)
    _close(_run_cuts(eng, "long", toks, [10] + [1] * 290), _ref("mix", toks), tol=6e-4)


@pytest.mark.parametrize("name", ["mix", "wide"])
def test_bfloat16_tracks_the_float32_restatement(name):
    """Whole prompts (library GEMMs) and decode-sized steps (at width 512 the tiled weight stream) in
    bfloat16 against the restatement and against each other.  Rounding may turn a close call of a
    router, which moves that position's logits by far more than rounding does: a few such positions
    are allowed, the rest must be close."""
    eng = _engine(name, dtype="bfloat16")
    if name == "wide":
        assert eng.runner._tiled_w, "no tiled weight copies at width 512"
    toks = _tokens(name, 64, 4)
    want = _ref(name, toks)
    whole = _run_cuts(eng, "h", toks, [64])
    for got in (whole, _run_cuts(eng, "h", toks, [30, 2] + [1] * 32)):
        for a, b in ((got, want), (got, whole)):
            d = a - b
            d = d - d.mean(1, keepdims=True)
            err = np.sqrt((d ** 2).mean(1)) / want.std()
            assert np.median(err) < 0.03 and (err > 0.1).sum() <= 4, (np.median(err), np.sort(err)[-6:])


@pytest.mark.parametrize("name,dtype", [("mix", "float32"), ("plain", "float32"), ("wide", "bfloat16")])
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
    tol = 2e-3 if dtype == "float32" else 0.3
    for p, o in zip(prompts, outs):
        assert len(o) == steps
        with torch.no_grad():
            z = R.forward(_weights(name), CONFIGS[name], p + o)[len(p) - 1: -1]
        for t in range(steps):
            best = int(torch.argmax(z[t]))
            assert o[t] == best or float(z[t, best] - z[t, o[t]]) <= tol, f"token {t}: {o[t]} vs {best}"


def test_served_from_a_model_directory(tmp_path):
    """The OpenAI server started on a directory with config.json + model.safetensors of this design: the
    model class chosen by config.json, weights from the checkpoint names, greedy completions by token
    id against the restatement (margin rule), and a seeded sampled completion through the sampler."""
    import json
    import os
    import signal
    import socket
    import subprocess
    import sys
    import time
    from safetensors.torch import save_file
    from conftest import PKG, ROOT
    from mi355_decode.harness import BenchClient
    name = "mix"
    cfg, w = CONFIGS[name], _weights(name)
    model_dir = tmp_path / "model"
    model_dir.mkdir()
    json.dump(cfg, open(model_dir / "config.json", "w"))
    save_file({k: v.to(torch.bfloat16).contiguous() for k, v in w.items()}, str(model_dir / "model.safetensors"))
    with socket.socket() as s:
        s.bind(("127.0.0.1", 0))
        port = s.getsockname()[1]
    args = ["--model", str(model_dir), "--served-model-name", "sandwich", "--host", "127.0.0.1", "--port", str(port),
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
        post = lambda **body: client.http.post(f"{url}/v1/completions", json={"model": "sandwich", **body})   # noqa: E731
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
        os.killpg(proc.pid, signal.SIGTERM)
        try:
            proc.wait(timeout=20)
        except subprocess.TimeoutExpired:
            os.killpg(proc.pid, signal.SIGKILL)
