"""Hybrid decoders (the Lozupel design), the parts that need no GPU: the config reader, the order
of layer runs, the fused weight layout, state-slot bookkeeping in the scheduler, and the float32
restatement's own invariants (a window edge, a state carried across a cut)."""
import pytest
import torch

from oracle import lozupel_ref as R


def _cfg(loop=None, softcap=9.0):
    left = {"heads": 4, "kv_heads": 2, "dim": 16, "vdim": 24, "mask": {"size": 5}, "rot": {"dims": 8, "base": 100.0},
            "scale": 0.3}
    d = {"architecture": "Lozupel", "embedding": {"scale": 2.0}, "width": 40, "vocab": 50, "norm": {"eps": 1e-5},
         "layers": [{"type": "parallel", "mixer": {"left": left, "right": {"heads": 2, "kv_heads": 1, "dim": 16, "vdim": 8, "conv": 3}},
                     "mlp": {"kind": "dense", "ff": 56}},
                    {"type": "delta", "mixer": {"heads": 2, "kv_heads": 2, "dim": 8, "vdim": 16, "conv": 2}, "mlp": None},
                    {"type": "delta", "mixer": {"heads": 1, "kv_heads": 1, "dim": 8, "vdim": 8, "conv": 4},
                     "mlp": {"kind": "dense", "ff": 24}}]}
    if loop:
        d["loop"] = loop
    if softcap:
        d["logit_softcap"] = softcap
    return d


def test_config_reader_and_layer_runs():
    from mi355_decode.config import ModelConfig
    c = ModelConfig.from_dict(_cfg(loop={"start": 1, "stop": 3, "times": 2}))
    assert c.family == "hybrid" and c.architecture == "Lozupel" and c.hidden_size == 40 and c.vocab_size == 50
    s = c.hybrid
    assert s.embed_scale == 2.0 and s.logit_softcap == 9.0 and c.rms_norm_eps == 1e-5
    assert s.runs() == [(0, None), (1, 0), (2, 0), (1, 1), (2, 1)] == R.layer_runs(_cfg(loop={"start": 1, "stop": 3, "times": 2}))
    a, d = s.layers[0].attn, s.layers[0].delta
    assert (a.heads, a.kv_heads, a.dim, a.vdim, a.window, a.rot_dims, a.rot_base, a.scale) == (4, 2, 16, 24, 5, 8, 100.0, 0.3)
    assert d.per_channel and d.conv == 3 and not s.layers[1].delta.per_channel
    assert s.layers[0].ff == 56 and s.layers[1].ff is None
    plain = ModelConfig.from_dict(_cfg(softcap=None)).hybrid
    assert plain.runs() == [(0, None), (1, None), (2, None)] and plain.logit_softcap is None
    whole = ModelConfig.from_dict(_cfg(loop={"start": 0, "stop": 3, "times": 3})).hybrid
    assert whole.runs() == [(i, t) for t in range(3) for i in range(3)]
    with pytest.raises(ValueError):
        ModelConfig.from_dict(_cfg(loop={"start": 2, "stop": 5, "times": 2}))
    bad = _cfg()
    bad["layers"][1]["type"] = "other"
    with pytest.raises(ValueError):
        ModelConfig.from_dict(bad)


def test_weight_layout_fuses_what_reads_the_layer_input():
    from mi355_decode import weights as W
    from mi355_decode.config import ModelConfig
    cfgd = _cfg(loop={"start": 1, "stop": 2, "times": 2})
    st = R.random_state(cfgd, seed=3, rank=5)
    c = ModelConfig.from_dict(cfgd)
    w = W.from_state_dict(c, st, torch.float32, "cpu")
    lw = w.layers[0]
    for name, key in (("lq", "l0.mix.left.q"), ("lg", "l0.mix.left.g"), ("q", "l0.mix.right.q"), ("b", "l0.mix.right.b"),
                      ("a1", "l0.mix.right.a1"), ("g1", "l0.mix.right.g1")):
        at, n = lw.seg[name]
        assert at % 8 == 0 and torch.equal(lw.in_w[at:at + n], st[key])
    q0 = lw.seg["q"][0]
    assert lw.seg["k"][0] == q0 + 16 and lw.seg["v"][0] == q0 + 32          # adjacent: one convolution launch
    assert torch.equal(lw.conv_w, torch.cat([st["l0.mix.right.q.conv"], st["l0.mix.right.k.conv"], st["l0.mix.right.v.conv"]]))
    assert lw.a2_w.shape == (2 * 16, 5) and lw.dt_bias.shape == (32,) and lw.dt_bias.dtype == torch.float32
    assert torch.equal(lw.gate_up_w, torch.cat([st["l0.mix.mlp.gate"] if False else st["l0.mlp.gate"], st["l0.mlp.up"]]))
    assert w.layers[1].norm2 is None and w.layers[1].gate_up_w is None and w.layers[1].dt_bias.shape == (2,)
    assert w.loop_step.shape == (2, 40) and w.final_norm.shape == (1,)
    del st["l2.mix.a"]
    with pytest.raises(KeyError):
        W.from_state_dict(c, st, torch.float32, "cpu")
    with pytest.raises(ValueError):
        W.from_state_dict(c, R.random_state(cfgd, 3), torch.float32, "cpu", tp_size=2)
    syn = W.hybrid_synthetic_state(c, seed=1, rank=7)
    assert set(syn) == set(R.random_state(cfgd, 0, rank=7)) and syn["l0.mix.right.a2"].shape == (32, 7)


def test_state_slots_follow_a_sequence_through_the_scheduler():
    from mi355_decode.engine import BlockAllocator, NoFreeBlocks, Scheduler, Sequence, SlotAllocator
    from mi355_decode.sampling_params import SamplingParams
    slots = SlotAllocator(2)
    sched = Scheduler(BlockAllocator(8), max_num_seqs=4, max_num_batched_tokens=64, max_model_len=128, slots=slots)
    seqs = [Sequence(str(i), list(range(20)), SamplingParams(max_tokens=4)) for i in range(3)]
    for s in seqs:
        sched.add(s)
    kind, chunks = sched.schedule()
    assert kind == "prefill" and [c[0] for c in chunks] == seqs[:2]            # the third waits for a slot
    assert sorted(s.state_slot for s in seqs[:2]) == [0, 1] and seqs[2].state_slot is None and slots.num_free == 0
    for s, _, n in chunks:
        s.num_computed = n
    freed = seqs[0].state_slot
    sched.release(seqs[0])
    assert seqs[0].state_slot is None and slots.num_free == 1
    kind, chunks = sched.schedule()
    assert kind == "prefill" and chunks[0][0] is seqs[2] and seqs[2].state_slot == freed
    late = Sequence("late", [], SamplingParams(max_tokens=1))
    with pytest.raises(NoFreeBlocks):
        sched.admit(late, 5)
    assert late.state_slot is None and late not in sched.running


def test_restatement_window_edge_and_cut_invariance():
    """The float32 restatement itself: a loud key is heard window - 1 tokens later and not after;
    the delta rule gives the same outputs when the sequence is cut and the state carried by hand."""
    T, d = 12, 4
    q = torch.zeros(T, 1, d)
    q[:, 0, 0] = 6.0
    k = torch.zeros(T, 1, d)
    k[2, 0, 0] = 6.0
    v = torch.zeros(T, 1, 2)
    v[2, 0, 1] = 1.0
    o = R.sigmoid_window_attention(q, k, v, 5, 1.0, torch.ones(1), torch.full((1,), -30.0))
    assert o[6, 0, 1] > 0.99 and o[7, 0, 1] < 1e-9 and o[1, 0, 1] == 0
    g = torch.Generator().manual_seed(0)
    x, w = torch.randn(9, 3, generator=g), torch.randn(3, 4, generator=g)
    y = R.short_conv_silu(x, w)
    assert torch.allclose(y[0], torch.nn.functional.silu(x[0] * w[:, 3]))
    assert torch.allclose(y[5], torch.nn.functional.silu((x[2:6] * w.T).sum(0)))
    cfgd = _cfg(loop={"start": 0, "stop": 2, "times": 2})
    wts = R.random_state(cfgd, 5)
    toks = list(range(30))
    z = R.forward(wts, cfgd, toks)
    assert torch.allclose(R.forward(wts, cfgd, toks[:17]), z[:17], atol=1e-5)     # causal
    assert float(z.abs().max()) <= 9.0


class _StatefulRunner:
    """A runner double whose 'model' is a running checksum per state slot and a token table in the KV
    pages: it fails loudly when a step hands it a slot whose state does not continue the request, a
    page that holds another request's tokens, or a chunk at position 0 that finds old state."""
    device, V, NUM_STAGES = "cpu", 50, 1

    def __init__(self, num_blocks, max_num_seqs, max_model_len, slots):
        import numpy as np
        self.np = np
        self.num_blocks, self.max_num_seqs, self.num_state_slots = num_blocks, max_num_seqs, slots
        self.max_blocks = (max_model_len + 15) // 16
        self.pages = np.full(num_blocks * 16, -1, dtype=np.int64)
        self.state = {s: (0, 0) for s in range(slots)}          # slot -> (tokens seen, checksum)
        self.batches = []

    def host_inputs(self, stage=0):
        B = self.max_num_seqs
        return self.np.zeros(3 * B, dtype=self.np.int64), self.np.zeros(B + B * self.max_blocks + B, dtype=self.np.int32)

    def run_prefill(self, token_ids, positions, slot_mapping, block_tables, cu_seqlens, context_lens, max_q_len,
                    sampling=None, logprobs=-1, prompt_logprobs=None, state_slots=None, logit_rows=None):
        np = self.np
        assert state_slots is not None and len(state_slots) == len(context_lens) and len(set(state_slots.tolist())) == len(state_slots)
        self.batches.append([int(cu_seqlens[i + 1] - cu_seqlens[i]) for i in range(len(context_lens))])
        rows = np.zeros((len(token_ids), self.V), dtype=np.float32)
        for i, slot in enumerate(state_slots.tolist()):
            a, b = int(cu_seqlens[i]), int(cu_seqlens[i + 1])
            start = int(positions[a])
            seen, acc = (0, 0) if start == 0 else self.state[slot]
            assert seen == start, f"slot {slot} holds {seen} tokens, the chunk starts at {start}"
            for r in range(a, b):
                self.pages[slot_mapping[r]] = token_ids[r]
                acc = (acc * 31 + int(token_ids[r]) + 1) % 1000003
                p = int(positions[r])
                ctx = self.pages[block_tables[i][np.arange(p + 1) // 16].astype(np.int64) * 16 + np.arange(p + 1) % 16]
                rows[r, 0], rows[r, 1] = acc, int(ctx.sum())    # what the state and what the pages remember
            self.state[slot] = (start + b - a, acc)
        return rows[np.asarray(logit_rows, dtype=np.int64)]


def test_forced_steps_keep_pages_and_slots_straight():
    """LLMEngine.forced_step on a double: mixed batches, a request that sits out, requests that end
    and hand their pages and slot to newcomers; every wanted row equals what the request alone gives."""
    import numpy as np
    from mi355_decode.engine import LLMEngine
    runner = _StatefulRunner(num_blocks=12, max_num_seqs=3, max_model_len=96, slots=3)
    eng = LLMEngine(runner, max_num_seqs=3, max_num_batched_tokens=1 << 20, max_model_len=96)
    rng = np.random.default_rng(0)
    toks = {r: rng.integers(0, 50, n).tolist() for r, n in (("a", 40), ("b", 17), ("c", 5), ("d", 33), ("e", 64))}

    def alone(t):
        acc, out = 0, []
        for i, x in enumerate(t):
            acc = (acc * 31 + x + 1) % 1000003
            out.append((acc, sum(t[: i + 1])))
        return out

    plan = [([("a", 16), ("b", 2), ("c", 5)], ["c"]), ([("a", 1), ("d", 20)], []), ([("a", 23), ("b", 15), ("d", 1)], ["a", "b"]),
            ([("d", 12), ("e", 64)], ["d", "e"])]
    at = {r: 0 for r in toks}
    for entries, end in plan:
        req = [(r, toks[r][at[r]:at[r] + n], [0, n - 1] if n > 1 else [0]) for r, n in entries]
        out = eng.forced_step(req, end)
        row = 0
        for r, t, want in req:
            for j in want:
                assert tuple(out[row][:2]) == tuple(float(v) for v in alone(toks[r])[at[r] + j]), (r, j)
                row += 1
            at[r] += len(t)
        assert row == out.shape[0]
    assert all(at[r] == len(toks[r]) for r in toks)
    assert runner.batches == [[16, 2, 5], [1, 20], [23, 15, 1], [12, 64]]
    assert eng.alloc.num_free == 12 and eng.slots.num_free == 3 and not eng.seqs
    with pytest.raises(ValueError):
        eng.forced_step([("z", [99], [0])])                      # outside the vocabulary
