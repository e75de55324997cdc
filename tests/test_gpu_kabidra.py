"""Kabidra through the engine against the plain restatement in oracle/kabidra_oracle.py.

Every test makes its own small configuration and weights.  The engine is built on a directory that holds config.json
(and, where the weights are made by the test, model.safetensors), as a user's would be; steps are given with
Engine.run_given (the replay entry point) or chosen by the scheduler (Engine.step / LLM.generate).  Comparisons are in
float32 unless a test says otherwise: there a structural fault (a key too many, a lost state) stands far above rounding.
"""
import asyncio
import json
import os

import numpy as np
import pytest
import torch

from oracle import kabidra_oracle as ko

pytestmark = pytest.mark.gpu

GRU = {"type": "mingru", "mixer": {"width": 48}, "mlp": {"kind": "dense", "ff": 80}}
ATT = {"type": "latent_attention", "mixer": {"heads": 3, "dim": 16, "vdim": 24, "q_rank": 40, "kv_rank": 24, "scale": 0.3},
       "mlp": {"kind": "dense", "ff": 56}}


def make_cfg(layers, width=32, vocab=61, taps=3, eps=1e-5):
    return {"architecture": "Kabidra", "vocab": vocab, "width": width, "norm": {"eps": eps}, "canon": {"taps": taps},
            "layers": json.loads(json.dumps(layers))}


def model_dir(tmp_path, cfg, weights=None, name="m"):
    d = tmp_path / name
    d.mkdir()
    (d / "config.json").write_text(json.dumps(cfg))
    if weights is not None:
        from safetensors.torch import save_file
        save_file({k: v.to(torch.bfloat16).contiguous() for k, v in weights.items()}, str(d / "model.safetensors"))
    return str(d)


def weights_of(cfg, seed=0):
    """The weights an engine built on a directory without a checkpoint draws for `seed`."""
    from nano_vllm_x_amd.kabidra import KabidraConfig, random_checkpoint
    return dict(random_checkpoint(KabidraConfig.from_dict(cfg), seed))


def make_engine(path, dtype="float32", pool=2048, max_bs=4, seed=0, **kw):
    from nano_vllm_x_amd.core.engine import Engine
    return Engine(model=path, gpu_memory_utilization=0.5, max_bs=max_bs, enforce_eager=True, context_len=pool, kv_cache_size=pool,
                  dtype=dtype, seed=seed, **kw)


def replay(engine, requests, schedule):
    """requests: id -> tokens; schedule: list of steps, each a list of (id, n).  Logits of every token, id -> (T, vocab)."""
    from nano_vllm_x_amd.core.common import SamplingParams
    at = {i: 0 for i in requests}
    rows = {i: [] for i in requests}
    for step in schedule:
        plan, want = [], []
        for i, n in step:
            piece = list(requests[i][at[i]:at[i] + n])
            if engine.scheduler.get_sequence(i) is None:
                engine.add_sequence(i, piece, SamplingParams(ignore_eos=True))
            else:
                engine.extend_sequence(i, piece)
            plan.append((i, n))
            want.append(list(range(n)))
        out = engine.run_given(plan, want).float().cpu()
        k = 0
        for i, n in step:
            rows[i].append(out[k:k + n])
            k += n
            at[i] += n
            if at[i] == len(requests[i]):
                engine.abort_sequence(i)
    return {i: torch.cat(r) for i, r in rows.items()}


def close(got, want, tol, what=""):
    got, want = got.double(), want.double()
    scale = want.std().item() + 1e-12
    err = (got - want).abs().max().item() / scale
    assert err < tol, f"{what}: max error {err:.3e} of the logits' spread (tolerance {tol})"


def tokens(n, vocab, seed):
    return torch.randint(0, vocab, (n,), generator=torch.Generator().manual_seed(seed)).tolist()


F32_TOL = 2e-4


# ---- each mechanism alone ------------------------------------------------------------------------------------------
@pytest.mark.parametrize("fmt", [torch.float32, torch.bfloat16, torch.float16])
def test_boundary_norm_against_its_equations(fmt):
    from nano_vllm_x_amd import ops
    g = torch.Generator().manual_seed(1)
    t, w, slots = 7, 100, 4
    m = torch.randn(t, w, generator=g).to(fmt)
    res, w_post, w_pre = torch.randn(t, w, generator=g), 0.3 * torch.randn(w, generator=g), 0.3 * torch.randn(w, generator=g)
    hist = torch.randn(slots, t, w, generator=g)
    mix = torch.randn(3, generator=g)
    eps = 1e-3
    hd = hist.cuda()
    x, y = ops.boundary_norm(m.cuda(), w_post.cuda(), eps, res=res.cuda(), hist=hd, hist_slot=2, mix=mix.cuda(), w_pre=w_pre.cuda())
    r = res + ko.norm_zero_centred(m.float(), w_post, eps)
    want_x = mix[0] * hist[0] + mix[1] * hist[1] + mix[2] * r
    assert torch.allclose(hd[2].cpu(), r, atol=1e-5) and torch.equal(hd[3].cpu(), hist[3])
    assert torch.allclose(x.cpu(), want_x, atol=1e-5)
    assert torch.allclose(y.cpu(), ko.norm_zero_centred(want_x, w_pre, eps), atol=1e-5)
    # no residual, no mixing, the pre-norm in the activations' format
    x, y = ops.boundary_norm(m.cuda(), w_post.cuda(), eps, w_pre=w_pre.cuda(), pre_f32=False)
    want_x = ko.norm_zero_centred(m.float(), w_post, eps)
    assert y.dtype == fmt and torch.allclose(x.cpu(), want_x, atol=1e-5)
    assert torch.allclose(y.float().cpu(), ko.norm_zero_centred(want_x, w_pre, eps), atol=2e-2 if fmt != torch.float32 else 1e-5)


def _layout(ops, lens, pos0, slots, decode=False):
    n = len(lens)
    p, s = torch.tensor(pos0, dtype=torch.int64).cuda(), torch.tensor(slots, dtype=torch.int32).cuda()
    if decode:
        return ops.StepLayout(n, n, p, s)
    qo = np.zeros(n + 1, dtype=np.int32)
    np.cumsum(lens, out=qo[1:])
    tok = np.repeat(np.arange(n, dtype=np.int32), lens)
    return ops.StepLayout(int(qo[-1]), n, p, s, torch.from_numpy(qo).cuda(), torch.from_numpy(tok).cuda())


@pytest.mark.parametrize("taps", [1, 2, 4, 6, 10])
def test_canon_conv_continues_over_cuts_of_every_length(taps):
    """Two sequences in slots that are not in order, cut into steps of 1, 2, taps - 1, taps and more tokens; a third
    sequence later takes over a used slot and must not see what is left there."""
    from nano_vllm_x_amd import ops
    g = torch.Generator().manual_seed(taps)
    w = 70
    k = torch.randn(w, taps, generator=g)
    full = {0: torch.randn(23, w, generator=g), 1: torch.randn(17, w, generator=g)}
    want = {i: ko.canon(h, k) for i, h in full.items()}
    state = torch.full((3, taps - 1, w), 7.0).cuda() if taps > 1 else None
    slot = {0: 2, 1: 0}
    cuts = {0: [1, 2, max(taps - 1, 1), taps, 1, 1, 23], 1: [5, 1, 1, 2, 17]}
    at = {0: 0, 1: 0}
    got = {0: [], 1: []}
    while any(at[i] < len(full[i]) for i in full):
        live = [i for i in full if at[i] < len(full[i])]
        lens = [min(cuts[i].pop(0), len(full[i]) - at[i]) for i in live]
        h = torch.cat([full[i][at[i]:at[i] + n] for i, n in zip(live, lens)])
        decode = all(n == 1 for n in lens)
        out = ops.canon_conv(h.cuda(), k.t().contiguous().cuda(), state, _layout(ops, lens, [at[i] for i in live], [slot[i] for i in live], decode),
                             torch.float32).cpu()
        o = 0
        for i, n in zip(live, lens):
            got[i].append(out[o:o + n])
            o += n
            at[i] += n
    for i in full:
        assert torch.allclose(torch.cat(got[i]), want[i], atol=1e-5), f"sequence {i}"
    fresh = torch.randn(5, w, generator=g)
    out = ops.canon_conv(fresh.cuda(), k.t().contiguous().cuda(), state, _layout(ops, [5], [0], [2]), torch.float32).cpu()
    assert torch.allclose(out, ko.canon(fresh, k), atol=1e-5), "a sequence at position 0 must not read the slot's old tail"


@pytest.mark.parametrize("taps,width", [(1, 8), (2, 1028), (4, 96), (5, 2052)])
def test_boundary_norm_with_the_convolution_of_a_decode_step(taps, width):
    """One token per sequence, step after step: the fused launch against norm + convolution over the whole history.  The
    second sequence starts two steps later in a slot that holds another sequence's tail."""
    from nano_vllm_x_amd import ops
    g = torch.Generator().manual_seed(taps)
    steps, eps = 7, 1e-4
    k = torch.randn(width, taps, generator=g)
    w_post, w_pre = 0.2 * torch.randn(width, generator=g), 0.2 * torch.randn(width, generator=g)
    m = torch.randn(2, steps, width, generator=g)
    res = torch.randn(2, steps, width, generator=g)
    start = [0, 2]
    want = []
    for b in range(2):
        x = res[b, start[b]:] + ko.norm_zero_centred(m[b, start[b]:], w_post, eps)
        want.append(ko.canon(ko.norm_zero_centred(x, w_pre, eps), k))
    state = torch.full((3, taps - 1, width), 9.0).cuda() if taps > 1 else None
    kt = k.t().contiguous().cuda()
    for s in range(steps):
        live = [b for b in range(2) if s >= start[b]]
        lay = _layout(ops, [1] * len(live), [s - start[b] for b in live], [2 - b for b in live], decode=True)
        x, y = ops.boundary_norm(torch.stack([m[b, s] for b in live]).cuda(), w_post.cuda(), eps, res=torch.stack([res[b, s] for b in live]).cuda(),
                                 w_pre=w_pre.cuda(), canon=(kt, state, lay))
        for i, b in enumerate(live):
            assert torch.allclose(y[i].cpu(), want[b][s - start[b]], atol=2e-5), (b, s)
            assert torch.allclose(x[i].cpu(), res[b, s] + ko.norm_zero_centred(m[b, s], w_post, eps), atol=1e-5)


@pytest.mark.parametrize("width", [24, 64, 130])
def test_mingru_scan_over_cuts_and_round_borders(width):
    """The scan works in rounds of 128 tokens: lengths around one and several rounds, steps of one token, a long memory
    (update gates near zero) so that a lost or stale state shows."""
    from nano_vllm_x_amd import ops
    g = torch.Generator().manual_seed(width)
    n_tok = {0: 300, 1: 129, 2: 128}
    pre = {i: (torch.randn(n, width, generator=g) - 3.0, 2 * torch.randn(n, width, generator=g), torch.randn(n, width, generator=g))
           for i, n in n_tok.items()}
    want = {i: ko.gru_scan(*p)[0] for i, p in pre.items()}
    state = torch.full((4, width), 5.0).cuda()
    slot = {0: 3, 1: 1, 2: 0}
    cuts = {0: [127, 1, 1, 128, 2, 41], 1: [128, 1], 2: [128]}
    at = {i: 0 for i in pre}
    got = {i: [] for i in pre}
    while any(at[i] < n_tok[i] for i in pre):
        live = [i for i in pre if at[i] < n_tok[i]]
        lens = [min(cuts[i].pop(0), n_tok[i] - at[i]) for i in live]
        zxg = torch.cat([torch.cat([p[at[i]:at[i] + n] for p in pre[i]], 1) for i, n in zip(live, lens)])
        decode = all(n == 1 for n in lens)
        out = ops.mingru_scan(zxg.cuda(), state, _layout(ops, lens, [at[i] for i in live], [slot[i] for i in live], decode)).cpu()
        o = 0
        for i, n in zip(live, lens):
            got[i].append(out[o:o + n])
            o += n
            at[i] += n
    for i in pre:
        assert torch.allclose(torch.cat(got[i]), want[i], atol=2e-5), f"sequence {i}"
        assert torch.allclose(state[slot[i]].cpu(), ko.gru_scan(*pre[i])[1], atol=2e-5), f"state of sequence {i}"


def test_relu2():
    from nano_vllm_x_amd import ops
    x = torch.randn(5, 77)
    assert torch.allclose(ops.relu2(x.cuda()).cpu(), torch.relu(x) ** 2)
    assert torch.allclose(ops.relu2(x.bfloat16().cuda()).float().cpu(), (torch.relu(x.bfloat16().float()) ** 2).bfloat16().float())


@pytest.mark.parametrize("heads,rank", [(1, 8), (3, 24), (5, 300)])
def test_latent_attn_sees_exactly_the_causal_prefix(heads, rank):
    """Scores are made peaked (large scale), so that one key carries a query's output: a key too many or too few, or a
    wrong slot, changes the result by its whole size.  Slots are scattered; two sequences with cached prefixes of unequal
    length; lengths cross the kernel's tile of 256 keys."""
    from nano_vllm_x_amd import ops
    g = torch.Generator().manual_seed(rank)
    pool = torch.randn(1500, rank, generator=g)
    kv_len, q_len = [300, 517], [44, 3]
    perm = torch.randperm(1500, generator=g).to(torch.int32)
    idx = [perm[:300], perm[300:817]]
    q = torch.randn(heads, sum(q_len), rank, generator=g)
    gate = torch.rand(sum(q_len), heads, generator=g)
    scale = 1.7
    lay = _layout(ops, q_len, [a - b for a, b in zip(kv_len, q_len)], [0, 1])
    out = ops.latent_attn(q.cuda(), pool.cuda(), torch.cat(idx).cuda(), torch.tensor([0, 300], dtype=torch.int64).cuda(),
                          torch.tensor(kv_len, dtype=torch.int32).cuda(), lay, scale, gate=gate.cuda()).cpu()
    t = 0
    for b in range(2):
        c = pool[idx[b].long()].double()
        for l in range(q_len[b]):
            n = kv_len[b] - q_len[b] + l + 1
            for h in range(heads):
                p = torch.softmax(scale * (c[:n] @ q[h, t].double()), 0)
                want = (p[:, None] * c[:n]).sum(0) * gate[t, h]
                assert torch.allclose(out[h, t].double(), want, atol=1e-4), (b, l, h)
            t += 1


@pytest.mark.parametrize("fmt", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("heads,rank", [(1, 32), (3, 96), (16, 256), (20, 512), (5, 40)])
def test_latent_attn_16_bit_formats_on_the_matrix_cores(fmt, heads, rank):
    """Ranks that are multiples of 32 take the matrix-core kernel (one, several and a partly filled group of 16 heads; key
    counts that are not multiples of its tile of 16 nor of its four waves), another rank the plain one.  Against float64
    on the rounded inputs; peaked scores, scattered slots, one token per sequence (a decode step) and ragged steps."""
    from nano_vllm_x_amd import ops
    g = torch.Generator().manual_seed(rank + heads)
    pool = torch.randn(1300, rank, generator=g).to(fmt)
    perm = torch.randperm(1300, generator=g).to(torch.int32)
    for kv_len, q_len in (([300, 517, 3], [44, 3, 3]), ([1, 70, 129], [1, 1, 1])):
        idx, o = [], 0
        for n in kv_len:
            idx.append(perm[o:o + n])
            o += n
        t_all = sum(q_len)
        q = (torch.randn(heads, t_all, rank, generator=g) * 0.5).to(fmt)
        gate = torch.rand(t_all, heads, generator=g)
        scale = 3.0 / rank ** 0.5
        decode = all(n == 1 for n in q_len)
        lay = _layout(ops, q_len, [a - b for a, b in zip(kv_len, q_len)], [0, 1, 2], decode)
        starts = torch.tensor([0, kv_len[0], kv_len[0] + kv_len[1]], dtype=torch.int64)
        out = ops.latent_attn(q.cuda(), pool.cuda(), torch.cat(idx).cuda(), starts.cuda(), torch.tensor(kv_len, dtype=torch.int32).cuda(),
                              lay, scale, gate=gate.cuda()).float().cpu()
        t = 0
        for b in range(3):
            c = pool[idx[b].long()].double()
            for l in range(q_len[b]):
                n = kv_len[b] - q_len[b] + l + 1
                for h in range(heads):
                    p = torch.softmax(scale * (c[:n] @ q[h, t].double()), 0)
                    want = (p[:, None] * c[:n]).sum(0) * gate[t, h]
                    assert torch.allclose(out[h, t].double(), want, atol=3e-2 if fmt == torch.bfloat16 else 4e-3, rtol=1e-2), (b, l, h)
                t += 1


# ---- the model through the engine ----------------------------------------------------------------------------------
SCHEDULE_SHAPES = [
    ("whole", lambda n: [n]),
    ("one by one after a prompt", lambda n: [n - 9] + [1] * 9),
    ("portions", lambda n: [2, 3, 2, 37, 2, 64, 1, 1] + [31] * 40),
]


@pytest.mark.parametrize("layers", [[GRU, ATT, GRU], [ATT, ATT], [GRU]], ids=["gru-att-gru", "att-att", "gru"])
def test_logits_do_not_depend_on_how_a_prompt_is_cut(tmp_path, layers):
    cfg = make_cfg(layers)
    eng = make_engine(model_dir(tmp_path, cfg), seed=3)
    toks = tokens(300, cfg["vocab"], 5)
    want = ko.forward(weights_of(cfg, 3), cfg, toks, torch.float64)
    for name, shape in SCHEDULE_SHAPES:
        cuts, left = [], len(toks)
        for n in shape(len(toks)):
            if left <= 0:
                break
            cuts.append(min(n, left))
            left -= cuts[-1]
        got = replay(eng, {"a": toks}, [[("a", n)] for n in cuts])["a"]
        close(got, want, F32_TOL, name)
    eng.shutdown()


def test_other_sizes_one_head_no_feed_forward_equal_ranks(tmp_path):
    """Sizes that a given model may happen to make equal or one: a single head, dim != vdim, q_rank == kv_rank ==
    width, a recurrence as wide as the model, a layer without feed-forward, taps of 1 and of 5, a large eps."""
    att = {"type": "latent_attention", "mixer": {"heads": 1, "dim": 8, "vdim": 40, "q_rank": 24, "kv_rank": 24, "scale": 1.0}, "mlp": None}
    gru = {"type": "mingru", "mixer": {"width": 24}, "mlp": None}
    for taps, eps in ((1, 1e-2), (5, 1e-6)):
        cfg = make_cfg([att, gru, GRU, att], width=24, vocab=17, taps=taps, eps=eps)
        eng = make_engine(model_dir(tmp_path, cfg, name=f"m{taps}"), seed=taps)
        toks = tokens(70, 17, taps)
        want = ko.forward(weights_of(cfg, taps), cfg, toks, torch.float64)
        got = replay(eng, {"a": toks}, [[("a", 33)], [("a", 2)], [("a", 1)], [("a", 34)]])["a"]
        close(got, want, F32_TOL, f"taps {taps}")
        eng.shutdown()


def test_sizes_that_fit_no_vector_width(tmp_path):
    """Odd width, odd recurrence width, ranks and head sizes that are multiples of nothing: every kernel's plain path."""
    att = {"type": "latent_attention", "mixer": {"heads": 2, "dim": 5, "vdim": 7, "q_rank": 11, "kv_rank": 13, "scale": 0.7},
           "mlp": {"kind": "dense", "ff": 19}}
    gru = {"type": "mingru", "mixer": {"width": 25}, "mlp": {"kind": "dense", "ff": 9}}
    cfg = make_cfg([gru, att, att, gru], width=30, vocab=23, taps=4)
    cfg["width"] = 27
    toks = tokens(150, 23, 8)
    want = ko.forward(weights_of(cfg, 4), cfg, toks, torch.float64)
    for dtype, tol in (("float32", F32_TOL), ("bfloat16", 0.15)):
        eng = make_engine(model_dir(tmp_path, cfg, name=dtype), dtype=dtype, seed=4)
        got = replay(eng, {"a": toks}, [[("a", 100)], [("a", 3)]] + [[("a", 1)]] * 47)["a"]
        close(got, want, tol, dtype)
        eng.shutdown()


def test_unequal_requests_in_one_batch_and_slots_that_change_hands(tmp_path):
    """Four live requests at most, in a pool that holds less than all of them: portions beside single tokens, requests
    that end and whose token slots and state slot go to the next one.  Every request against itself alone."""
    cfg = make_cfg([GRU, ATT, GRU, ATT])
    eng = make_engine(model_dir(tmp_path, cfg), pool=420, seed=1)
    reqs = {i: tokens(n, cfg["vocab"], 10 + k) for k, (i, n) in enumerate([("a", 200), ("b", 41), ("c", 1), ("d", 90), ("e", 150), ("f", 33)])}
    schedule = [
        [("a", 2), ("c", 1), ("b", 30), ("d", 3)],            # c ends: its slots are free from here on
        [("a", 60), ("b", 1), ("d", 1), ("e", 29)],
        [("a", 1), ("b", 10), ("d", 86), ("e", 2)],           # b and d end
        [("a", 100), ("e", 1), ("f", 2)],
        [("f", 31), ("a", 37), ("e", 118)],                   # all end
    ]
    got = replay(eng, reqs, schedule)
    w = weights_of(cfg, 1)
    for i, toks in reqs.items():
        close(got[i], ko.forward(w, cfg, toks, torch.float64), F32_TOL, f"request {i}")
    assert eng.scheduler.state_slots.num_free() == 4 and eng.scheduler.kv_manager.kv_cache_allocator.num_free() == 420
    eng.shutdown()


def _needle_weights(cfg, seed):
    """Weights under which a fault shows: update gates near zero (the recurrence remembers hundreds of tokens), large
    taps, and attention queries and keys scaled up so that single scores stand out."""
    w = weights_of(cfg, seed)
    for name in w:
        if name.endswith("mix.z.b"):
            w[name] = w[name] - 4.0
        if name.endswith(("canon1", "canon2")):
            w[name] = w[name] * 3.0
        if name.endswith(("mix.uq", "mix.uk")):
            w[name] = w[name] * 2.5
    return {k: v.to(torch.bfloat16).float() for k, v in w.items()}


def test_far_keys_and_old_state_count(tmp_path):
    """A long prompt with sharpened weights, its last tokens one by one: the first token, a key hundreds of tokens back
    and the state carried all the way decide the last logits."""
    cfg = make_cfg([GRU, ATT, GRU, ATT])
    w = _needle_weights(cfg, 7)
    eng = make_engine(model_dir(tmp_path, cfg, w), seed=0)
    toks = tokens(600, cfg["vocab"], 2)
    want = ko.forward(w, cfg, toks, torch.float64)
    got = replay(eng, {"a": toks}, [[("a", 255)], [("a", 1)], [("a", 1)], [("a", 2)], [("a", 300)]] + [[("a", 1)]] * 41)["a"]
    close(got, want, F32_TOL, "sharpened")
    # the same prompt without its first token is another function of the rest: the first token is seen
    other = ko.forward(w, cfg, toks[1:], torch.float64)
    assert (other[-1] - want[-1]).abs().max() > 100 * F32_TOL * want.std()
    eng.shutdown()


def test_bfloat16_and_float16_stay_within_rounding(tmp_path):
    cfg = make_cfg([GRU, ATT, GRU])
    toks = tokens(120, cfg["vocab"], 4)
    want = ko.forward(weights_of(cfg, 2), cfg, toks, torch.float64)
    for dtype in ("bfloat16", "float16"):
        eng = make_engine(model_dir(tmp_path, cfg, name=dtype), dtype=dtype, seed=2)
        got = replay(eng, {"a": toks}, [[("a", 50)], [("a", 2)]] + [[("a", 1)]] * 68)["a"]
        close(got, want, 0.12 if dtype == "bfloat16" else 0.03, dtype)
        eng.shutdown()


def test_checkpoint_with_a_missing_or_misshapen_tensor_is_refused(tmp_path):
    cfg = make_cfg([GRU])
    w = weights_of(cfg, 0)
    bad = dict(w)
    del bad["l0.mix.x.b"]
    with pytest.raises(KeyError):
        make_engine(model_dir(tmp_path, cfg, bad, name="missing"))
    bad = dict(w)
    bad["l0.canon1"] = torch.zeros(cfg["width"], cfg["canon"]["taps"] + 1)
    with pytest.raises(ValueError):
        make_engine(model_dir(tmp_path, cfg, bad, name="shape"))


# ---- generation: the scheduler's own choices ---------------------------------------------------------------------------
def oracle_greedy(w, cfg, prompt, n_new):
    toks = list(prompt)
    for _ in range(n_new):
        toks.append(int(ko.forward(w, cfg, toks, torch.float64)[-1].argmax()))
    return toks[len(prompt):]


@pytest.mark.parametrize("chunked", [False, True], ids=["whole prompts", "chunked prefill"])
def test_greedy_generation_through_the_engine(tmp_path, chunked):
    """Prompts of unequal length admitted together, decoded as one batch; more requests than state slots, so the later
    ones wait for a slot that an earlier one gives back; with chunked prefill the prompts are computed in portions of
    seven tokens.  Long decoding (40 tokens) for one of them."""
    from nano_vllm_x_amd.core.common import SamplingParams
    cfg = make_cfg([GRU, ATT, GRU])
    kw = dict(max_prefill_tokens=7, chunked_prefill=True) if chunked else {}
    eng = make_engine(model_dir(tmp_path, cfg), pool=400, max_bs=3, seed=9, **kw)
    w = weights_of(cfg, 9)
    prompts = {f"r{k}": tokens(n, cfg["vocab"], 20 + k) for k, n in enumerate([5, 23, 1, 12, 9])}
    new = {"r0": 40, "r1": 6, "r2": 9, "r3": 4, "r4": 7}
    for i, p in prompts.items():
        eng.add_sequence(i, list(p), SamplingParams(temperature=0.0, ignore_eos=True, max_new_tokens=new[i]))
    out = {i: [] for i in prompts}
    steps = 0
    while eng.has_unfinished_sequences():
        for o in eng.step():
            out[o.seq_id].append(o.new_token_id)
        steps += 1
        assert steps < 400
    for i, p in prompts.items():
        assert out[i] == oracle_greedy(w, cfg, p, new[i]), i
    assert eng.scheduler.state_slots.num_free() == 3
    eng.shutdown()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_decode_steps_replay_a_captured_graph(tmp_path, dtype):
    """With graphs on, every decode step replays the graph of its batch size, with prefill steps of later requests (eager
    work on the same cache and state) between the replays; batch sizes change as requests end.  float32: the tokens are
    the restatement's; bfloat16: the graph's tokens are those of eager steps (same kernels, same order)."""
    from nano_vllm_x_amd.core.common import SamplingParams
    from nano_vllm_x_amd.core.engine import Engine
    cfg = make_cfg([GRU, ATT, GRU, ATT])
    path = model_dir(tmp_path, cfg)
    prompts = {f"r{k}": tokens(n, cfg["vocab"], 40 + k) for k, n in enumerate([9, 30, 2, 17, 5])}
    new = {"r0": 25, "r1": 5, "r2": 12, "r3": 3, "r4": 8}

    def run(eager):
        eng = Engine(model=path, gpu_memory_utilization=0.5, max_bs=3, enforce_eager=eager, context_len=128, kv_cache_size=300,
                     dtype=dtype, seed=5)
        for i, p in prompts.items():
            eng.add_sequence(i, list(p), SamplingParams(temperature=0.0, ignore_eos=True, max_new_tokens=new[i]))
        out = {i: [] for i in prompts}
        while eng.has_unfinished_sequences():
            for o in eng.step():
                out[o.seq_id].append(o.new_token_id)
        stats = dict(eng.model_runner.stats)
        eng.shutdown()
        return out, stats

    got, stats = run(False)
    assert stats["graph_steps"] > 20 and stats["eager_decode_steps"] == 0
    if dtype == "float32":
        w = weights_of(cfg, 5)
        for i, p in prompts.items():
            assert got[i] == oracle_greedy(w, cfg, p, new[i]), i
    else:
        assert got == run(True)[0]


def test_decode_steps_queued_ahead_give_the_same_tokens(tmp_path):
    """run_ahead: decode step N+1 is queued before step N's ids reach the host; the rows' state slots and slot lists of both
    steps are in flight at once."""
    from nano_vllm_x_amd.core.common import SamplingParams
    from nano_vllm_x_amd.core.engine import Engine
    cfg = make_cfg([GRU, ATT, GRU])
    path = model_dir(tmp_path, cfg)
    eng = Engine(model=path, gpu_memory_utilization=0.5, max_bs=3, enforce_eager=False, context_len=128, kv_cache_size=300, dtype="float32",
                 seed=8, run_ahead=True)
    prompts = {f"r{k}": tokens(n, cfg["vocab"], 60 + k) for k, n in enumerate([7, 19, 3])}
    new = {"r0": 21, "r1": 9, "r2": 15}
    for i, p in prompts.items():
        eng.add_sequence(i, list(p), SamplingParams(temperature=0.0, ignore_eos=True, max_new_tokens=new[i]))
    out = {i: [] for i in prompts}
    while eng.has_unfinished_sequences() or eng.step_in_flight:
        for o in eng.step_overlapped():
            out[o.seq_id].append(o.new_token_id)
    assert eng.ahead_steps > 5
    w = weights_of(cfg, 8)
    for i, p in prompts.items():
        assert out[i] == oracle_greedy(w, cfg, p, new[i]), i
    eng.shutdown()


def test_generate_entry_point(tmp_path):
    from nano_vllm_x_amd import LLM, SamplingParams
    cfg = make_cfg([ATT, GRU], vocab=300)
    llm = LLM(model_dir(tmp_path, cfg), gpu_memory_utilization=0.5, max_bs=2, enforce_eager=True, context_len=256, kv_cache_size=256,
              dtype="float32", seed=4)
    prompt = tokens(11, 300, 1)

    async def run():
        ids = []
        async for o in llm.generate(list(prompt), SamplingParams(temperature=0.0, ignore_eos=True, max_new_tokens=5, eos_token_id=0)):
            ids.append(o.token_id)
        return ids

    assert asyncio.run(run()) == oracle_greedy(weights_of(cfg, 4), cfg, prompt, 5)
    llm.shutdown()


def test_preempted_sequence_starts_again_from_an_empty_state(tmp_path):
    from nano_vllm_x_amd.core.common import SamplingParams
    cfg = make_cfg([GRU, ATT])
    eng = make_engine(model_dir(tmp_path, cfg), pool=64, max_bs=2, seed=6)
    w = weights_of(cfg, 6)
    prompts = {"a": tokens(20, cfg["vocab"], 1), "b": tokens(25, cfg["vocab"], 2)}
    for i, p in prompts.items():
        eng.add_sequence(i, list(p), SamplingParams(temperature=0.0, ignore_eos=True, max_new_tokens=14))
    out = {i: [] for i in prompts}
    while eng.has_unfinished_sequences():       # 45 + 2 * 14 tokens do not fit 64 slots: the younger sequence is preempted
        for o in eng.step():
            out[o.seq_id].append(o.new_token_id)
    for i, p in prompts.items():
        assert out[i] == oracle_greedy(w, cfg, p, 14), i
    eng.shutdown()


def test_command_line_generates_what_the_restatement_does(tmp_path):
    import subprocess
    import sys
    cfg = make_cfg([GRU, ATT], vocab=90)
    path = model_dir(tmp_path, cfg)
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    out = subprocess.run([sys.executable, "-m", "nano_vllm_x_amd", "--model", path, "--prompt-ids", "5,17,3,44", "--prompt-ids", "8",
                          "--max-new-tokens", "6", "--dtype", "float32", "--kv-cache-size", "128", "--context-len", "64", "--max-bs", "2",
                          "--seed", "3"], cwd=root, capture_output=True, text=True, timeout=300)
    assert out.returncode == 0, out.stderr[-2000:]
    lines = [json.loads(x) for x in out.stdout.splitlines() if x.startswith("{")]
    w = weights_of(cfg, 3)
    assert [x["prompt"] for x in lines] == [[5, 17, 3, 44], [8]]
    for x in lines:
        assert x["generated_ids"] == oracle_greedy(w, cfg, x["prompt"], 6)
