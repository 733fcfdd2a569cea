"""Sigudra (sequential post-norm layered decoder) against the plain oracle of tests/sigudra_oracle.py.

Small configurations with random weights made here; the framework side always runs through the
engine (scheduler admission, pages, state slots, runner) or the ops' public entry points.  CPU
tensors exercise the ops' PyTorch forms, ``cuda`` ones the HIP kernels (marked gpu).
"""
import copy

import pytest
import torch

import sigudra_oracle as oracle
from financial_chatbot_llm_amd.config import EngineConfig
from financial_chatbot_llm_amd.engine import LLMEngine, SamplingParams
from financial_chatbot_llm_amd.models import mixers as blocks
from financial_chatbot_llm_amd.models.configs import layered_config
from financial_chatbot_llm_amd.models.sigudra import SigudraModel, example_config
from financial_chatbot_llm_amd.ops import mixers as mx

DEVICES = ["cpu", pytest.param("cuda", marks=pytest.mark.gpu)]
DTYPES = [torch.float32, torch.bfloat16]
TOL = {torch.float32: 3e-4, torch.bfloat16: 8e-2}


def random_weights(model, seed, ranks=(6, 5)):
    g = torch.Generator().manual_seed(seed)
    sd = {}
    for name, shape in model.full_shapes().items():
        leaf = name.rsplit(".", 1)[-1]
        r = torch.randn(shape, generator=g)
        if leaf in ("norm1", "norm2", "norm", "out") and len(shape) == 1:
            t = 1.0 + 0.2 * r
        elif leaf == "A_log":
            t = torch.log(0.3 + 2 * torch.rand(shape, generator=g))
        elif leaf == "dt_bias":
            t = -2.0 + r
        elif leaf == "lam":
            t = -1.5 + r
        elif name.endswith("a2.b"):
            t = 3.0 + r
        elif leaf == "b" and (len(shape) == 1 or name.endswith(("ra.b", "ri.b"))):
            t = 0.3 * r
        elif leaf == "conv":
            t = 0.6 * r
        elif leaf in ("embed", "bigram"):
            t = r
        else:
            t = r * shape[-1] ** -0.5 * 1.3
        sd[name] = t.to(torch.bfloat16)
    return sd


def small_config(pattern="dGPg", **over):
    c = example_config(width=over.pop("width", 96), vocab=over.pop("vocab", 160), pattern=pattern)
    for l in c["layers"]:
        for k, v in over.items():
            if k in l["mixer"]:
                l["mixer"][k] = v
    return c


def build(cfgd, device, dtype, seed=1, blocks_=24, seqs=4, graphs=False, async_=False, max_len=1024):
    mc = layered_config(cfgd, "sigudra-test")
    model = SigudraModel(mc, device=device, dtype=dtype)
    sd = random_weights(model, seed)
    model.load_state(sd)
    eng = LLMEngine(EngineConfig(model="sigudra-test", device=device, dtype="fp32" if dtype == torch.float32 else "bf16",
                                 num_kv_blocks=blocks_, max_num_seqs=seqs, max_model_len=max_len,
                                 max_num_batched_tokens=512, enable_prefix_caching=False, use_cuda_graph=graphs,
                                 async_scheduling=async_, graph_batch_sizes=(1, 2, 4)), model=model)
    return eng, sd


def _poison(entry):
    for t in entry[1:]:
        if isinstance(t, dict):
            for v in t.values():
                v.fill_(float("nan"))
        elif isinstance(t, tuple):
            _poison(t)
        else:
            t.fill_(float("nan"))


def poison(eng):
    """Pages and slots as a previous owner might have left them: nothing may depend on their content."""
    for lay in eng.kv.layers:
        _poison(lay)
    eng.kv.model["last_token"].fill_(123456)


def close(got, want, dtype, flips=None):
    """``flips``: the share of positions that may be off (bf16 runs with many experts: a rounding of the
    router's input can swap two experts whose scores nearly tie)."""
    got, want = got.double().cpu(), want.double().cpu()
    assert torch.isfinite(got).all()
    if flips is None:
        flips = 0.0 if dtype == torch.float32 else 0.05
    err = (got - want).abs().flatten(1).max(-1).values / max(want.abs().max().item(), 1e-9)
    bad = int((err > TOL[dtype]).sum())
    assert bad <= flips * err.numel(), f"{bad} of {err.numel()} positions over {TOL[dtype]}: worst {err.max().item():.3e}"


def tokens(n, vocab, seed):
    return torch.randint(0, vocab, (n,), generator=torch.Generator().manual_seed(seed)).tolist()


def run_whole(eng, rid, toks):
    return eng.replay_step([(rid, toks, list(range(len(toks))))], [rid])


# ---------------------------------------------------------------------------------------------------
# each mechanism alone: one-layer models
# ---------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("pattern", ["d", "g", "p", "G"])
def test_one_layer_against_oracle(device, dtype, pattern):
    cfgd = small_config(pattern)
    eng, sd = build(cfgd, device, dtype)
    poison(eng)
    toks = tokens(90, cfgd["vocab"], 3)          # crosses a 64-token page and the 37-token window
    close(run_whole(eng, "r", toks), oracle.forward(cfgd, sd, toks), dtype)


@pytest.mark.parametrize("device", DEVICES)
def test_residual_stream_after_every_layer(device):
    cfgd = small_config("dPg")
    eng, sd = build(cfgd, device, torch.float32)
    toks = tokens(40, cfgd["vocab"], 4)
    want = []
    oracle.forward(cfgd, sd, toks, want)
    eng.model.capture = []
    run_whole(eng, "r", toks)
    for got, ref in zip(eng.model.capture, want):
        close(got, ref, torch.float32)


@pytest.mark.parametrize("device", DEVICES)
def test_no_feed_forward_no_mask_no_pairs_single_sizes(device):
    """mlp: null, no mask entry (plain causal), no pair embedding, one head, one block, two taps,
    top 1, tau 1."""
    cfgd = small_config("dpgG")
    del cfgd["embedding"]
    cfgd["layers"][0]["mlp"] = None
    cfgd["layers"][0]["mixer"].update(heads=1, kv_heads=1, conv=2)
    del cfgd["layers"][1]["mixer"]["left"]["mask"]
    cfgd["layers"][1]["mixer"]["left"].update(heads=1, kv_heads=1)
    cfgd["layers"][1]["mixer"]["right"].update(blocks=1, conv=1)
    cfgd["layers"][2]["mixer"].update(heads=1, tau=1.0)
    cfgd["layers"][3]["mlp"]["router"].update(top=1)
    eng, sd = build(cfgd, device, torch.float32)
    poison(eng)
    toks = tokens(70, cfgd["vocab"], 5)
    close(run_whole(eng, "r", toks), oracle.forward(cfgd, sd, toks), torch.float32)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
def test_other_sizes(device, dtype):
    """Sizes unlike the small default: odd head counts, key and value sizes that fill no wave and differ,
    a key size above 128, a window longer than a page, seven-tap convolutions, many experts, other
    hashing constants."""
    cfgd = small_config("PdGg", width=80, vocab=97)
    cfgd["embedding"]["bigram"].update(buckets=64, mul_prev=1, mul_cur=1000003)
    for l in cfgd["layers"]:
        if l["type"] == "parallel":
            l["mixer"]["left"].update(dim=12, vdim=70, heads=6, kv_heads=1, mask={"size": 70}, scale=0.31)
            l["mixer"]["right"].update(width=55, blocks=5, conv=7)
        elif l["type"] == "channel_delta":
            l["mixer"].update(heads=3, kv_heads=3, dim=33, vdim=9, conv=7)
        else:
            l["mixer"].update(heads=2, dim=132, vdim=17, tau=3.0)
        if l["mlp"]["kind"] == "moe":
            l["mlp"]["router"].update(experts=70, top=5)
            l["mlp"]["expert"].update(ff=20)
    eng, sd = build(cfgd, device, dtype, blocks_=8)
    poison(eng)
    toks = tokens(150, cfgd["vocab"], 7)
    close(run_whole(eng, "r", toks), oracle.forward(cfgd, sd, toks), dtype, flips=0.0 if dtype == torch.float32 else 0.15)


@pytest.mark.parametrize("device", DEVICES)
def test_first_tokens(device):
    """Sequences of one and two tokens, and the first tokens of a longer one, each request alone."""
    cfgd = small_config("dGPg")
    eng, sd = build(cfgd, device, torch.float32)
    poison(eng)
    for n in (1, 2, 5):
        toks = tokens(n, cfgd["vocab"], 60 + n)
        close(run_whole(eng, f"r{n}", toks), oracle.forward(cfgd, sd, toks), torch.float32)


# ---------------------------------------------------------------------------------------------------
# cache, state, batching
# ---------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
def test_prefill_then_token_by_token(device, dtype):
    cfgd = small_config("dGPg")
    eng, sd = build(cfgd, device, dtype)
    poison(eng)
    toks = tokens(130, cfgd["vocab"], 11)
    want = oracle.forward(cfgd, sd, toks)
    got = [eng.replay_step([("r", toks[:40], list(range(40)))])]
    for i in range(40, len(toks)):               # long decoding: over the window and a page border
        got.append(eng.replay_step([("r", toks[i:i + 1], [0])], ["r"] if i == len(toks) - 1 else []))
    close(torch.cat(got), want, dtype)
    assert eng.bm.num_free() == eng.bm.num_blocks and eng.state_slots.num_free() == 4


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("sizes", [[2, 2, 3, 60, 2, 1, 1, 64, 5], [63, 1, 1, 2, 70], [1, 1, 1, 130], [2] * 20])
def test_portions(device, sizes):
    cfgd = small_config("gPDp")
    eng, sd = build(cfgd, device, torch.float32)
    poison(eng)
    toks = tokens(sum(sizes), cfgd["vocab"], 13)
    want = oracle.forward(cfgd, sd, toks)
    got, at = [], 0
    for n in sizes:
        got.append(eng.replay_step([("r", toks[at:at + n], list(range(n)))]))
        at += n
    close(torch.cat(got), want, torch.float32)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
def test_mixed_batches_and_reuse(device, dtype):
    """Unequal requests in one batch (portions beside single tokens), more requests than slots and a
    pool that only fits what is live: pages and slots are freed and used again."""
    cfgd = small_config("pDgP")
    eng, sd = build(cfgd, device, dtype, blocks_=7, seqs=3)
    poison(eng)
    V = cfgd["vocab"]
    reqs = {f"q{i}": tokens(n, V, 20 + i) for i, n in enumerate([150, 70, 33, 100, 5, 64])}
    want = {k: oracle.forward(cfgd, sd, t) for k, t in reqs.items()}
    got = {k: [] for k in reqs}
    at = {k: 0 for k in reqs}
    sched = [
        [("q0", 50), ("q1", 3), ("q2", 33)],            # q2 complete at once
        [("q0", 1), ("q1", 60), ("q3", 2)],             # q3 takes q2's slot and pages
        [("q0", 30), ("q1", 1), ("q3", 62)],
        [("q1", 1), ("q0", 69), ("q3", 1)],
        [("q1", 5), ("q3", 35)],                        # q1, q3, q0 complete
        [("q4", 5), ("q5", 2)],
        [("q5", 62), ("q4", 0)],
    ]
    for step in sched:
        entries, end = [], []
        for k, n in step:
            if n == 0:
                continue
            entries.append((k, reqs[k][at[k]:at[k] + n], list(range(n))))
            at[k] += n
            if at[k] == len(reqs[k]):
                end.append(k)
        out = eng.replay_step(entries, end)
        o = 0
        for k, t, _ in entries:
            got[k].append(out[o:o + len(t)])
            o += len(t)
    assert eng.state_slots.reuses > 0
    assert all(at[k] == len(reqs[k]) for k in reqs)
    close(torch.cat([torch.cat(got[k]) for k in reqs]), torch.cat([want[k] for k in reqs]), dtype)


# ---------------------------------------------------------------------------------------------------
# window and page edges, far keys: scores and states that stand out
# ---------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("window", [5, 64, 70])
def test_window_edges_stand_out(device, dtype, window):
    """One key per query gets an overwhelming score: first the oldest key inside the window (the
    output must be that key's value), then the newest key outside it (the output must not show it).
    Queries sit before, on and after page borders, as rows of a prompt chunk and as single decoded
    rows; three query heads share each of two key/value heads."""
    H, G, D, P, pages, n = 6, 2, 16, 12, 4, 200
    g = torch.Generator().manual_seed(window)
    table = torch.tensor([[2, 0, 3, 1]], dtype=torch.int32)
    row = lambda j: int(table[0, j // 64]) * 64 + j % 64  # noqa: E731
    cache = torch.zeros(pages * 64, G * (D + P))
    for j in range(n):
        cache[row(j), G * D:] = torch.randn(G * P, generator=g)           # values; keys stay zero
    chunks = [list(range(p0, p0 + 8)) for p0 in (window, 60, 124, 188) if p0 >= window]
    chunks += [[p] for p in (window, 63, 64, 65, 127, 128, 199) if p >= window]
    for shift, inside in ((window - 1, True), (window, False)):
        for seg in chunks:
            m = len(seg)
            kc = cache.clone()
            q = torch.zeros(m, H, D)
            for i, p in enumerate(seg):          # query i asks for key coordinate i; only its target key is large there
                for kvh in range(G):
                    kc[row(p - shift), kvh * D + i] = 50.0
                q[i, :, i] = 4.0
            out = mx.window_attend(q.reshape(m, H * D).to(dtype).to(device), kc.to(dtype).to(device),
                                   torch.tensor([0, m], dtype=torch.int32, device=device),
                                   torch.tensor(seg, dtype=torch.int32, device=device), table.to(device), window, 1.0,
                                   m, H, G, D, P).float().cpu().view(m, H, P)
            kcr = kc.to(dtype).float()
            for i, p in enumerate(seg):
                rows_ = [row(j) for j in range(max(0, p - window + 1), p + 1)]
                for h in range(H):
                    kvh = h // (H // G)
                    pr = torch.softmax(kcr[rows_, kvh * D + i] * 4.0, 0)
                    ref = (pr[:, None] * kcr[rows_, G * D + kvh * P:G * D + (kvh + 1) * P]).sum(0)
                    tol = 1e-4 if dtype == torch.float32 else 0.05
                    assert (out[i, h] - ref).abs().max() < tol, (shift, seg, i, h)
                    target = kcr[row(p - shift), G * D + kvh * P:G * D + (kvh + 1) * P]
                    assert bool((out[i, h] - target).abs().max() < 0.05) == inside


@pytest.mark.parametrize("device", DEVICES)
def test_far_key_in_a_long_prompt_chunk_and_decoded_rows(device):
    """No window: one far key among hundreds carries the score, seen from a chunk deep in the sequence
    and from single rows; a window shorter than the distance hides it."""
    H, G, D, P = 4, 2, 24, 8
    n, pages, far = 400, 8, 7
    g = torch.Generator().manual_seed(2)
    perm = torch.randperm(pages, generator=g).to(torch.int32)[None]
    rows = 0.1 * torch.randn(n, G * (D + P), generator=g)
    rows[far, 1] = rows[far, D + 1] = 30.0                 # both key heads, coordinate 1
    rows[far, G * D:] = 9.0
    cache = torch.zeros(pages * 64, G * (D + P))
    for j in range(n):
        cache[int(perm[0, j // 64]) * 64 + j % 64] = rows[j]
    pos = torch.arange(330, 400, dtype=torch.int32)
    q = torch.zeros(len(pos), H, D)
    q[:, :, 1] = 3.0
    cu = torch.tensor([0, len(pos)], dtype=torch.int32)
    for window, hit in ((1 << 30, True), (300, False)):
        out = mx.window_attend(q.view(len(pos), -1).to(device), cache.to(device), cu.to(device), pos.to(device),
                               perm.to(device), window, 1.0, len(pos), H, G, D, P).cpu()
        assert bool((out > 8.0).all()) == hit
        for dt in DTYPES:
            one = mx.window_attend(q[:1].view(1, -1).to(dt).to(device), cache.to(dt).to(device),
                                   torch.tensor([0, 1], dtype=torch.int32, device=device),
                                   torch.tensor([399], dtype=torch.int32, device=device), perm.to(device), window, 1.0,
                                   1, H, G, D, P).float().cpu()
            assert bool((one > 8.0).all()) == hit


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("mode", ["gla", "delta"])
def test_matrix_state_keeps_a_far_write(device, mode):
    """A value written hundreds of tokens back under a decay close to one is read out by a matching query
    at the end, through portions that hand the state over in a reused slot; under a fast decay it is gone."""
    H, G, D, P, n = 2, 1, 20, 12, 300
    g = torch.Generator().manual_seed(6)
    far = 3
    # (the delta rule makes every key a unit vector and erases along it: its other keys are zero)
    k = 0.01 * torch.randn(n, G * D, generator=g) * (0.0 if mode == "delta" else 1.0)
    v = 0.01 * torch.randn(n, H * P, generator=g)
    q = torch.zeros(n, G * D)
    k[far] = 0
    k[far, 5] = 1.0
    v[far] = 7.0
    q[-1, 5] = D ** 0.5
    beta = torch.full((n, H), 10.0)
    for slow in (True, False):
        a = torch.full((n, H * D), 12.0 if mode == "gla" else -12.0) * (1 if slow else -1)
        a_bias, A_log = torch.zeros(H * D), torch.zeros(H)
        state = torch.full((3, H, D, P), float("nan")).to(device)
        outs, at = [], 0
        for m in (100, 1, 1, 2, 196):
            pos = torch.arange(at, at + m, dtype=torch.int32, device=device)
            sl = slice(at, at + m)
            outs.append(mx.matrix_scan(q[sl].to(device), k[sl].to(device), v[sl].to(device), a[sl].to(device),
                                       a_bias.to(device), state, torch.tensor([0, m], dtype=torch.int32, device=device),
                                       torch.tensor([1], dtype=torch.int32, device=device), pos, H, G, D, P, mode, tau=2.0,
                                       A_log=A_log.to(device), beta=beta[sl].to(device)).cpu())
            at += m
        last = torch.cat(outs)[-1]
        assert bool((last > 1.0).all()) == slow, last        # 7 (gla) or 7 dim^-1/2 (delta: q is a unit vector first)


@pytest.mark.parametrize("device", DEVICES)
def test_lru_state_carries_far(device):
    """The diagonal recurrence: a large input far back survives a slow decay (r small) and is forgotten
    under a fast one; also checks the first token starts from S = 0 with the sqrt(1 - a^2) factor."""
    R, Bk, n = 12, 3, 200
    u = torch.zeros(n, R)
    u[2] = 100.0
    for zr, keep in ((-8.0, True), (8.0, False)):
        z = torch.zeros(Bk, n, 2 * R // Bk)
        z[:, :, :R // Bk] = zr
        z[:, :, R // Bk:] = 20.0                          # input gate open
        state = torch.full((2, R), float("nan")).to(device)
        outs, at = [], 0
        for m in (3, 1, 96, 100):
            pos = torch.arange(at, at + m, dtype=torch.int32, device=device)
            outs.append(mx.lru_scan(u[at:at + m].to(device).contiguous(), z[:, at:at + m].to(device).contiguous(), Bk,
                                    torch.zeros(R, device=device), torch.zeros(R, device=device),
                                    torch.zeros(R, device=device), torch.full((m, R), 3.0, device=device), None, state,
                                    torch.tensor([0, m], dtype=torch.int32, device=device),
                                    torch.tensor([0], dtype=torch.int32, device=device), pos, torch.float32).cpu())
            at += m
        out = torch.cat(outs)
        assert bool((out[-1] > 1.0).all()) == keep
        assert (out[:2] == 0).all()


@pytest.mark.gpu
@pytest.mark.parametrize("lens", [[15, 16, 17, 33], [255, 257], [600, 1, 300]])
def test_segments_across_the_kernels_chunks(lens):
    """Segments whose lengths sit on and around the kernels' internal chunk sizes (16 tokens of the matrix
    scan, 16 x 16 tokens of the LRU fold), several per step, against the ops' plain forms on the CPU."""
    g = torch.Generator().manual_seed(sum(lens))
    T, S = sum(lens), len(lens)
    cu = torch.tensor([0] + torch.tensor(lens).cumsum(0).tolist(), dtype=torch.int32)
    pos = torch.cat([torch.arange(7 * i, 7 * i + n) for i, n in enumerate(lens)]).to(torch.int32)   # the first starts at 0
    slot = torch.arange(S, dtype=torch.int32).flip(0)
    dev = lambda *ts: [t.cuda() for t in ts]  # noqa: E731
    H, G, D, P = 3, 1, 40, 24
    for mode in ("gla", "delta"):
        q, k, v = torch.randn(T, G * D, generator=g), torch.randn(T, G * D, generator=g) * 0.2, torch.randn(T, H * P, generator=g)
        a = torch.randn(T, H * D, generator=g) + 3
        ab, Al, beta = torch.zeros(H * D), torch.zeros(H), torch.randn(T, H, generator=g)
        st = torch.randn(S, H, D, P, generator=g) * 0.1
        s1, s2 = st.clone(), st.clone().cuda()
        want = mx.matrix_scan(q, k, v, a.clone(), ab, s1, cu, slot, pos, H, G, D, P, mode, tau=4.0, A_log=Al, beta=beta)
        got = mx.matrix_scan(*dev(q, k, v, a.clone(), ab), s2, *dev(cu, slot, pos), H, G, D, P, mode, tau=4.0, A_log=Al.cuda(),
                             beta=beta.cuda(), max_len=max(lens))
        assert (got.cpu() - want).abs().max() <= 2e-4 * want.abs().max()
        assert (s2.cpu() - s1).abs().max() <= 2e-4 * s1.abs().max()
    R, Bk = 40, 2
    u, z = torch.randn(T, R, generator=g), torch.randn(Bk, T, 2 * R // Bk, generator=g)
    rb, ib, lam, y = torch.zeros(R), torch.zeros(R), torch.randn(R, generator=g) - 2, torch.randn(T, R, generator=g)
    st = torch.randn(S, R, generator=g)
    s1, s2 = st.clone(), st.clone().cuda()
    want = mx.lru_scan(u.clone(), z.clone(), Bk, rb, ib, lam, y, None, s1, cu, slot, pos, torch.float32)
    got = mx.lru_scan(*dev(u.clone(), z.clone()), Bk, *dev(rb, ib, lam, y), None, s2, *dev(cu, slot, pos), torch.float32,
                      max_len=max(lens))
    assert (got.cpu() - want).abs().max() <= 2e-5 * want.abs().max()
    assert (s2.cpu() - s1).abs().max() <= 2e-5 * s1.abs().max().clamp(min=1.0)


# ---------------------------------------------------------------------------------------------------
# routing, embedding
# ---------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("device", DEVICES)
def test_sigmoid_routing_weights(device):
    z = torch.tensor([[2.0, 1.0, 0.5, 0.0, -1.0], [-3.0, -2.0, -2.5, -9.0, -2.0]])
    w, i = mx.route_scores(z.to(device), 2, "sigmoid")
    assert i.cpu().tolist() == [[0, 1], [1, 4]]                       # ties: the lower index
    assert torch.allclose(w.cpu(), torch.sigmoid(torch.tensor([[2.0, 1.0], [-2.0, -2.0]])), atol=1e-6)   # not renormalised


@pytest.mark.parametrize("device", DEVICES)
def test_routed_ff_bucketed_and_dense_forms_agree(device, monkeypatch):
    cfgd = small_config("G")
    eng, sd = build(cfgd, device, torch.float32)
    toks = tokens(80, cfgd["vocab"], 31)
    want = oracle.forward(cfgd, sd, toks)
    monkeypatch.setattr(blocks, "DENSE_MAX_PAIRS", 0)          # every step buckets rows by expert
    close(run_whole(eng, "a", toks), want, torch.float32)
    monkeypatch.setattr(blocks, "DENSE_MAX_PAIRS", 1 << 30)    # every step runs all experts densely
    close(run_whole(eng, "b", toks), want, torch.float32)


@pytest.mark.parametrize("device", DEVICES)
def test_pair_embedding_rows_and_carried_token(device):
    """Row ``buckets`` for a first token; the previous token comes from the step's own rows or, at the
    start of a portion, from the slot; a slot left by another sequence is not read at position 0."""
    V, W, B = 50, 8, 13
    table = torch.zeros(V, W)
    pairs = torch.arange(B + 1, dtype=torch.float32)[:, None].expand(B + 1, W).contiguous()
    last = torch.tensor([40, 41, 42], dtype=torch.int32).to(device)
    ids = torch.tensor([7, 9, 11, 5, 6], dtype=torch.int32)
    cu = torch.tensor([0, 3, 5], dtype=torch.int32)
    slot = torch.tensor([2, 0], dtype=torch.int32)
    pos = torch.tensor([0, 1, 2, 17, 18], dtype=torch.int32)
    out = mx.embed_pairs(ids.to(device), table.to(device), pairs.to(device), 3, 4, last, cu.to(device), slot.to(device),
                         pos.to(device), 3).cpu()
    want = [B, (7 * 3 + 9 * 4) % B, (9 * 3 + 11 * 4) % B, (40 * 3 + 5 * 4) % B, (5 * 3 + 6 * 4) % B]
    assert out[:, 0].tolist() == [float(x) for x in want]
    assert last.cpu().tolist() == [6, 41, 11]


# ---------------------------------------------------------------------------------------------------
# generation through the engine's own scheduler
# ---------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("device,graphs", [("cpu", False), pytest.param("cuda", False, marks=pytest.mark.gpu),
                                           pytest.param("cuda", True, marks=pytest.mark.gpu)])
@pytest.mark.parametrize("async_", [False, True])
def test_greedy_generation(device, graphs, async_):
    cfgd = small_config("dGPg", vocab=256)
    eng, sd = build(cfgd, device, torch.float32, blocks_=12, seqs=2, graphs=graphs, async_=async_)
    poison(eng)
    prompts = [tokens(70, 256, 41), tokens(9, 256, 42), tokens(30, 256, 43)]     # three requests, two slots
    outs = eng.generate(prompts, SamplingParams(temperature=0.0, max_tokens=12, ignore_eos=True))
    for p, o in zip(prompts, outs):
        assert o == oracle.greedy(cfgd, sd, p, 12)
    assert eng.state_slots.num_free() == 2 and eng.bm.num_free() == eng.bm.num_blocks
    if graphs:
        assert eng.runner.stats["graph_steps"] > 0


def test_preemption_recomputes_state():
    """A pool too small for both sequences: the younger one is preempted, gives its slot back and is
    recomputed from its first token."""
    cfgd = small_config("pD", vocab=256)
    eng, sd = build(cfgd, "cpu", torch.float32, blocks_=3, seqs=2)
    prompts = [tokens(60, 256, 51), tokens(62, 256, 52)]
    outs = eng.generate(prompts, SamplingParams(temperature=0.0, max_tokens=10, ignore_eos=True))
    assert eng.scheduler.num_preemptions > 0
    for p, o in zip(prompts, outs):
        assert o == oracle.greedy(cfgd, sd, p, 10)


def test_registry_and_config_errors():
    from financial_chatbot_llm_amd.models import get_model_config
    c = get_model_config("sigudra-tiny")
    assert c.arch == "sigudra" and len(c.layers) == c.num_layers and c.embedding["bigram"]["buckets"] == 251
    bad = copy.deepcopy(example_config())
    bad["layers"][0]["type"] = "mamba2"              # a mixer of another design
    with pytest.raises(ValueError):
        SigudraModel(layered_config(bad, "bad"), device="cpu")
    bad = copy.deepcopy(example_config())
    bad["layers"][0]["mlp"]["kind"] = "other"
    with pytest.raises(ValueError):
        SigudraModel(layered_config(bad, "bad"), device="cpu")
    sd = random_weights(SigudraModel(layered_config(example_config(), "ok"), device="cpu"), 0)
    open_ = copy.deepcopy(example_config())
    for l in open_["layers"]:                        # as a checkpoint's config.json: no ranks
        l["mixer"].pop("decay_rank", None)
        l["mixer"].pop("gate_rank", None)
    m = SigudraModel(layered_config(open_, "ok"), device="cpu")
    with pytest.raises(ValueError):
        m.init_random()
    sd["l0.mix.a1"] = sd["l0.mix.a1"][:7]            # a low-rank projection's rank is the tensor's ...
    sd["l0.mix.a2"] = sd["l0.mix.a2"][:, :7]
    m.load_state(sd)
    assert m.layers[0].mixer.ra == 7
    sd["l0.mix.q"] = sd["l0.mix.q"][:-1]             # ... every other size is the config's
    with pytest.raises(ValueError):
        m.load_state(sd)
    sd.pop("l0.norm1")
    with pytest.raises(KeyError):
        m.load_state(sd)
