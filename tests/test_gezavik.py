"""Gezavik (layered hybrid decoder) against the plain oracle of tests/gezavik_oracle.py.

Small configurations with random weights made here; the framework side always runs through the
engine (scheduler admission, pages, state slots, runner) or the ops' public entry points.  CPU
tensors exercise the ops' PyTorch forms, ``cuda`` ones the HIP kernels (marked gpu).
"""
import copy

import pytest
import torch

import gezavik_oracle as oracle
from financial_chatbot_llm_amd.config import EngineConfig
from financial_chatbot_llm_amd.engine import LLMEngine, SamplingParams
from financial_chatbot_llm_amd.models import mixers as blocks
from financial_chatbot_llm_amd.models.configs import layered_config
from financial_chatbot_llm_amd.models.gezavik import GezavikModel, example_config
from financial_chatbot_llm_amd.ops import mixers as mx

DEVICES = ["cpu", pytest.param("cuda", marks=pytest.mark.gpu)]
DTYPES = [torch.float32, torch.bfloat16]
TOL = {torch.float32: 3e-4, torch.bfloat16: 6e-2}


def random_weights(model, seed):
    g = torch.Generator().manual_seed(seed)
    sd = {}
    for name, shape in model.full_shapes().items():
        leaf = name.rsplit(".", 1)[-1]
        r = torch.randn(shape, generator=g)
        if leaf in ("norm1", "norm") and len(shape) == 1:
            t = 1.0 + 0.2 * r
        elif leaf == "A_log":
            t = torch.log(0.5 + 4 * torch.rand(shape, generator=g))
        elif leaf == "dt_bias":
            t = -3.0 + r
        elif leaf == "D":
            t = 1.0 + 0.3 * r
        elif leaf == "correction":
            t = 0.08 * r          # large enough to change which experts are chosen
        elif leaf == "b":
            t = 0.2 * r
        elif leaf == "conv":
            t = 0.6 * r
        elif leaf == "embed":
            t = r
        else:
            t = r * shape[-1] ** -0.5 * 1.3
        sd[name] = t.to(torch.bfloat16)
    return sd


def small_config(pattern="amAM", **over):
    c = example_config(width=over.pop("width", 96), vocab=over.pop("vocab", 160), heads=over.pop("heads", 3), pattern=pattern)
    for l in c["layers"]:
        for k, v in over.items():
            if k in l["mixer"]:
                l["mixer"][k] = v
    return c


def build(cfgd, device, dtype, seed=1, blocks_=24, seqs=4, graphs=False, async_=False, max_len=1024):
    mc = layered_config(cfgd, "gezavik-test")
    model = GezavikModel(mc, device=device, dtype=dtype)
    sd = random_weights(model, seed)
    model.load_state(sd)
    eng = LLMEngine(EngineConfig(model="gezavik-test", device=device, dtype="fp32" if dtype == torch.float32 else "bf16",
                                 num_kv_blocks=blocks_, max_num_seqs=seqs, max_model_len=max_len,
                                 max_num_batched_tokens=512, enable_prefix_caching=False, use_cuda_graph=graphs,
                                 async_scheduling=async_, graph_batch_sizes=(1, 2, 4)), model=model)
    return eng, sd


def poison(eng):
    """Pages and slots as a previous owner might have left them: nothing may depend on their content."""
    for lay in eng.kv.layers:
        for t in lay[1:]:
            t.fill_(float("nan"))


def close(got, want, dtype):
    got, want = got.double().cpu(), want.double().cpu()
    err = (got - want).abs().max().item() / max(want.abs().max().item(), 1e-9)
    assert err <= TOL[dtype], f"relative error {err:.3e} > {TOL[dtype]}"


def tokens(n, vocab, seed):
    return torch.randint(0, vocab, (n,), generator=torch.Generator().manual_seed(seed)).tolist()


def run_whole(eng, rid, toks):
    return eng.replay_step([(rid, toks, list(range(len(toks))))], [rid])


# ---------------------------------------------------------------------------------------------------
# each mechanism alone: one-layer models
# ---------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("pattern", ["m", "a", "A", "M"])
def test_one_layer_against_oracle(device, dtype, pattern):
    cfgd = small_config(pattern)
    eng, sd = build(cfgd, device, dtype)
    poison(eng)
    toks = tokens(90, cfgd["vocab"], 3)          # crosses a 64-token page and several windows
    close(run_whole(eng, "r", toks), oracle.forward(cfgd, sd, toks, torch.float64), dtype)


@pytest.mark.parametrize("device", DEVICES)
def test_no_feed_forward_no_mask_single_groups(device):
    """mlp: null, no mask entry (plain causal), groups = norm_groups = 1, no identity / shared expert, top 1."""
    cfgd = small_config("amA")
    cfgd["layers"][0]["mlp"] = None
    del cfgd["layers"][0]["mixer"]["mask"]
    cfgd["layers"][1]["mixer"].update(groups=1, norm_groups=1, conv=2, heads=4, vdim=12, state=17)
    cfgd["layers"][2]["mlp"]["router"].update(identity=0, top=1)
    cfgd["layers"][2]["mlp"]["shared"] = None
    eng, sd = build(cfgd, device, torch.float32)
    poison(eng)
    toks = tokens(70, cfgd["vocab"], 5)
    close(run_whole(eng, "r", toks), oracle.forward(cfgd, sd, toks, torch.float64), torch.float32)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
def test_other_sizes(device, dtype):
    """Sizes unlike the small default: odd head counts, state and value sizes that fill no wave, an odd
    latent width, a window longer than a page, five-tap convolution, many experts."""
    cfgd = small_config("aMmA", width=80, vocab=97, heads=5)
    for l in cfgd["layers"]:
        if l["type"] == "latent_attention":
            l["mixer"].update(dim=12, rot_dim=6, vdim=28, kv_rank=35, q_rank=44, mask={"size": 70}, scale=0.31,
                              rot={"base": 500.0, "dims": 6})
        else:
            l["mixer"].update(heads=3, vdim=33, state=50, groups=3, norm_groups=3, conv=5)
        if l["mlp"]["kind"] == "moe":
            l["mlp"]["router"].update(experts=70, identity=3, top=5)
            l["mlp"]["expert"].update(ff=20, limit=0.7)
    eng, sd = build(cfgd, device, dtype, blocks_=8)
    poison(eng)
    toks = tokens(150, cfgd["vocab"], 7)
    close(run_whole(eng, "r", toks), oracle.forward(cfgd, sd, toks, torch.float64), dtype)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("pattern", ["aA", "mM"])
def test_single_mixer_kind_models(device, pattern):
    """Only attention layers (no state slots at all) and only Mamba-2 layers (no latent cache)."""
    cfgd = small_config(pattern)
    eng, sd = build(cfgd, device, torch.float32)
    poison(eng)
    assert (eng.state_slots is None) == (pattern == "aA")
    toks = tokens(100, cfgd["vocab"], 17)
    want = oracle.forward(cfgd, sd, toks, torch.float64)
    got = [eng.replay_step([("r", toks[:70], list(range(70)))])]
    got += [eng.replay_step([("r", toks[i:i + 1], [0])]) for i in range(70, 100)]
    close(torch.cat(got), want, torch.float32)


# ---------------------------------------------------------------------------------------------------
# cache, state, batching
# ---------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
def test_prefill_then_token_by_token(device, dtype):
    cfgd = small_config("amAM")
    eng, sd = build(cfgd, device, dtype)
    poison(eng)
    toks = tokens(130, cfgd["vocab"], 11)
    want = oracle.forward(cfgd, sd, toks, torch.float64)
    got = [eng.replay_step([("r", toks[:40], list(range(40)))])]
    for i in range(40, len(toks)):               # long decoding: over the window and a page border
        got.append(eng.replay_step([("r", toks[i:i + 1], [0])], ["r"] if i == len(toks) - 1 else []))
    close(torch.cat(got), want, dtype)
    assert eng.bm.num_free() == eng.bm.num_blocks and eng.state_slots.num_free() == 4


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("sizes", [[2, 2, 3, 60, 2, 1, 1, 64, 5], [63, 1, 1, 2, 70], [1, 1, 1, 130]])
def test_portions(device, sizes):
    cfgd = small_config("mAaM")
    eng, sd = build(cfgd, device, torch.float32)
    poison(eng)
    toks = tokens(sum(sizes), cfgd["vocab"], 13)
    want = oracle.forward(cfgd, sd, toks, torch.float64)
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
    cfgd = small_config("aMmA")
    eng, sd = build(cfgd, device, dtype, blocks_=7, seqs=3)
    poison(eng)
    V = cfgd["vocab"]
    reqs = {f"q{i}": tokens(n, V, 20 + i) for i, n in enumerate([150, 70, 33, 100, 5, 64])}
    want = {k: oracle.forward(cfgd, sd, t, torch.float64) for k, t in reqs.items()}
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
    for k in reqs:
        assert at[k] == len(reqs[k])
        close(torch.cat(got[k]), want[k], dtype)


# ---------------------------------------------------------------------------------------------------
# window and page edges with scores that stand out
# ---------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("window", [5, 64, 70])
def test_window_edges_stand_out(device, dtype, window):
    """One key per query gets an overwhelming score: first the oldest key inside the window (the
    output must be that key's latent), then the newest key outside it (the output must not show it).
    Queries sit before, on and after page borders, as rows of a prompt chunk and as single decoded rows."""
    H, R, Dr, pages, n = 2, 16, 4, 4, 200
    g = torch.Generator().manual_seed(window)
    lat = torch.randn(n, R + Dr, generator=g)
    lat[:, R:] = 0
    table = torch.tensor([[2, 0, 3, 1]], dtype=torch.int32)
    row = lambda j: int(table[0, j // 64]) * 64 + j % 64  # noqa: E731
    cache = torch.zeros(pages * 64, R + Dr)
    for j in range(n):
        cache[row(j)] = lat[j]
    chunks = [list(range(p0, p0 + 8)) for p0 in (window, 60, 124, 188) if p0 >= window]
    chunks += [[p] for p in (window, 63, 64, 65, 127, 128, 199) if p >= window]
    for shift, inside in ((window - 1, True), (window, False)):
        for seg in chunks:
            m = len(seg)
            kc = cache.clone()
            q = torch.zeros(m, H, R)
            for i, p in enumerate(seg):          # query i asks for coordinate i; only its target key is large there
                kc[row(p - shift), i] = 50.0
                q[i, :, i] = 4.0
            out = mx.latent_attend(q.to(dtype).to(device), torch.zeros(m, H, Dr, dtype=dtype, device=device),
                                   kc.to(dtype).to(device), torch.tensor([0, m], dtype=torch.int32, device=device),
                                   torch.tensor(seg, dtype=torch.int32, device=device), table.to(device), window, 1.0,
                                   m).float().cpu()
            for i, p in enumerate(seg):
                keys = kc[[row(j) for j in range(max(0, p - window + 1), p + 1)]]
                ref = (torch.softmax(keys[:, i] * 4.0, 0)[:, None] * keys[:, :R]).sum(0)
                tol = 1e-4 if dtype == torch.float32 else 0.3
                assert (out[i] - ref[None]).abs().max() < tol, (shift, seg, i)
                assert bool(out[i, 0, i] > 40.0) == inside


@pytest.mark.parametrize("device", DEVICES)
def test_far_key_in_a_long_prompt_chunk(device):
    """A chunk of queries deep in a sequence, no window: one far key among hundreds carries the score."""
    H, R, Dr = 3, 24, 8
    n = 400
    g = torch.Generator().manual_seed(2)
    pages = 8
    perm = torch.randperm(pages, generator=g).to(torch.int32)[None]
    lat = 0.1 * torch.randn(n, R + Dr, generator=g)
    far = 7
    lat[far, 1] = 30.0
    cache = torch.zeros(pages * 64, R + Dr)
    for j in range(n):
        cache[int(perm[0, j // 64]) * 64 + j % 64] = lat[j]
    pos = torch.arange(330, 400, dtype=torch.int32)
    q = torch.zeros(len(pos), H, R)
    q[:, :, 1] = 3.0
    cu = torch.tensor([0, len(pos)], dtype=torch.int32)
    for window, hit in ((1 << 30, True), (300, False)):
        out = mx.latent_attend(q.to(device), torch.zeros(len(pos), H, Dr, device=device), cache.to(device), cu.to(device),
                               pos.to(device), perm.to(device), window, 1.0, len(pos)).cpu()
        assert bool((out[:, :, 1] > 25.0).all()) == hit
        # the same far key seen from single decoded rows (bf16: the split-key form on the GPU)
        for dt in DTYPES:
            one = mx.latent_attend(q[:1].to(dt).to(device), torch.zeros(1, H, Dr, dtype=dt, device=device),
                                   cache.to(dt).to(device), torch.tensor([0, 1], dtype=torch.int32, device=device),
                                   torch.tensor([399], dtype=torch.int32, device=device), perm.to(device), window, 1.0,
                                   1).float().cpu()
            assert bool((one[:, :, 1] > 25.0).all()) == hit


@pytest.mark.gpu
@pytest.mark.parametrize("window", [1 << 30, 150])
def test_decode_rows_split_over_keys(window):
    """Single decoded rows of bf16 models walk their keys with several blocks whose parts are merged:
    rows at unequal depths, pages in scrambled order, against the one-pass CPU form."""
    H, R, Dr, pages = 5, 48, 16, 12
    g = torch.Generator().manual_seed(9)
    cache = torch.randn(pages * 64, R + Dr, generator=g).bfloat16()
    depths = [700, 33, 64, 301, 1]
    bt = torch.stack([torch.randperm(pages, generator=g) for _ in depths]).to(torch.int32)
    pos = torch.tensor([d - 1 for d in depths], dtype=torch.int32)
    cu = torch.arange(len(depths) + 1, dtype=torch.int32)
    q = (0.3 * torch.randn(len(depths), H, R, generator=g)).bfloat16()
    qr = (0.3 * torch.randn(len(depths), H, Dr, generator=g)).bfloat16()
    gate = torch.randn(len(depths), H, generator=g).bfloat16()
    want = mx.latent_attend(q, qr, cache, cu, pos, bt, window, 0.2, 1, gate=gate).float()
    got = mx.latent_attend(q.cuda(), qr.cuda(), cache.cuda(), cu.cuda(), pos.cuda(), bt.cuda(), window, 0.2, 1,
                           gate=gate.cuda()).float().cpu()
    assert (got - want).abs().max() < 2e-2


# ---------------------------------------------------------------------------------------------------
# routing
# ---------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("device", DEVICES)
def test_router_bias_changes_choice_not_weight(device):
    z = torch.tensor([[2.0, 1.0, 0.5, 0.0, -1.0]] * 3)
    bias = torch.tensor([0.0, 0.0, 0.0, 0.9, 0.0])
    w, i = mx.route_biased(z.to(device), bias.to(device), 2)
    s = torch.softmax(z[0], 0)
    assert sorted(i[0].tolist()) == [0, 3]                    # entry 3 wins on its bias ...
    got = dict(zip(i[0].tolist(), w[0].tolist()))
    assert abs(got[3] - s[3].item()) < 1e-6 and abs(got[0] - s[0].item()) < 1e-6   # ... and weighs its plain score
    assert abs(sum(got.values()) - 1.0) > 0.1                 # not renormalised


@pytest.mark.parametrize("device", DEVICES)
def test_routed_ff_bucketed_and_dense_forms_agree(device, monkeypatch):
    cfgd = small_config("A")
    eng, sd = build(cfgd, device, torch.float32)
    toks = tokens(80, cfgd["vocab"], 31)
    want = oracle.forward(cfgd, sd, toks, torch.float64)
    monkeypatch.setattr(blocks, "DENSE_MAX_PAIRS", 0)          # every step buckets rows by expert
    close(run_whole(eng, "a", toks), want, torch.float32)
    monkeypatch.setattr(blocks, "DENSE_MAX_PAIRS", 1 << 30)    # every step runs all experts densely
    close(run_whole(eng, "b", toks), want, torch.float32)


# ---------------------------------------------------------------------------------------------------
# generation through the engine's own scheduler
# ---------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("device,graphs", [("cpu", False), pytest.param("cuda", False, marks=pytest.mark.gpu),
                                           pytest.param("cuda", True, marks=pytest.mark.gpu)])
@pytest.mark.parametrize("async_", [False, True])
def test_greedy_generation(device, graphs, async_):
    cfgd = small_config("amAM", vocab=256)
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
    cfgd = small_config("mA", vocab=256)
    eng, sd = build(cfgd, "cpu", torch.float32, blocks_=3, seqs=2)
    prompts = [tokens(60, 256, 51), tokens(62, 256, 52)]
    outs = eng.generate(prompts, SamplingParams(temperature=0.0, max_tokens=10, ignore_eos=True))
    assert eng.scheduler.num_preemptions > 0
    for p, o in zip(prompts, outs):
        assert o == oracle.greedy(cfgd, sd, p, 10)


def test_registry_and_config_errors():
    from financial_chatbot_llm_amd.models import get_model_config
    c = get_model_config("gezavik-tiny")
    assert c.arch == "gezavik" and len(c.layers) == c.num_layers
    bad = copy.deepcopy(example_config())
    bad["layers"][0]["type"] = "something_else"
    with pytest.raises(ValueError):
        GezavikModel(layered_config(bad, "bad"), device="cpu")
    bad = copy.deepcopy(example_config())
    bad["layers"][0]["mlp"]["kind"] = "other"
    with pytest.raises(ValueError):
        GezavikModel(layered_config(bad, "bad"), device="cpu")
    m = GezavikModel(layered_config(example_config(), "ok"), device="cpu")
    sd = random_weights(m, 0)
    sd.pop("l0.norm1")
    with pytest.raises(KeyError):
        m.load_state(sd)
