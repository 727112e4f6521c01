"""Tukedra (pre-norm layered decoder with several residual streams) against the plain oracle of
tests/tukedra_oracle.py.

Small configurations with random weights made here; the framework side always runs through the
engine (scheduler admission, pages, state slots, runner) or the ops' public entry points.  CPU
tensors exercise the ops' PyTorch forms, ``cuda`` ones the HIP kernels (marked gpu).
"""
import copy
import math

import pytest
import torch

import tukedra_oracle as oracle
from financial_chatbot_llm_amd.config import EngineConfig
from financial_chatbot_llm_amd.engine import LLMEngine, SamplingParams
from financial_chatbot_llm_amd.models import mixers as blocks
from financial_chatbot_llm_amd.models.configs import layered_config
from financial_chatbot_llm_amd.models.tukedra import TukedraModel, example_config
from financial_chatbot_llm_amd.ops import mixers as mx

DEVICES = ["cpu", pytest.param("cuda", marks=pytest.mark.gpu)]
DTYPES = [torch.float32, torch.bfloat16]
TOL = {torch.float32: 3e-4, torch.bfloat16: 8e-2}


def random_weights(model, seed):
    g = torch.Generator().manual_seed(seed)
    sd = {}
    for name, shape in model.full_shapes().items():
        leaf = name.rsplit(".", 1)[-1]
        r = torch.randn(shape, generator=g)
        if ".hc" in name and leaf == "mix":
            t = torch.eye(shape[0]) * 0.9 + 0.3 * r
        elif ".hc" in name and leaf == "in":
            t = (1.0 + 0.5 * r) / shape[0]
        elif leaf in ("norm1", "norm2", "norm", "out") and len(shape) == 1:
            t = 1.0 + 0.2 * r
        elif leaf == "b" and len(shape) == 1:
            t = 0.3 * r
        elif leaf == "embed":
            t = r
        else:
            t = r * shape[-1] ** -0.5 * 1.3
        sd[name] = t.to(torch.bfloat16)
    return sd


def small_config(pattern="lRaL", **over):
    c = example_config(width=over.pop("width", 96), vocab=over.pop("vocab", 160), pattern=pattern,
                       streams=over.pop("streams", 3))
    for l in c["layers"]:
        for k, v in over.items():
            if k in l["mixer"]:
                l["mixer"][k] = v
    return c


def build(cfgd, device, dtype, seed=1, blocks_=24, seqs=4, graphs=False, async_=False, max_len=1024):
    mc = layered_config(cfgd, "tukedra-test")
    model = TukedraModel(mc, device=device, dtype=dtype)
    sd = random_weights(model, seed)
    model.load_state(sd)
    eng = LLMEngine(EngineConfig(model="tukedra-test", device=device, dtype="fp32" if dtype == torch.float32 else "bf16",
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


def close(got, want, dtype, flips=None):
    """``flips``: the share of positions that may be off (bf16 runs with many experts: a rounding of the
    router's input can swap two experts whose logits nearly tie)."""
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


def i32(x, device="cpu"):
    return torch.tensor(x, dtype=torch.int32, device=device)


# ---------------------------------------------------------------------------------------------------
# each mechanism alone: one-layer models
# ---------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("pattern", ["l", "r", "a", "L"])
def test_one_layer_against_oracle(device, dtype, pattern):
    cfgd = small_config(pattern)
    eng, sd = build(cfgd, device, dtype)
    poison(eng)
    toks = tokens(90, cfgd["vocab"], 3)          # crosses a 64-token page and two 37-token blocks of the mask
    close(run_whole(eng, "r", toks), oracle.forward(cfgd, sd, toks), dtype)


@pytest.mark.parametrize("device", DEVICES)
def test_stream_sum_after_every_layer(device):
    cfgd = small_config("lARr")
    eng, sd = build(cfgd, device, torch.float32)
    toks = tokens(40, cfgd["vocab"], 4)
    want = []
    oracle.forward(cfgd, sd, toks, want)
    eng.model.capture = []
    run_whole(eng, "r", toks)
    assert len(eng.model.capture) == len(want) == 4
    for got, ref in zip(eng.model.capture, want):
        close(got, ref, torch.float32)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("streams", [0, 1, 2, 5, 16])
def test_stream_counts(device, streams):
    """No ``streams`` entry is the plain residual sum (no hc tensors at all); one stream still has its
    read, write and mix weights."""
    cfgd = small_config("lAr", streams=streams)
    assert ("streams" in cfgd) == bool(streams)
    eng, sd = build(cfgd, device, torch.float32)
    assert any(".hc1." in k for k in sd) == bool(streams)
    toks = tokens(50, cfgd["vocab"], 5)
    close(run_whole(eng, "r", toks), oracle.forward(cfgd, sd, toks), torch.float32)


@pytest.mark.parametrize("device", DEVICES)
def test_absent_entries_and_single_sizes(device):
    """mlp: null, no mask (plain causal), no rotation, no frequency scaling, no shared expert, top 1, one
    head, no embedding scale, no logit scale or cap, decays 0 and 1."""
    cfgd = small_config("alRrA")
    for k in ("embedding", "logit_scale", "logit_softcap"):
        del cfgd[k]
    L = cfgd["layers"]
    L[0]["mlp"] = None
    del L[0]["mixer"]["mask"]
    del L[0]["mixer"]["rot"]["scaling"]
    L[0]["mixer"].update(heads=1, kv_heads=1)
    L[1]["mlp"] = None
    L[1]["mixer"].update(heads=1, decay=[1.0])
    del L[2]["mlp"]["shared"]
    L[2]["mlp"]["router"].update(top=1)
    L[2]["mixer"].update(heads=2, decay=[0.0, 1.0])
    del L[3]["mixer"]["rot"]
    del L[4]["mixer"]["rot"]
    L[4]["mixer"].update(kv_heads=6)
    eng, sd = build(cfgd, device, torch.float32)
    assert "l0.norm2" not in sd and "l0.hc2.in" not in sd and "l2.mlp.shared.up" not in sd
    poison(eng)
    toks = tokens(70, cfgd["vocab"], 5)
    close(run_whole(eng, "r", toks), oracle.forward(cfgd, sd, toks), torch.float32)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
def test_other_sizes(device, dtype):
    """Sizes unlike the small default: odd head counts, key and value sizes that fill no wave and differ, a
    key size above 128, a mask block longer than a page, rotation over the whole head and over a small
    part, many experts, other constants.  (bf16 runs route in one layer only: among 70 experts the fifth
    and sixth logits are often closer than the rounding of the router's input.)"""
    cfgd = small_config("ArLlaR" if dtype == torch.float32 else "arLlar", width=80, vocab=97, streams=4)
    cfgd["embedding"]["scale"] = 0.7
    cfgd["norm"]["eps"] = 0.02               # large enough to show in every norm
    cfgd["logit_scale"], cfgd["logit_softcap"] = 1.7, 6.0
    L = cfgd["layers"]
    L[0]["mixer"].update(dim=40, vdim=40, heads=6, kv_heads=1, mask={"size": 70}, scale=0.31,
                         rot={"base": 777.0, "dims": 40, "scaling": {"factor": 16.0, "fast": 8.0, "original": 64, "slow": 0.5}})
    L[1]["mixer"].update(heads=5, dim=12, vdim=9, decay=[0.5, 0.9, 0.97, 0.99, 0.999], rot={"base": 100.0, "dims": 4})
    L[2]["mixer"].update(heads=2, dim=132, vdim=17, decay=[0.93, 0.999])
    L[3]["mixer"].update(heads=1, dim=9, vdim=70, decay=[0.98])
    L[4]["mixer"].update(dim=18, vdim=18, heads=4, kv_heads=4, mask={"size": 3}, rot={"base": 50.0, "dims": 2})
    L[5]["mixer"].update(heads=3, dim=34, vdim=33, decay=[0.8, 0.9, 1.0], rot={"base": 1e6, "dims": 34})
    for l in L:
        if l["mlp"]["kind"] == "moe":
            l["mlp"]["router"].update(experts=70, top=5)
            l["mlp"]["expert"].update(ff=20)
            l["mlp"]["shared"].update(ff=9)
    eng, sd = build(cfgd, device, dtype, blocks_=8)
    poison(eng)
    toks = tokens(150, cfgd["vocab"], 7)
    close(run_whole(eng, "r", toks), oracle.forward(cfgd, sd, toks), dtype, flips=0.0 if dtype == torch.float32 else 0.1)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
def test_wide_attention_heads(device, dtype):
    """A head size beyond what the matrix-core attention covers (bf16 then takes the f32-lane kernel)."""
    cfgd = small_config("a", width=64)
    cfgd["layers"][0]["mixer"].update(dim=264, vdim=264, heads=2, kv_heads=1, scale=0.9)
    eng, sd = build(cfgd, device, dtype, blocks_=4)
    toks = tokens(80, cfgd["vocab"], 8)
    close(run_whole(eng, "r", toks), oracle.forward(cfgd, sd, toks), dtype)


@pytest.mark.parametrize("device", DEVICES)
def test_first_tokens(device):
    """Sequences of one and two tokens, and the first tokens of a longer one, each request alone."""
    cfgd = small_config("lRaL")
    eng, sd = build(cfgd, device, torch.float32)
    poison(eng)
    for n in (1, 2, 5):
        toks = tokens(n, cfgd["vocab"], 60 + n)
        close(run_whole(eng, f"r{n}", toks), oracle.forward(cfgd, sd, toks), torch.float32)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("pattern", ["aA", "lR"])
def test_single_mixer_kind_models(device, pattern):
    """Only attention layers (no state slots at all) and only recurrent layers (no paged rows)."""
    cfgd = small_config(pattern)
    eng, sd = build(cfgd, device, torch.float32)
    poison(eng)
    assert (eng.state_slots is None) == (pattern == "aA")
    toks = tokens(100, cfgd["vocab"], 17)
    want = oracle.forward(cfgd, sd, toks)
    got = [eng.replay_step([("r", toks[:70], list(range(70)))])]
    got += [eng.replay_step([("r", toks[i:i + 1], [0])]) for i in range(70, 100)]
    close(torch.cat(got), want, torch.float32)


# ---------------------------------------------------------------------------------------------------
# cache, state, batching
# ---------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
def test_prefill_then_token_by_token(device, dtype):
    cfgd = small_config("lRaL")
    eng, sd = build(cfgd, device, dtype)
    poison(eng)
    toks = tokens(130, cfgd["vocab"], 11)
    want = oracle.forward(cfgd, sd, toks)
    got = [eng.replay_step([("r", toks[:40], list(range(40)))])]
    for i in range(40, len(toks)):               # long decoding: over block edges of the mask and a page border
        got.append(eng.replay_step([("r", toks[i:i + 1], [0])], ["r"] if i == len(toks) - 1 else []))
    close(torch.cat(got), want, dtype)
    assert eng.bm.num_free() == eng.bm.num_blocks and eng.state_slots.num_free() == 4


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("sizes", [[2, 2, 3, 60, 2, 1, 1, 64, 5], [63, 1, 1, 2, 70], [1, 1, 1, 130], [2] * 20, [36, 2, 36, 1, 37]])
def test_portions(device, sizes):
    """Portions cut inside pages and inside blocks of the mask, down to two tokens."""
    cfgd = small_config("rAlL")
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
    cfgd = small_config("aLrA")
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


@pytest.mark.parametrize("device", DEVICES)
def test_batch_rows_do_not_depend_on_their_neighbours(device):
    """The same request alone and between two others gives the same logits bit for bit (f32)."""
    cfgd = small_config("lRa")
    eng, sd = build(cfgd, device, torch.float32)
    V = cfgd["vocab"]
    a, b, c = tokens(45, V, 1), tokens(20, V, 2), tokens(70, V, 3)
    alone = run_whole(eng, "x", b)
    poison(eng)
    out = eng.replay_step([("a", a, []), ("b", b, list(range(len(b)))), ("c", c, [])], ["a", "b", "c"])
    assert (out - alone).abs().max() <= 2e-6 * alone.abs().max()


# ---------------------------------------------------------------------------------------------------
# block edges of the mask, page borders, far keys: scores and states that stand out
# ---------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("size", [5, 64, 70])
def test_mask_block_edges_stand_out(device, dtype, size):
    """One key per query gets an overwhelming score: first the FIRST key of the query's block of ``size``
    positions (the output must be that key's value), then the LAST key of the block before (the output
    must not show it).  Queries sit at the start, inside and at the end of blocks and around page
    borders, as rows of a prompt chunk and as single decoded rows; three query heads share each of two
    key/value heads."""
    H, G, D, P, pages, n = 6, 2, 16, 12, 4, 200
    g = torch.Generator().manual_seed(size)
    table = i32([[2, 0, 3, 1]])
    row = lambda j: int(table[0, j // 64]) * 64 + j % 64  # noqa: E731
    cache = torch.zeros(pages * 64, G * (D + P))
    for j in range(n):
        cache[row(j), G * D:] = torch.randn(G * P, generator=g)           # values; keys stay zero
    chunks = [list(range(p0, p0 + 8)) for p0 in (size, 60, 124, 188, 2 * size - 3)]
    chunks += [[p] for p in (size, size + 1, 2 * size - 1, 2 * size, 63, 64, 65, 127, 128, 199)]
    for inside in (True, False):
        for seg in chunks:
            m = len(seg)
            kc = cache.clone()
            q = torch.zeros(m, H, D)
            target = []
            for i, p in enumerate(seg):          # query i asks for key coordinate i; only its target key is large there
                first = (p // size) * size
                t = first if inside else first - 1
                target.append(t)
                for kvh in range(G):
                    kc[row(t), kvh * D + i] = 50.0
                q[i, :, i] = 4.0
            out = mx.window_attend(q.reshape(m, H * D).to(dtype).to(device), kc.to(dtype).to(device), i32([0, m], device),
                                   i32(seg, device), table.to(device), size, 1.0, m, H, G, D, P,
                                   chunked=True).float().cpu().view(m, H, P)
            kcr = kc.to(dtype).float()
            for i, p in enumerate(seg):
                rows_ = [row(j) for j in range((p // size) * size, p + 1)]
                for h in range(H):
                    kvh = h // (H // G)
                    pr = torch.softmax(kcr[rows_, kvh * D + i] * 4.0, 0)
                    ref = (pr[:, None] * kcr[rows_, G * D + kvh * P:G * D + (kvh + 1) * P]).sum(0)
                    tol = 1e-4 if dtype == torch.float32 else 0.05
                    assert (out[i, h] - ref).abs().max() < tol, (inside, seg, i, h)
                    tv = kcr[row(target[i]), G * D + kvh * P:G * D + (kvh + 1) * P]
                    assert bool((out[i, h] - tv).abs().max() < 0.05) == inside


@pytest.mark.parametrize("device", DEVICES)
def test_far_key_in_a_long_block_and_decoded_rows(device):
    """One far key among hundreds carries the score, seen from a chunk deep in the sequence and from
    single rows: with no mask, and with a block that still holds it; a block that starts after it hides it."""
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
    cu = i32([0, len(pos)])
    for size, chunked, hit in ((1 << 30, False, True), (512, True, True), (320, True, False), (8, True, False)):
        out = mx.window_attend(q.view(len(pos), -1).to(device), cache.to(device), cu.to(device), pos.to(device),
                               perm.to(device), size, 1.0, len(pos), H, G, D, P, chunked=chunked).cpu()
        assert bool((out > 8.0).all()) == hit
        for dt in DTYPES:
            one = mx.window_attend(q[:1].view(1, -1).to(dt).to(device), cache.to(dt).to(device), i32([0, 1], device),
                                   i32([399], device), perm.to(device), size, 1.0, 1, H, G, D, P,
                                   chunked=chunked).float().cpu()
            assert bool((one > 8.0).all()) == hit


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("act", ["none", "silu"])
def test_fixed_decay_state_keeps_a_far_write(device, act):
    """A value written hundreds of tokens back under a decay close to one is read out by a matching query at
    the end, through portions that hand the state over in a reused slot; under a fast decay it is gone.
    Head 0 keeps, head 1 forgets: the decays are per head."""
    H, D, P, n = 2, 20, 12, 300
    g = torch.Generator().manual_seed(6)
    far = 3
    k = 0.01 * torch.randn(n, H * D, generator=g)
    v = 0.01 * torch.randn(n, H * P, generator=g)
    q = torch.zeros(n, H * D)
    k[far] = 0
    k[far, 5] = k[far, D + 5] = 3.0
    v[far] = 7.0
    q[-1, 5] = q[-1, D + 5] = 3.0
    decay = torch.tensor([0.9995, 0.5])
    state = torch.full((3, H, D, P), float("nan")).to(device)
    outs, at = [], 0
    for m in (100, 1, 1, 2, 196):
        sl = slice(at, at + m)
        outs.append(mx.decay_scan(q[sl].to(device), k[sl].to(device), v[sl].to(device), decay.to(device), state,
                                  i32([0, m], device), i32([1], device), torch.arange(at, at + m, dtype=torch.int32, device=device),
                                  H, D, P, act=act, out_scale=0.5, max_len=m).cpu())
        at += m
    last = torch.cat(outs)[-1].view(H, P)
    f = (lambda z: z * torch.sigmoid(z)) if act == "silu" else (lambda z: z)
    keep = 0.5 * float(f(torch.tensor(3.0)) ** 2 * f(torch.tensor(7.0))) * 0.9995 ** (n - 1 - far)
    assert (last[0] - keep).abs().max() < 0.05 * keep
    assert last[1].abs().max() < 1e-3 * keep


@pytest.mark.gpu
@pytest.mark.parametrize("lens", [[15, 16, 17, 33], [255, 257], [600, 1, 300]])
def test_segments_across_the_scan_kernels_chunks(lens):
    """Segments whose lengths sit on and around the scan kernel's internal chunk of 16 tokens, several per
    step, f32 q / k beside bf16 v and all-bf16 with the activation, against the op's plain form on the CPU."""
    g = torch.Generator().manual_seed(sum(lens))
    T, S = sum(lens), len(lens)
    cu = i32([0] + torch.tensor(lens).cumsum(0).tolist())
    pos = torch.cat([torch.arange(7 * i, 7 * i + n) for i, n in enumerate(lens)]).to(torch.int32)   # the first starts at 0
    slot = torch.arange(S, dtype=torch.int32).flip(0)
    for (H, D, P) in ((3, 40, 24), (2, 132, 70), (1, 300, 16)):
        decay = torch.rand(H, generator=g) * 0.2 + 0.8
        for qdt, vdt, act in ((torch.float32, torch.bfloat16, "none"), (torch.bfloat16, torch.bfloat16, "silu"),
                              (torch.float32, torch.float32, "silu")):
            q = torch.randn(T, H * D, generator=g).to(qdt)
            k = (torch.randn(T, H * D, generator=g) * 0.2).to(qdt)
            v = torch.randn(T, H * P, generator=g).to(vdt)
            st = torch.randn(S, H, D, P, generator=g) * 0.1
            s1, s2 = st.clone(), st.clone().cuda()
            want = mx.decay_scan(q, k, v, decay, s1, cu, slot, pos, H, D, P, act=act, out_scale=0.3)
            got = mx.decay_scan(q.cuda(), k.cuda(), v.cuda(), decay.cuda(), s2, cu.cuda(), slot.cuda(), pos.cuda(), H, D, P,
                                act=act, out_scale=0.3, max_len=max(lens))
            assert (got.cpu() - want).abs().max() <= 2e-4 * want.abs().max()
            assert (s2.cpu() - s1).abs().max() <= 2e-4 * s1.abs().max()


# ---------------------------------------------------------------------------------------------------
# rotation, streams, routing, logits
# ---------------------------------------------------------------------------------------------------
def test_scaled_frequencies_against_the_oracle_table():
    for rot in ({"dims": 16, "base": 3000.0, "scaling": {"factor": 4.0, "fast": 16.0, "original": 256, "slow": 2.0}},
                {"dims": 64, "base": 1e4, "scaling": {"factor": 32.0, "fast": 32.0, "original": 4096, "slow": 1.0}},
                {"dims": 6, "base": 10.0}):
        f, m = mx.rope_freqs(rot["dims"], rot["base"], rot.get("scaling"))
        fo, mo = oracle.rot_table(rot)
        assert torch.allclose(f.double(), fo, rtol=1e-6) and abs(m - mo) < 1e-12
    sc = {"factor": 4.0, "fast": 16.0, "original": 256, "slow": 2.0}
    f, m = mx.rope_freqs(16, 3000.0, sc)
    plain, _ = mx.rope_freqs(16, 3000.0)
    assert f[0] == plain[0] and abs(float(f[-1] / plain[-1]) - 0.25) < 1e-6 and m == 0.1 * math.log(4.0) + 1.0


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("layout", ["pairs", "half"])
def test_rotation_layouts_norm_and_cache_rows(device, layout):
    """Both pair layouts at large positions, the part of the head that is not rotated, the norm after the
    rotation, the scales, and the cache row [finished k | raw k] at the token's slot."""
    T, H, G, D, rot = 5, 3, 2, 10, 6
    g = torch.Generator().manual_seed(9)
    q, k = torch.randn(T, H * D, generator=g), torch.randn(T, G * D, generator=g)
    pos = i32([0, 1, 77, 4096, 100000])
    f = torch.tensor([1.0, 0.1, 0.003])
    ang = pos.double()[:, None] * f.double()[None]

    def ref(x, nh):
        x = x.double().view(T, nh, D).clone()
        idx = [(2 * i, 2 * i + 1) for i in range(rot // 2)] if layout == "pairs" else [(i, i + rot // 2) for i in range(rot // 2)]
        out = x.clone()
        for i, (a, b) in enumerate(idx):
            c, s = 1.3 * torch.cos(ang[:, i])[:, None], 1.3 * torch.sin(ang[:, i])[:, None]
            out[..., a] = x[..., a] * c - x[..., b] * s
            out[..., b] = x[..., b] * c + x[..., a] * s
        return out

    qo, ko = mx.rope_heads(q.to(device), k.to(device), H, G, D, f.to(device), pos.to(device), layout, 1.3, q_scale=2.0,
                           k_scale=0.5)
    assert torch.allclose(qo.cpu().double().view(T, H, D), 2.0 * ref(q, H), atol=2e-3)        # f32 angles at position 1e5
    assert torch.allclose(ko.cpu().double().view(T, G, D), 0.5 * ref(k, G), atol=2e-3)
    assert torch.equal(qo.cpu().view(T, H, D)[:, :, rot:], 2.0 * q.view(T, H, D)[:, :, rot:])       # not rotated: passes unchanged
    cache = torch.full((128, G * D + G * D + 3), -5.0).to(device)
    slots = i32([70, -1, 3, 127, 0], device)
    qn, none = mx.rope_heads(q.to(device), k.to(device), H, G, D, f.to(device), pos.to(device), layout, 1.3, norm_eps=1e-5,
                             k_out=cache, slots=slots, v=k.to(device))
    assert none is None
    rq, rk = ref(q, H), ref(k, G)
    rq = rq / torch.sqrt((rq * rq).mean(-1, keepdim=True) + 1e-5)
    rk = rk / torch.sqrt((rk * rk).mean(-1, keepdim=True) + 1e-5)
    assert torch.allclose(qn.cpu().double().view(T, H, D), rq, atol=2e-3)
    c = cache.cpu()
    for t, s in enumerate(slots.tolist()):
        if s >= 0:
            assert torch.allclose(c[s, :G * D].double(), rk[t].reshape(-1), atol=2e-3)
            assert torch.equal(c[s, G * D:2 * G * D], k[t])
            assert (c[s, 2 * G * D:] == -5.0).all()
    assert (c[1] == -5.0).all() and (c[71] == -5.0).all()          # the row without a slot wrote nothing


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("S", [1, 2, 3, 8, 13])
def test_stream_update_read_and_norm(device, S):
    """x_t <- sum_s mix[s, t] x_s + out[t] y with mix indexed [from, to] (an asymmetric mix shows a
    transposed read), all streams from the OLD ones, then the read with the next weights and its norm."""
    T, W = 7, 50
    g = torch.Generator().manual_seed(S)
    x = torch.randn(T, S, W, generator=g)
    y = torch.randn(T, W, generator=g)
    mix, wo, wi, w = torch.randn(S, S, generator=g), torch.randn(S, generator=g), torch.randn(S, generator=g), torch.randn(W, generator=g)
    new = torch.stack([sum(mix[s, t] * x[:, s] for s in range(S)) + wo[t] * y for t in range(S)], 1)
    u = sum(wi[t] * new[:, t] for t in range(S))
    want = u / torch.sqrt((u * u).mean(-1, keepdim=True) + 1e-5) * w
    xd = x.clone().to(device)
    h = mx.hyper_mix(xd, y.to(device), mix.to(device), wo.to(device), wi.to(device), w.to(device), 1e-5, torch.float32)
    assert torch.allclose(xd.cpu(), new, atol=1e-5) and torch.allclose(h.cpu(), want, atol=1e-4)
    first = mx.hyper_mix(xd, None, None, None, wi.to(device), w.to(device), 1e-5, torch.float32)    # read only
    assert torch.allclose(xd.cpu(), new, atol=1e-5) and torch.allclose(first.cpu(), want, atol=1e-4)
    e = mx.embed_scaled(i32([3, 0], device), torch.arange(40.0).view(4, 10).to(device), 0.5, S)
    assert e.shape == (2, S, 10) and torch.equal(e[0, S - 1].cpu(), torch.arange(30.0, 40.0) * 0.5)


@pytest.mark.parametrize("device", DEVICES)
def test_softmax_over_the_chosen_logits(device):
    z = torch.tensor([[2.0, 1.0, 0.5, 0.0, -1.0], [-3.0, -2.0, -2.5, -9.0, -2.0], [0.0, 0.0, 0.0, 0.0, 0.0]])
    w, i = mx.route_scores(z.to(device), 2, "softmax_top")
    assert i.cpu().tolist() == [[0, 1], [1, 4], [0, 1]]                       # ties: the lower index
    want = torch.softmax(torch.tensor([[2.0, 1.0], [-2.0, -2.0], [0.0, 0.0]]), -1)   # over the chosen two only
    assert torch.allclose(w.cpu(), want, atol=1e-6)
    w1, i1 = mx.route_scores(z.to(device), 1, "softmax_top")
    assert i1.cpu().tolist() == [[0], [1], [0]] and torch.equal(w1.cpu(), torch.ones(3, 1))


@pytest.mark.parametrize("device", DEVICES)
def test_routed_ff_bucketed_and_dense_forms_agree(device, monkeypatch):
    cfgd = small_config("L")
    eng, sd = build(cfgd, device, torch.float32)
    toks = tokens(80, cfgd["vocab"], 31)
    want = oracle.forward(cfgd, sd, toks)
    monkeypatch.setattr(blocks, "DENSE_MAX_PAIRS", 0)          # every step buckets rows by expert
    close(run_whole(eng, "a", toks), want, torch.float32)
    monkeypatch.setattr(blocks, "DENSE_MAX_PAIRS", 1 << 30)    # every step runs all experts densely
    close(run_whole(eng, "b", toks), want, torch.float32)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
def test_logit_scale_and_cap(device, dtype):
    x = torch.linspace(-40, 40, 101).to(dtype)
    got = mx.logit_cap(x.clone().to(device), 0.5, 6.0).float().cpu()
    want = 6.0 * torch.tanh(x.float() * 0.5 / 6.0)
    assert torch.allclose(got, want, atol=1e-5 if dtype == torch.float32 else 0.05) and got.abs().max() <= 6.0
    assert torch.equal(mx.logit_cap(x.clone().to(device), 2.0, 0.0).float().cpu(), (x.float() * 2.0).to(dtype).float())


# ---------------------------------------------------------------------------------------------------
# generation through the engine's own scheduler
# ---------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("device,graphs", [("cpu", False), pytest.param("cuda", False, marks=pytest.mark.gpu),
                                           pytest.param("cuda", True, marks=pytest.mark.gpu)])
@pytest.mark.parametrize("async_", [False, True])
def test_greedy_generation(device, graphs, async_):
    cfgd = small_config("lRaL", vocab=256)
    eng, sd = build(cfgd, device, torch.float32, blocks_=12, seqs=2, graphs=graphs, async_=async_)
    poison(eng)
    prompts = [tokens(70, 256, 41), tokens(9, 256, 42), tokens(30, 256, 43)]     # three requests, two slots
    outs = eng.generate(prompts, SamplingParams(temperature=0.0, max_tokens=12, ignore_eos=True))
    for p, o in zip(prompts, outs):
        assert o == oracle.greedy(cfgd, sd, p, 12)
    assert eng.state_slots.num_free() == 2 and eng.bm.num_free() == eng.bm.num_blocks
    if graphs:
        assert eng.runner.stats["graph_steps"] > 0


@pytest.mark.gpu
def test_sampling_reads_the_capped_logits():
    """A model of a width the fused LM-head sampler accepts still samples from scaled, capped logits."""
    cfgd = small_config("l", width=256, vocab=512)
    eng, sd = build(cfgd, "cuda", torch.bfloat16)
    assert not eng.runner._fused_sampling(torch.zeros(2, 256, dtype=torch.bfloat16, device="cuda"))
    outs = eng.generate([tokens(20, 512, 1)], SamplingParams(temperature=0.0, max_tokens=4, ignore_eos=True))
    assert len(outs[0]) == 4


def test_preemption_recomputes_state():
    """A pool too small for both sequences: the younger one is preempted, gives its slot back and is
    recomputed from its first token."""
    cfgd = small_config("aL", vocab=256)
    eng, sd = build(cfgd, "cpu", torch.float32, blocks_=3, seqs=2)
    prompts = [tokens(60, 256, 51), tokens(62, 256, 52)]
    outs = eng.generate(prompts, SamplingParams(temperature=0.0, max_tokens=10, ignore_eos=True))
    assert eng.scheduler.num_preemptions > 0
    for p, o in zip(prompts, outs):
        assert o == oracle.greedy(cfgd, sd, p, 10)


def test_registry_and_config_errors():
    from financial_chatbot_llm_amd.models import get_model_config
    c = get_model_config("tukedra-tiny")
    assert c.arch == "tukedra" and len(c.layers) == c.num_layers and c.streams == 2 and c.logit_softcap == 20.0
    bad = copy.deepcopy(example_config())
    bad["layers"][0]["type"] = "gla"                 # a mixer of another design
    with pytest.raises(ValueError):
        TukedraModel(layered_config(bad, "bad"), device="cpu")
    bad = copy.deepcopy(example_config())
    bad["layers"][0]["mlp"]["kind"] = "other"
    with pytest.raises(ValueError):
        TukedraModel(layered_config(bad, "bad"), device="cpu")
    bad = copy.deepcopy(example_config())
    bad["layers"][0]["mixer"]["decay"] = [0.5]       # one decay per head
    with pytest.raises(ValueError):
        TukedraModel(layered_config(bad, "bad"), device="cpu")
    bad = copy.deepcopy(example_config())
    bad["layers"][2]["mixer"]["vdim"] = 20           # the values are the keys
    with pytest.raises(ValueError):
        TukedraModel(layered_config(bad, "bad"), device="cpu")
    bad = copy.deepcopy(example_config())
    bad["streams"] = 17
    with pytest.raises(ValueError):
        TukedraModel(layered_config(bad, "bad"), device="cpu")
    m = TukedraModel(layered_config(example_config(), "ok"), device="cpu")
    sd = random_weights(m, 0)
    m.load_state(sd)
    short = dict(sd)
    short["l0.hc1.mix"] = sd["l0.hc1.mix"][:1]
    with pytest.raises(ValueError):
        m.load_state(short)
    short = dict(sd)
    short.pop("l2.mix.q.b")
    with pytest.raises(KeyError):
        m.load_state(short)
    m.init_random(seed=3)                            # registry examples run with random weights
