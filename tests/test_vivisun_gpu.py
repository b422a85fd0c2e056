"""The Vivisun decoder in the engine against the plain decoder (plain_vivisun.py): the new kernels one by one, every
mechanism alone at many sizes, the replay regimes (whole prompts, decoding through the cache and the state, portions
down to two tokens, mixed batches under a pool and slots that are used again), inputs made so that a far key, a sink,
a convolution's first taps or a pass's own cache shows in the logits, long decoding, and greedy generation through
the scheduler."""
from __future__ import annotations

import pytest
import torch

from emulated_kernels import EmulatedKernels
from llm_rs_amd import Engine, StepEntry
from llm_rs_amd.engine.trace import TraceReplayer
from llm_rs_amd.kernels import kernels
from plain_vivisun import plain_dyt, plain_vivisun_logits
from replay_cases import collect, live_token_need, mixed, portions, random_tokens, tail_decoded, whole
from vivisun_cases import (BENT, CONFIGS, PAGE_SIZE, allowed_error, attention, check_rows, config, dense, latent, make_folder, make_model,
                           one_layer, reference)

pytestmark = pytest.mark.gpu
DTYPES = ["float32", "bfloat16"]


def replay(engine, steps):
    replayer = TraceReplayer.for_engine(engine)
    outputs = []
    for step in steps:
        out = replayer.step(step)
        outputs.append(None if out is None else torch.from_numpy(out.copy()))
    return collect(steps, outputs)


def engine_for(typed, tensors, dtype, page_size, tokens, max_requests=4):
    return Engine(typed, tensors, dtype=dtype, page_size=page_size, num_pages=max(-(-tokens // page_size), 1), max_requests=max_requests)


def run_regimes(cfg, typed, tensors, dtype, page_size, requests, regimes, allowed=None):
    exact = reference(cfg, tensors, requests)
    allowed = allowed if allowed is not None else allowed_error(dtype, cfg, tensors, requests, exact)
    for name, steps in regimes.items():
        eng = engine_for(typed, tensors, dtype, page_size, live_token_need(steps, 64))
        check_rows(replay(eng, steps), exact, requests, allowed, name)
        core = eng.cache.core
        assert core.slots_in_use() == 0 and all(core.pages_free(g) == core.pages_total(g) for g in range(core.n_groups)), name


def close(got, want, dtype, what=""):
    tol = 2e-6 if dtype == torch.float32 else 1e-2
    err = float((got.detach().cpu().double() - want.double()).abs().max())
    assert err <= tol * max(float(want.abs().max()), 1e-3), (what, err, float(want.abs().max()))


# ---- the kernels one by one, against the same operation in plain tensor code ---------------------------------------

@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_dynamic_tanh(dtype):
    g = torch.Generator().manual_seed(0)
    k = kernels()
    for T, D in ((1, 7), (5, 64), (21, 1000), (3, 1030), (300, 72), (2, 4100)):
        x = torch.randn(T, D, generator=g) * 3
        w, b, w2, b2 = (torch.randn(D, generator=g) for _ in range(4))
        a, a2 = torch.tensor([0.7]), torch.tensor([-1.3])
        got = torch.empty(T, D, dtype=dtype, device="cuda")
        k.dyt(got, x.cuda(), w.cuda(), b.cuda(), a.cuda())
        close(got, plain_dyt(x.double(), w.double(), b.double(), a.double()), dtype, f"dyt {T}x{D}")
        got2 = torch.empty(T, D, dtype=dtype, device="cuda")
        got.zero_()
        k.dyt(got, x.cuda(), w.cuda(), b.cuda(), a.cuda(), second=(got2, w2.cuda(), b2.cuda(), a2.cuda()))
        close(got, plain_dyt(x.double(), w.double(), b.double(), a.double()), dtype, f"dyt twice, first {T}x{D}")
        close(got2, plain_dyt(x.double(), w2.double(), b2.double(), a2.double()), dtype, f"dyt twice, second {T}x{D}")
        rows = torch.tensor([T - 1, 0], dtype=torch.int32)
        some = torch.empty(2, D, dtype=dtype, device="cuda")
        k.dyt(some, x.cuda(), w.cuda(), b.cuda(), a.cuda(), rows.cuda())
        close(some, plain_dyt(x[rows.long()].double(), w.double(), b.double(), a.double()), dtype, f"dyt of rows {T}x{D}")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads,n_in,n_out", [(1, 1, 1), (3, 5, 9), (2, 8, 16), (4, 64, 256), (8, 256, 64), (5, 24, 40), (2, 136, 72), (3, 32, 18),
                                              (1, 512, 128)])
def test_every_head_by_its_own_matrix(heads, n_in, n_out, dtype):
    g = torch.Generator().manual_seed(heads * 1000 + n_in)
    k = kernels()
    w = (torch.randn(heads, n_out, n_in, generator=g) * n_in ** -0.5).to(dtype)
    for T in (1, 8, 16, 17, 100, 600):        # (few rows, rows in one block, many: three tilings with the same sums)
        a = torch.randn(600, heads * n_in, generator=g)[:T].to(dtype)
        gate = torch.randn(T, heads, generator=g) * 2
        want = torch.einsum("thk,hnk->thn", a.double().view(T, heads, n_in), w.double())
        for gt in (None, gate):
            got = torch.empty(T, heads * n_out, dtype=dtype, device="cuda")
            k.head_product(a.cuda(), w.cuda(), got, gate=None if gt is None else gt.cuda())
            ref = want if gt is None else want * (1.0 / (1.0 + torch.exp(-gt.double())))[:, :, None]
            close(got, ref.reshape(T, heads * n_out), dtype, f"{T} rows")
    # rows inside wider rows (a stride), and a row's result is the same bits whatever else is in the step
    a = torch.randn(600, heads * n_in, generator=g).to(dtype)
    full = torch.empty(600, heads * n_out, dtype=dtype, device="cuda")
    k.head_product(a.cuda(), w.cuda(), full)
    for T in (1, 16, 100):
        part = torch.empty(T, heads * n_out, dtype=dtype, device="cuda")
        k.head_product(a[:T].cuda(), w.cuda(), part)
        assert torch.equal(part.cpu(), full[:T].cpu()), T


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_the_small_kernels_around_the_two_attentions(dtype):
    g = torch.Generator().manual_seed(1)
    emu, k = EmulatedKernels(), kernels()
    dev = lambda t: None if t is None else t.cuda()
    # the latent vector: normed, into its pages as a row and as a column; q rounded beside it
    for q_size, rank, page_size in ((6, 9, 4), (64, 128, 16), (40, 500, 16), (256, 64, 8)):
        T, pages = 13, 5
        sums = torch.randn(T, q_size + rank + 3, generator=g)
        w = torch.randn(rank, generator=g)
        slot_map = torch.randperm(pages * page_size, generator=g)[:T].to(torch.int32)
        want_q, got_q = torch.empty(T, q_size, dtype=dtype), torch.empty(T, q_size, dtype=dtype, device="cuda")
        wk, wv = torch.zeros(pages * page_size * rank, dtype=dtype), torch.zeros(pages * page_size * rank, dtype=dtype)
        gk, gv = wk.cuda(), wv.cuda()
        emu.latent_finish(sums, want_q, q_size, rank, w, 1e-5, slot_map, wk, wv, page_size, pages, True)
        k.latent_finish(sums.cuda(), got_q, q_size, rank, w.cuda(), 1e-5, slot_map.cuda(), gk, gv, page_size, pages, True)
        close(got_q, want_q.float(), dtype, "latent q")
        close(gk, wk.float(), dtype, "latent rows")
        close(gv, wv.float(), dtype, "latent columns")
    # the gate on the heads' outputs, one a feature and one a head
    for T, N, per in ((7, 30, 1), (7, 30, 5), (300, 128, 32), (2, 1024, 64)):
        o = torch.randn(T, N, generator=g).to(dtype)
        gate = torch.randn(T, N // per, generator=g) * 3
        want, got = o.clone(), o.cuda()
        emu.sigmoid_gate(want, gate, per)
        k.sigmoid_gate(got, gate.cuda(), per)
        close(got, want.float(), dtype, "gate")
    # the convolutions' last rows: portions longer and shorter than the taps reach back, and single tokens
    for taps, C in ((2, 5), (4, 64), (5, 130)):
        lengths, slots = [1, 7, 2, taps - 1, 3], [4, 0, 2, 5, 1]
        starts = [0]
        for n in lengths:
            starts.append(starts[-1] + n)
        sums = torch.randn(starts[-1], C, generator=g)
        state = torch.randn(6, (taps - 1) * C + 3, generator=g)
        q_starts, sl = torch.tensor(starts, dtype=torch.int32), torch.tensor(slots, dtype=torch.int32)
        want, got = state.clone(), state.cuda()
        emu.conv_state_update(sums, want, q_starts, sl, C, taps)
        k.conv_state_update(sums.cuda(), got, q_starts.cuda(), sl.cuda(), C, taps)
        assert torch.equal(got.cpu(), want), (taps, C)
    # q, k and v from the product's sums: convolved from the state on, normed with a weight, turned with a gain, into pages
    # (rows of whole 16-byte pieces under heads of a power of two go to the kernel with four columns a lane, others not)
    for heads, kv, hd, vd, taps, rot, pad in ((2, 1, 6, 4, 3, 4, 5), (4, 2, 64, 64, 4, 32, 5), (4, 2, 64, 64, 4, 32, 8), (3, 3, 20, 36, 1, 20, 0),
                                              (2, 2, 128, 32, 5, 0, 0), (1, 1, 8, 8, 0, 8, 4), (2, 1, 16, 8, 2, 10, 0), (3, 1, 8, 12, 3, 6, 0),
                                              (5, 5, 32, 4, 1, 32, 0), (2, 1, 256, 64, 4, 64, 0), (1, 1, 8, 8, 4, 2, 3)):
        lengths, slots, page_size, pages = [1, 6, 2, 9], [2, 0, 3, 1], 4, 8
        starts = [0]
        for n in lengths:
            starts.append(starts[-1] + n)
        T, C = starts[-1], (heads + kv) * hd + kv * vd
        full = torch.randn(T, C + pad, generator=g)            # (the rows lie inside wider rows)
        tp = torch.randn(C, taps, generator=g) if taps else None
        state = torch.randn(4, max(taps - 1, 1) * C, generator=g) if taps else None
        token_entry = torch.tensor([e for e, n in enumerate(lengths) for _ in range(n)], dtype=torch.int32)
        q_starts, sl = torch.tensor(starts, dtype=torch.int32), torch.tensor(slots, dtype=torch.int32)
        positions = torch.tensor([5 + i for n in lengths for i in range(n)], dtype=torch.int32)
        inv_freq = torch.rand(rot // 2, generator=g) if rot else None
        qw, kw = torch.randn(hd, generator=g), torch.randn(hd, generator=g)
        slot_map = torch.randperm(pages * page_size, generator=g)[:T].to(torch.int32)
        outs = []
        for kk, to in ((emu, lambda t: t), (k, dev)):
            q = to(torch.empty(T, heads * hd, dtype=dtype))
            kc, vc = to(torch.zeros(pages * kv * page_size * hd, dtype=dtype)), to(torch.zeros(pages * kv * page_size * vd, dtype=dtype))
            conv = None if not taps else (to(tp), to(state) if taps > 1 else None, to(q_starts), to(sl), to(token_entry))
            kk.qkv_finish(to(full)[:, :C], None, q, to(slot_map), kc, vc, heads, kv, hd, vd, page_size, pages, True, 1e-5, to(positions), to(inv_freq), rot,
                          q_weight=to(qw), k_weight=to(kw), gain=1.3, conv=conv)
            outs.append((q, kc, vc))
        for want, got, what in zip(outs[0], outs[1], ("q", "keys", "values")):
            close(got, want.float(), dtype, f"qkv_finish {what} heads of {hd}, {taps} taps")


def plain_sink_attention(q, keys, sink, scale):
    """q [T, H, R] and keys [T, R] of one request, causal: the weighted sums of the keys themselves, [T, H, R]."""
    T = q.shape[0]
    s = torch.einsum("ihr,jr->hij", q, keys) * scale
    s = s.masked_fill(torch.arange(T)[None, :] > torch.arange(T)[:, None], float("-inf"))
    m = torch.maximum(s.max(-1, keepdim=True).values, sink[:, None, None])
    e = torch.exp(s - m)
    p = e / (e.sum(-1, keepdim=True) + torch.exp(sink[:, None, None] - m))
    return torch.einsum("hij,jr->ihr", p, keys)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads,rank", [(3, 9), (8, 64), (4, 128), (16, 256), (2, 160), (5, 320), (40, 32)])
def test_attention_with_a_sink_over_one_latent_head(heads, rank, dtype):
    """Prompt portions and single tokens in one call, over pages in no order; a sink that outweighs the keys for one
    head, one that hardly counts for another."""
    g = torch.Generator().manual_seed(rank)
    k = kernels()
    page_size, T0 = 16, 150
    lengths = [T0, 70, 33]
    scale = 0.3 * rank ** -0.5
    sink = torch.randn(heads, generator=g)
    sink[0], sink[-1] = 8.0, -9.0
    pages_of, n_pages = [], 0
    for n in lengths:
        pages_of.append(list(range(n_pages, n_pages + -(-n // page_size))))
        n_pages += len(pages_of[-1])
    order = torch.randperm(n_pages, generator=g).tolist()
    table = torch.zeros(len(lengths), max(len(p) for p in pages_of), dtype=torch.int32)
    kc, vc = torch.zeros(n_pages, 1, page_size, rank), torch.zeros(n_pages, 1, rank, page_size)
    qs, cs, want = [], [], []
    for e, n in enumerate(lengths):
        q, c = torch.randn(n, heads, rank, generator=g).to(dtype).float(), torch.randn(n, rank, generator=g).to(dtype).float()
        qs.append(q)
        cs.append(c)
        want.append(plain_sink_attention(q.double(), c.double(), sink.double(), scale))
        for j, p in enumerate(pages_of[e]):
            table[e, j] = order[p]
            rows = c[j * page_size:(j + 1) * page_size]
            kc[order[p], 0, :rows.shape[0]] = rows
            vc[order[p], 0, :, :rows.shape[0]] = rows.T
    # the step: the last 40 tokens of the first request, the last token of the second, the last 2 of the third
    new = [40, 1, 2]
    q = torch.cat([qs[e][lengths[e] - n:] for e, n in enumerate(new)]).reshape(sum(new), heads * rank)
    ref = torch.cat([want[e][lengths[e] - n:] for e, n in enumerate(new)]).reshape(sum(new), heads * rank)
    dev = lambda v, t=torch.int32: torch.tensor(v, dtype=t, device="cuda")
    starts = [0, 40, 41, 43]
    token_entry = dev([e for e, n in enumerate(new) for _ in range(n)])
    positions = dev([lengths[e] - n + i for e, n in enumerate(new) for i in range(n)])
    out = torch.empty(sum(new), heads * rank, dtype=dtype, device="cuda")
    need = k.attention_scratch_floats(3, heads, rank, max(lengths), 1, 1)
    scratch = torch.empty(max(need, 1), dtype=torch.float32, device="cuda")
    k.attention(q.to(dtype).cuda(), out, kc.to(dtype).cuda(), vc.to(dtype).cuda(), table.cuda(), token_entry, positions, dev(starts), dev(lengths),
                heads, 1, rank, page_size, n_pages, 0, scale, scratch, max(lengths), 1, sink=sink.cuda())
    close(out, ref, dtype, "with the sink")
    for per in (1, rank):           # the output gate, one a feature and one a head
        gate = torch.randn(sum(new), heads * rank // per, generator=g) * 2
        k.attention(q.to(dtype).cuda(), out, kc.to(dtype).cuda(), vc.to(dtype).cuda(), table.cuda(), token_entry, positions, dev(starts), dev(lengths),
                    heads, 1, rank, page_size, n_pages, 0, scale, scratch, max(lengths), 1, sink=sink.cuda(), gate=gate.cuda(), gate_per=per)
        close(out, ref * (1.0 / (1.0 + torch.exp(-gate.double()))).repeat_interleave(per, dim=1), dtype, f"with a gate for every {per}")
    assert float((ref.view(-1, heads, rank)[:, 0].abs().max())) < 0.5 * float(ref.view(-1, heads, rank)[:, -1].abs().max())     # the sink shows


# ---- each mechanism alone -----------------------------------------------------------------------------------------

ALONE = {
    "attention: three taps, part of the head rotated with bent frequencies": attention(4, 2, 12, 12, 0.4, conv=3, rot_dims=6, base=100.0, scaling=BENT),
    "attention: no convolution, no rotation, wide values": attention(3, 3, 8, 24, 1.3, conv=0, rot_dims=None, mlp=dense(32)),
    "attention: one tap, the whole head rotated, one key head": attention(5, 1, 20, 4, 0.05, conv=1, rot_dims=20, base=50.0),
    "attention: five taps, a rotation of two features": attention(2, 2, 16, 16, 0.25, conv=5, rot_dims=2, mlp=dense(24)),
    "attention: heads of 64 in pairs": attention(4, 2, 64, 64, 0.11, conv=4, rot_dims=32, scaling=BENT, mlp=dense(16)),
    "attention: heads of 32, seven to a key head": attention(7, 1, 32, 32, 0.3, conv=2, rot_dims=10),
    "attention: heads of 128, values of 32": attention(2, 1, 128, 32, 0.09, conv=4, rot_dims=64, base=200000.0,
                                                       scaling={"factor": 16.0, "original": 64, "fast": 24.0, "slow": 2.0}),
    "attention: one head of one key": attention(1, 1, 2, 1, 1.0, conv=2, rot_dims=2),
    "latent: narrow": latent(3, 5, 7, 9, 0.4),
    "latent: one head, a feed-forward": latent(1, 13, 4, 17, 0.2, mlp=dense(17)),
    "latent: a vector of 64 under heads of 16": latent(4, 16, 16, 64, 0.25, mlp=dense(40)),
    "latent: a vector of 128, wide values": latent(8, 32, 48, 128, 0.18),
    "latent: a vector of 256 under many heads": latent(16, 24, 8, 256, 0.2),
    "latent: a vector narrower than a head": latent(2, 64, 64, 32, 0.12, mlp=dense(8)),
    "latent: a vector of 160": latent(6, 8, 8, 160, 0.35),
}


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("which", list(ALONE))
def test_one_layer_of_each_kind(which, dtype):
    cfg = one_layer(ALONE[which], width=48 if "64" in which or "128" in which or "256" in which else 40)
    typed, tensors = make_model(cfg, seed=1)
    requests = {f"r{i}": random_tokens(cfg["vocab"], n, i) for i, n in enumerate([37, 1, 2, 70])}
    run_regimes(cfg, typed, tensors, dtype, 4 if "narrow" in which or "taps" in which else 16, requests,
                {"whole": whole(requests), "decoded": tail_decoded(requests, tail=5), "portions": portions(requests, (2, 3, 30)),
                 "mixed": mixed(requests, live=3, prefill_sizes=(3, 2, 9))})


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("loop", [None, (0, 1, 1), (0, 2, 3), (1, 3, 2), (2, 3, 4), (0, 3, 2), (1, 1, 5)])
def test_stretches_of_layers_that_run_again(loop, dtype):
    """Every pass has caches and convolution states of its own and sees the embeddings again: three layers of which
    none, the first two, the last two, the last or all run several times."""
    cfg = config(40, 61, [attention(2, 1, 8, 12, 0.3, conv=3, rot_dims=4, mlp=dense(24)), latent(3, 6, 5, 10, 0.4),
                          attention(4, 4, 6, 6, 0.5, conv=2, rot_dims=6, mlp=dense(16))], loop=loop)
    typed, tensors = make_model(cfg, seed=2)
    requests = {f"r{i}": random_tokens(61, n, 30 + i) for i, n in enumerate([29, 2, 50, 1, 11])}
    run_regimes(cfg, typed, tensors, dtype, 4, requests,
                {"whole": whole(requests), "decoded": tail_decoded(requests, tail=7), "portions": portions(requests, (2, 3, 13)),
                 "mixed": mixed(requests, live=4, prefill_sizes=(3, 2, 9))})


# ---- whole models in every regime -----------------------------------------------------------------------------------

@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("which", list(CONFIGS))
def test_replay_regimes(which, dtype):
    cfg = CONFIGS[which]
    typed, tensors = make_model(cfg, seed=3)
    lengths = [1, 2, 23, 70, 131, 40, 17]          # more requests than slots: slots and pages are used again
    requests = {f"r{i}": random_tokens(cfg["vocab"], n, 10 + i) for i, n in enumerate(lengths)}
    run_regimes(cfg, typed, tensors, dtype, PAGE_SIZE[which], requests,
                {"whole": whole(requests), "decoded": tail_decoded(requests, tail=32), "portions": portions(requests),
                 "portions of two and three": portions(requests, (2, 3)), "mixed": mixed(requests, live=4),
                 "mixed, two live": mixed(requests, live=2, prefill_sizes=(2, 31, 4))})


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_batch_of_unequal_requests_equals_each_alone(dtype):
    cfg = CONFIGS["odd"]
    typed, tensors = make_model(cfg, seed=5)
    requests = {"long": random_tokens(cfg["vocab"], 90, 1), "short": random_tokens(cfg["vocab"], 2, 2),
                "one": random_tokens(cfg["vocab"], 1, 3), "mid": random_tokens(cfg["vocab"], 33, 4)}
    eng = engine_for(typed, tensors, dtype, 4, 4 * 128)
    together = [{"step": 0, "entries": [{"id": r, "tokens": t, "want": list(range(len(t)))} for r, t in requests.items()], "end": list(requests)}]
    rows_together = replay(eng, together)
    rows_alone = replay(eng, whole(requests))        # the same engine: the slots and pages of the batch, used again
    exact = reference(cfg, tensors, requests)
    allowed = allowed_error(dtype, cfg, tensors, requests, exact)
    check_rows(rows_together, exact, requests, allowed, "together")
    check_rows(rows_alone, exact, requests, allowed, "alone")


# ---- inputs under which a fault shows -------------------------------------------------------------------------------

def with_loud_values(t, layer="l0"):
    """Values large enough that which keys a query weighs shows in the logits."""
    for leaf, factor in (("v", 64.0), ("uv", 8.0)):
        if f"{layer}.mix.{leaf}" in t:
            t[f"{layer}.mix.{leaf}"] = (t[f"{layer}.mix.{leaf}"].double() * factor).to(torch.bfloat16)


def marked_model(kind, shape, mark=7, width=48, vocab=50):
    """One layer in which the key of token `mark` stands out for every query, wherever it stands.  The mixer's input
    is made to hold a one at feature 0 (the norm's weight there is 0, its bias 1) and the query matrix to read nothing
    else, so every query is the same vector: in a latent layer, for each head, the marked token's key scaled so that
    its score is `loudness` (keys have no positions); in an attention layer, with one tap so that a key is its
    token's own, the last feature of a head, which no rotation touches and only the marked token's key has."""
    if kind == "latent":
        cfg = one_layer(latent(shape["heads"], shape["dim"], shape["vdim"], shape["rank"], 1.0), width=width, vocab=vocab)
    else:
        cfg = one_layer(attention(shape["heads"], shape["kv_heads"], shape["dim"], shape["vdim"], 1.0, conv=1, rot_dims=shape["rot_dims"]), width=width, vocab=vocab)

    loudness = shape.get("loudness", 14.0)

    def change(t):
        d = lambda n: t[n].double()
        t["l0.norm1.b"][0], t["l0.norm1"][0] = 1.0, 0.0
        h = plain_dyt(d("embed")[mark], d("l0.norm1"), d("l0.norm1.b"), d("l0.norm1.alpha"))
        H, dim = shape["heads"], shape["dim"]
        wq = torch.zeros(H * dim, width, dtype=torch.float64)
        if kind == "latent":
            c = d("l0.mix.dkv") @ h
            c = (c / torch.sqrt((c * c).mean() + 1e-5) * d("l0.mix.dkv.norm")).to(torch.bfloat16).double()
            key = (d("l0.mix.uk") @ c).view(H, dim)
            wq[:, 0] = (loudness * key / (key * key).sum(-1, keepdim=True)).reshape(-1)
            t["l0.mix.sink"] = torch.full_like(t["l0.mix.sink"], -2.0)
        else:
            # only the marked token has feature 1 of the mixer's input, only the last feature of a key (which is not
            # rotated) reads it, and every query is that feature alone: the marked key scores `loudness`, the others 0
            G = shape["kv_heads"]
            assert shape["rot_dims"] < dim
            t["embed"][:, 1] = 0.0
            t["embed"][mark, 1] = 8.0
            t["l0.norm1"][1], t["l0.norm1.b"][1] = 1.0, 0.0
            wk = d("l0.mix.k")
            for g in range(G):
                wk[g * dim + dim - 1] = 0.0
                wk[g * dim + dim - 1, 1] = 30.0
            t["l0.mix.k"] = wk.to(torch.bfloat16)
            t["l0.mix.k.conv"], t["l0.mix.q.conv"] = torch.ones_like(t["l0.mix.k.conv"]), torch.ones_like(t["l0.mix.q.conv"])
            h = plain_dyt(d("embed")[mark], d("l0.norm1"), d("l0.norm1.b"), d("l0.norm1.alpha"))
            key = (d("l0.mix.k") @ h).view(G, dim)
            key = key / torch.sqrt((key * key).mean(-1, keepdim=True) + 1e-5) * d("l0.mix.k.norm")
            wq[dim - 1::dim, 0] = 1.0
            nw = torch.zeros(dim, dtype=torch.float64)
            nw[dim - 1] = loudness / (dim ** 0.5 * float(key[:, dim - 1].mean()))
            t["l0.mix.q.norm"] = nw.to(torch.bfloat16)
        t["l0.mix.q"] = wq.to(torch.bfloat16)
        with_loud_values(t)
    typed, tensors = make_model(cfg, seed=11, change=change)
    return cfg, typed, tensors


def sequence_with_mark(vocab, n, at, mark, seed):
    toks = [t if t != mark else (t + 1) % vocab for t in random_tokens(vocab, n, seed)]
    toks[at] = mark
    return toks


def shows(cfg, tensors, toks, at, where):
    """How far the logits at `where` move when the token at `at` is another one, as a part of the largest logit."""
    exact = reference(cfg, tensors, {"m": toks})["m"]
    other = [t if i != at else (t + 2) % cfg["vocab"] for i, t in enumerate(toks)]
    return float((reference(cfg, tensors, {"m": other})["m"][where] - exact[where]).abs().max()) / float(exact.abs().max())


MARKED = {"latent, any sizes": ("latent", dict(heads=3, dim=10, vdim=6, rank=12, loudness=40.0)),
          "latent, a vector of 64": ("latent", dict(heads=4, dim=16, vdim=16, rank=64)),
          "latent, a vector of 128": ("latent", dict(heads=4, dim=32, vdim=24, rank=128)),
          "latent, a vector of 256": ("latent", dict(heads=2, dim=64, vdim=32, rank=256)),
          "attention, any sizes": ("attention", dict(heads=2, kv_heads=1, dim=16, vdim=12, rot_dims=8)),
          "attention, heads of 64": ("attention", dict(heads=4, kv_heads=2, dim=64, vdim=64, rot_dims=32)),
          "attention, heads of 128": ("attention", dict(heads=2, kv_heads=1, dim=128, vdim=128, rot_dims=64))}


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("which", list(MARKED))
def test_a_far_key_among_hundreds_across_pages(which, dtype):
    kind, shape = MARKED[which]
    cfg, typed, tensors = marked_model(kind, shape)
    for at in (0, 15, 16, 250):
        toks = sequence_with_mark(cfg["vocab"], 600, at, 7, seed=at)
        requests = {"m": toks}
        exact = reference(cfg, tensors, requests)
        assert shows(cfg, tensors, toks, at, 599) > 0.05, (which, at)
        allowed = allowed_error(dtype, cfg, tensors, requests, exact)
        for name, steps in {"whole": whole(requests), "decoded": tail_decoded(requests, tail=40),
                            "portions": portions(requests, (64, 3, 130, 2))}.items():
            eng = engine_for(typed, tensors, dtype, 16, 640)
            check_rows(replay(eng, steps), exact, requests, allowed, f"mark at {at}, {name}")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("rank,heads", [(12, 3), (64, 4), (128, 8), (256, 4)])
def test_a_sink_that_outweighs_the_keys(rank, heads, dtype):
    """Sinks of +5 (first head: nearly all of the weight), -5 (hardly any) and between: left out, counted twice, scaled
    or given to the wrong head, each moves the logits by far more than rounding does."""
    cfg = one_layer(latent(heads, 16, 16, rank, 0.25), width=48)

    def change(t):
        t["l0.mix.sink"] = torch.linspace(5.0, -5.0, heads).to(torch.bfloat16)
        with_loud_values(t)
    typed, tensors = make_model(cfg, seed=13, change=change)
    requests = {"a": random_tokens(61, 200, 1), "b": random_tokens(61, 3, 2)}
    exact = reference(cfg, tensors, requests)
    least = 1.0
    for wrong in (lambda s: torch.full_like(s, -60.0), lambda s: s + 0.6931, lambda s: s.flip(0), lambda s: s * 0.25):
        other = dict(tensors)
        other["l0.mix.sink"] = wrong(tensors["l0.mix.sink"].float()).to(torch.bfloat16)
        moved = float((reference(cfg, other, requests)["a"] - exact["a"]).abs().max()) / float(exact["a"].abs().max())
        assert moved > 0.02, moved
        least = min(least, moved)
    allowed = allowed_error(dtype, cfg, tensors, requests, exact)
    assert allowed < 0.6 * least, (allowed, least)
    run_regimes(cfg, typed, tensors, dtype, 16, requests,
                {"whole": whole(requests), "decoded": tail_decoded(requests, tail=40), "portions": portions(requests, (2, 70, 3)),
                 "both at once": mixed(requests, live=2, prefill_sizes=(40, 2, 7))}, allowed)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("taps", [2, 4, 5])
def test_the_first_tokens_and_the_taps_across_portions(taps, dtype):
    """Loud early taps: what the convolution reads before a sequence's start (zeros), before a portion's start (the
    request's state, also where a portion is shorter than the taps reach back) and in a slot that another request
    left shows in the logits."""
    cfg = one_layer(attention(2, 1, 8, 8, 0.4, conv=taps, rot_dims=4, mlp=dense(16)), width=32, vocab=40)

    def change(t):
        for n in ("q", "k", "v"):
            w = t[f"l0.mix.{n}.conv"].double()
            w[:, 0] = 3.0 * (1 + w[:, 0].abs())              # the tap that reaches furthest back
            t[f"l0.mix.{n}.conv"] = w.to(torch.bfloat16)
        with_loud_values(t)
    typed, tensors = make_model(cfg, seed=17, change=change)
    requests = {f"r{i}": random_tokens(40, n, 40 + i) for i, n in enumerate([1, 2, 3, taps - 1, taps, taps + 1, 12, 31])}
    exact = reference(cfg, tensors, requests)
    # the tap shows: another token `taps - 1` places back moves the logits
    toks = requests["r7"]
    other = plain_vivisun_logits(cfg, tensors, [(t + 1) % 40 if i == 30 - (taps - 1) else t for i, t in enumerate(toks)])
    assert float((other[30] - exact["r7"][30]).abs().max()) / float(exact["r7"].abs().max()) > 0.02
    run_regimes(cfg, typed, tensors, dtype, 4, requests,
                {"whole": whole(requests), "decoded": tail_decoded(requests, tail=8), "token by token": tail_decoded(requests, tail=1000),
                 "portions of two": portions(requests, (2,)), "portions of two and three": portions(requests, (3, 2)),
                 "portions": portions(requests, (1, 2, 1, 5, 2)), "mixed": mixed(requests, live=3, prefill_sizes=(2, 3, 1, 4))})


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_slot_used_again_starts_from_nothing(dtype):
    cfg = CONFIGS["plain"]

    def change(t):
        for name in list(t):
            if name.endswith(".conv"):
                t[name] = (t[name].double() * 3).to(torch.bfloat16)
    typed, tensors = make_model(cfg, seed=4, change=change)
    first, second = random_tokens(cfg["vocab"], 50, 1), random_tokens(cfg["vocab"], 30, 2)
    eng = Engine(typed, tensors, dtype=dtype, page_size=16, num_pages=8, max_requests=1)      # one slot, pages for one request
    exact = reference(cfg, tensors, {"first": first, "second": second})
    allowed = allowed_error(dtype, cfg, tensors, {"first": first, "second": second}, exact)
    for rid, toks in (("first", first), ("second", second), ("first", first)):
        slot = eng.open_request()
        assert slot == 0
        head = eng.step([StepEntry(slot, 0, toks[:20], list(range(20)))]).cpu().clone()
        tail = eng.step([StepEntry(slot, 20, toks[20:], list(range(len(toks) - 20)))]).cpu()
        eng.close_request(slot)
        got = torch.cat([head, tail]).double()
        err = float((got - exact[rid]).abs().max()) / float(exact[rid].abs().max())
        assert err <= allowed, (rid, err, allowed)


@pytest.mark.parametrize("dtype", DTYPES)
def test_long_decoding_with_recorded_steps(dtype):
    cfg = CONFIGS["odd"]
    typed, tensors = make_model(cfg, seed=6)
    requests = {"a": random_tokens(cfg["vocab"], 330, 1), "b": random_tokens(cfg["vocab"], 321, 2)}
    exact = reference(cfg, tensors, requests)
    allowed = allowed_error(dtype, cfg, tensors, requests, exact)
    steps = [{"step": 0, "entries": [{"id": r, "tokens": t[:9], "want": list(range(9))} for r, t in requests.items()], "end": []}]
    for i in range(9, 330):
        live = [r for r, t in requests.items() if i < len(t)]
        steps.append({"step": len(steps), "entries": [{"id": r, "tokens": [requests[r][i]], "want": [0]} for r in live],
                      "end": [r for r in live if i == len(requests[r]) - 1]})
    eng = engine_for(typed, tensors, dtype, 4, 704)
    check_rows(replay(eng, steps), exact, requests, allowed, "decoding")
    assert eng.runner.graph_replays > 100           # the single-token steps were recorded and replayed


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_step_of_more_than_a_thousand_tokens(dtype):
    cfg = config(64, 40, [attention(2, 1, 32, 32, 0.2, conv=4, rot_dims=16, scaling=BENT, mlp=dense(24)), latent(4, 8, 12, 64, 0.3, mlp=dense(16))],
                 loop=(0, 2, 2))
    typed, tensors = make_model(cfg, seed=12)
    requests = {"a": random_tokens(40, 1100, 1), "b": random_tokens(40, 40, 2)}
    exact = reference(cfg, tensors, requests)
    allowed = allowed_error(dtype, cfg, tensors, requests, exact)
    cuts = {"a": 1031, "b": 5}
    steps = [{"step": 0, "entries": [{"id": r, "tokens": t[:cuts[r]], "want": list(range(cuts[r]))} for r, t in requests.items()], "end": []},
             {"step": 1, "entries": [{"id": r, "tokens": t[cuts[r]:], "want": list(range(len(t) - cuts[r]))} for r, t in requests.items()], "end": list(requests)}]
    eng = engine_for(typed, tensors, dtype, 16, 1280)
    check_rows(replay(eng, steps), exact, requests, allowed, "two steps")


# ---- configurations drawn at random -----------------------------------------------------------------------------------

def random_configuration(seed):
    import random
    r = random.Random(seed)
    width = r.choice([24, 40, 64, 96, 136])
    layers = []
    for _ in range(r.randint(2, 5)):
        mlp = r.choice([None, dense(8 * r.randint(2, 12)), dense(r.randint(5, 70))])
        if r.random() < 0.5:
            heads = r.choice([1, 2, 3, 4, 8, 12])
            layers.append(latent(heads, r.choice([4, 8, 20, 32, 64]), r.choice([4, 12, 32, 64]), r.choice([8, 20, 32, 64, 96, 128, 192, 256]),
                                 r.uniform(0.05, 0.5), mlp))
            continue
        kv = r.choice([1, 2, 3])
        dim = r.choice([8, 20, 32, 64, 128])
        vdim = r.choice([dim, dim, 4 * r.randint(1, 10)])
        layers.append(attention(kv * r.choice([1, 2, 4]), kv, dim, vdim, r.uniform(0.05, 0.5), conv=r.choice([0, 1, 2, 3, 4, 5]),
                                rot_dims=r.choice([None, 0, dim // 2 // 2 * 2, dim]), base=r.choice([100.0, 10000.0, 1000000.0]),
                                scaling=r.choice([None, BENT, {"factor": 6.0, "original": 256, "fast": 16.0, "slow": 0.5}]), mlp=mlp))
    n = len(layers)
    a = r.randint(0, n - 1)
    loop = r.choice([None, (a, r.randint(a, n), r.randint(1, 3))])
    return config(width, r.randint(30, 200), layers, loop=loop, eps=r.choice([1e-5, 1e-6, 1e-3]))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("seed", range(8))
def test_configurations_drawn_at_random(seed, dtype):
    cfg = random_configuration(seed)
    typed, tensors = make_model(cfg, seed=seed)
    requests = {f"r{i}": random_tokens(cfg["vocab"], n, 70 + i) for i, n in enumerate([150, 3, 66, 1, 35])}
    run_regimes(cfg, typed, tensors, dtype, 16, requests,
                {"whole": whole(requests), "decoded": tail_decoded(requests, tail=36), "portions": portions(requests, (2, 70, 3, 33)),
                 "mixed": mixed(requests, live=3)})


# ---- generation through the scheduler --------------------------------------------------------------------------------

def plain_greedy(cfg, tensors, prompt, n):
    toks, margins = list(prompt), []
    for _ in range(n):
        row = plain_vivisun_logits(cfg, tensors, toks)[-1]
        top = torch.topk(row, 2).values
        margins.append(float(top[0] - top[1]) / float(row.abs().max()))
        toks.append(int(torch.argmax(row)))
    return toks[len(prompt):], margins


@pytest.mark.parametrize("which", ["odd", "plain"])
def test_greedy_generation_through_the_scheduler(which):
    cfg = CONFIGS[which]
    typed, tensors = make_model(cfg, seed=8)
    prompts = [random_tokens(cfg["vocab"], n, 20 + n) for n in (1, 5, 19, 40, 3, 27)]
    eng = Engine(typed, tensors, dtype="float32", page_size=PAGE_SIZE[which], num_pages=96, max_requests=3, max_batch_tokens=24)
    outs = eng.generate(prompts, max_new_tokens=12)
    for prompt, out in zip(prompts, outs):
        want, margins = plain_greedy(cfg, tensors, prompt, 12)
        out = list(out.tokens if hasattr(out, "tokens") else out)
        for i, (a, b) in enumerate(zip(out, want)):
            if a != b:
                assert margins[i] < 1e-4, (prompt, i, out, want)       # a tie within rounding may fall either way
                break


# ---- the programs, on a model folder ----------------------------------------------------------------------------------

def test_the_programs_on_a_model_folder(tmp_path):
    """A folder with config.json and model.safetensors through `bin/trace_run` (a mixed trace under a small pool, both
    dtypes) and through `bin/llm-rs complete` (greedy): the architecture is chosen by the file."""
    import json
    import os
    import subprocess
    import sys

    import numpy as np
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    cfg = CONFIGS["plain"]
    folder = make_folder(tmp_path, cfg, seed=11)
    typed, tensors = make_model(cfg, seed=11)
    requests = {f"r{i}": random_tokens(cfg["vocab"], n, 50 + i) for i, n in enumerate([33, 2, 90, 47, 18])}
    exact = reference(cfg, tensors, requests)
    steps = mixed(requests, live=3)
    text = "".join(json.dumps(s) + "\n" for s in steps)
    for dtype in DTYPES:
        out = tmp_path / f"out_{dtype}"
        p = subprocess.run([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", folder, "--dtype", dtype, "--out", str(out),
                            "--max-tokens", str(live_token_need(steps, 64))], input=text, capture_output=True, text=True, timeout=600)
        assert p.returncode == 0, p.stderr[-2000:]
        assert [l for l in p.stdout.split("\n") if l.startswith("done")] == [f"done {s['step']}" for s in steps]
        outputs = []
        for s in steps:
            n = sum(len(e["want"]) for e in s["entries"])
            outputs.append(torch.from_numpy(np.fromfile(out / f"{s['step']}.f32", dtype="<f4").reshape(n, cfg["vocab"]).copy()) if n else None)
        check_rows(collect(steps, outputs), exact, requests, allowed_error(dtype, cfg, tensors, requests, exact), f"trace_run {dtype}")
    prompt = requests["r3"]
    p = subprocess.run([sys.executable, os.path.join(root, "bin", "llm-rs"), "-m", folder, "--dtype", "float32", "--num-pages", "64", "complete",
                        "--prompt-ids", " ".join(map(str, prompt)), "-n", "10", "--temperature", "0"], capture_output=True, text=True, timeout=600)
    assert p.returncode == 0, p.stderr[-2000:]
    got = [int(t) for t in p.stdout.split()]
    want, margins = plain_greedy(cfg, tensors, prompt, 10)
    for i, (a, b) in enumerate(zip(got, want)):
        if a != b:
            assert margins[i] < 1e-4, (i, got, want)
            break
    assert len(got) == 10
