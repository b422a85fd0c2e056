"""The Gokosun decoder in the engine against the plain decoder (plain_gokosun.py): the new kernels one by one, every
mechanism alone at many sizes, the replay regimes (whole prompts, decoding through the cache and the state, portions
down to two tokens, mixed batches under a pool and slots that are used again), inputs made so that a far key, a sink,
the first layer's values, the router's correction or a memory's first token shows in the logits, long decoding, and
greedy generation through the scheduler."""
from __future__ import annotations

import math

import pytest
import torch

from gokosun_cases import (BENT, CONFIGS, PAGE_SIZE, allowed_error, attention, check_rows, config, dense, latent, make_folder, make_model, mlstm,
                           moe, one_layer, reference)
from llm_rs_amd import Engine, StepEntry
from llm_rs_amd.engine.trace import TraceReplayer
from llm_rs_amd.kernels import kernels
from plain_gokosun import (plain_frequencies, plain_gokosun_logits, plain_layernorm, plain_mlstm_gates, plain_mlstm_head, plain_rmsnorm,
                           plain_rotate, plain_route, plain_sigmoid)
from replay_cases import collect, live_token_need, mixed, portions, random_tokens, tail_decoded, whole

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
        check_rows(replay(eng, steps), exact, requests, allowed, name, few_may_pass=dtype == "bfloat16")
        core = eng.cache.core
        assert core.slots_in_use() == 0 and all(core.pages_free(g) == core.pages_total(g) for g in range(core.n_groups)), name


def close(got, want, dtype, what="", tol=None):
    tol = tol if tol is not None else (3e-6 if dtype == torch.float32 else 1e-2)
    err = float((got.detach().cpu().double() - want.double()).abs().max())
    assert err <= tol * max(float(want.abs().max()), 1e-3), (what, err, float(want.abs().max()))


def rand(*shape, seed=0, scale=1.0):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed), dtype=torch.float32) * scale


# ---- the kernels one by one, against the same operation in plain tensor code ---------------------------------------

@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("D", [1, 5, 46, 320, 1024, 1500, 4096, 5000, 9001])
def test_layer_norm(D, dtype):
    x = rand(7, D, seed=D) * 3.0 + 5.0            # a mean that a sum of squares without it would drown the deviations in
    w, b = 1.0 + rand(D, seed=1) * 0.1, rand(D, seed=2)
    want = plain_layernorm(x.double(), w.double(), b.double(), 1e-5)
    out = torch.empty(7, D, dtype=dtype, device="cuda")
    kernels().layernorm(out, x.cuda(), w.cuda(), b.cuda(), 1e-5)
    close(out, want, dtype, "every row")
    rows = torch.tensor([6, 0, 3], dtype=torch.int32)
    out = torch.empty(3, D, dtype=dtype, device="cuda")
    kernels().layernorm(out, x.cuda(), w.cuda(), b.cuda(), 1e-5, rows.cuda())
    close(out, want[rows.long()], dtype, "gathered rows")


@pytest.mark.parametrize("heads,dk,dv", [(1, 1, 1), (3, 5, 7), (2, 16, 32), (4, 48, 40), (2, 64, 64), (1, 128, 96), (2, 200, 24), (1, 320, 130)])
def test_the_matrix_memory_with_its_gates(heads, dk, dv):
    """The gates' kernel, the recurrence with gates that move with the token and a column of ones, and the read-out's
    division and norm, against the plain head walked token by token; entries of 1, 2 and 150 tokens, one of them
    continuing a state that an earlier call left."""
    k = kernels()
    lens = [150, 1, 2, 70]
    T, cap, eps = sum(lens), 6.0, 1e-5
    q, kk, v = rand(T, heads * dk, seed=1), rand(T, heads * dk, seed=2), rand(T, heads * dv, seed=3)
    gi, gf = rand(T, heads, seed=4) * 4.0, rand(T, heads, seed=5) * 4.0 + 2.0
    bi, bf = rand(heads, seed=6), rand(heads, seed=7)
    gate, w = rand(T, heads * dv, seed=8), 1.0 + rand(heads * dv, seed=9) * 0.1
    cols = dv + 1
    n_matrix = heads * cols * dk
    state = torch.zeros(5, n_matrix + heads, device="cuda")
    q_starts = torch.tensor([0, 150, 151, 153, 223], dtype=torch.int32).cuda()
    slots = torch.tensor([3, 0, 4, 1], dtype=torch.int32).cuda()
    d = lambda t: t.cuda()
    gates = torch.empty(3, T, heads, device="cuda")

    def run(lo, hi, starts, slot_ids):
        n = hi - lo
        sums_g = torch.cat([gi[lo:hi], gf[lo:hi]], dim=1).cuda()
        k.exp_gates(sums_g[:, :heads], sums_g[:, heads:], d(bi), d(bf), cap, state[:, n_matrix:], starts, slot_ids, gates[0, :n], gates[1, :n], gates[2, :n])
        o = torch.empty(n, heads * cols, device="cuda")
        k.linear_scan(d(q[lo:hi]), d(kk[lo:hi]), d(v[lo:hi]), state[:, :n_matrix], starts, slot_ids, heads, heads, dk, cols, o,
                      gates=(gates[0, :n], gates[1, :n]), v_cols=dv)
        out = torch.empty(n, heads * dv, device="cuda")
        k.gated_rmsnorm(out, o, d(gate[lo:hi]), d(w), dv, eps, floor=gates[2, :n], x_scale=dk ** -0.5, den_add=1e-6)
        return out.cpu()
    got = run(0, T, q_starts, slots)
    # the last entry once more in two calls, from an empty slot: its first 33 tokens, then the rest from the state
    state[2].zero_()
    two = torch.tensor([2], dtype=torch.int32).cuda()
    a = run(153, 186, torch.tensor([0, 33], dtype=torch.int32).cuda(), two)
    b = run(186, 223, torch.tensor([0, 37], dtype=torch.int32).cuda(), two)
    w64 = {"i": torch.eye(heads).double(), "i.b": bi.double(), "f": torch.eye(heads).double(), "f.b": bf.double()}
    at = 0
    for e, n in enumerate(lens):
        i64, f64 = plain_mlstm_gates(gi[at:at + n].double(), w64, cap)
        f64 = plain_mlstm_gates(gf[at:at + n].double(), w64, cap)[1]
        for h in range(heads):
            o, (S, nn, m) = plain_mlstm_head(q[at:at + n, h * dk:(h + 1) * dk].double() * dk ** -0.5, kk[at:at + n, h * dk:(h + 1) * dk].double(),
                                              v[at:at + n, h * dv:(h + 1) * dv].double(), i64[:, h], f64[:, h])
            cs = slice(h * dv, (h + 1) * dv)
            want = plain_rmsnorm(o, None, eps) * w.double()[cs] * plain_sigmoid(gate[at:at + n, cs].double())
            close(got[at:at + n, cs], want, torch.float32, f"entry {e} head {h}", tol=2e-5)
            st = state[int(slots[e])].cpu().double()
            mem = st[h * cols * dk:(h + 1) * cols * dk].view(cols, dk)
            close(mem[:dv].T, S, torch.float32, f"S of entry {e} head {h}", tol=2e-5)
            close(mem[dv], nn, torch.float32, f"n of entry {e} head {h}", tol=2e-5)
            assert abs(float(st[n_matrix + h]) - float(m)) < 1e-5
            if e == 3:
                close(torch.cat([a, b])[:, cs], want, torch.float32, f"in two calls, head {h}", tol=2e-5)
        at += n


@pytest.mark.parametrize("E,top", [(1, 1), (5, 2), (8, 3), (64, 6), (100, 100), (300, 7)])
def test_the_router_with_sigmoid_scores_and_a_correction(E, top):
    T = 37
    logits, corr = rand(T, E, seed=E) * 2.0, rand(E, seed=1) * 0.5
    weights = torch.empty(T, E, device="cuda")
    kernels().route_topk(logits.cuda(), weights, top, True, "sigmoid", corr.cuda(), 2.5)
    chosen, want = plain_route(logits.double(), {"router": torch.eye(E).double(), "correction": corr.double()}, top, 2.5)
    full = torch.zeros(T, E, dtype=torch.float64).scatter_(1, chosen, want)
    close(weights, full, torch.float32, "weights")
    assert ((weights.cpu() > 0).sum(1) == top).all()
    kernels().route_topk(logits.cuda(), weights, top, False, "sigmoid", None, 1.0)         # as they are, chosen by the score itself
    s = plain_sigmoid(logits.double())
    keep = torch.zeros(T, E, dtype=torch.float64).scatter_(1, torch.topk(s, top, dim=1).indices, 1.0)
    close(weights, s * keep, torch.float32, "scores as they are")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("M", [1, 2, 8, 16, 17, 40, 64, 65, 100, 300, 1031, 2048])
@pytest.mark.parametrize("N,K", [(14, 10), (64, 64), (512, 320), (2048, 256), (6144, 1024)])
def test_the_gate_and_up_product_with_the_clamped_activation(M, N, K, dtype):
    """Every tiling of the product (by its number of rows and its widths) finishes the same activation; two different
    pairs of constants one after the other, as two feed-forwards of a layer have them, each in a slot of its own that
    the same pair gets again."""
    from llm_rs_amd.kernels import EPI_GLU_CLAMP
    x, w = (rand(M, K, seed=M) * 0.8).to(dtype), (rand(N, K, seed=N) * 0.2).to(dtype)
    sums = x.double() @ w.double().T
    for limit, alpha in ((1.25, 1.702), (0.5, 1.0)):
        g, u = torch.clamp(sums[:, 0::2], max=limit), torch.clamp(sums[:, 1::2], min=-limit, max=limit)
        want = g * plain_sigmoid(alpha * g) * (u + 1.0)
        out = torch.empty(M, N // 2, dtype=dtype, device="cuda")
        k = kernels()
        n_ws = k.gemm_workspace_floats(M, N, K)
        ws = torch.empty(n_ws, device="cuda") if n_ws else None
        k.gemm(x.cuda(), w.cuda(), out, EPI_GLU_CLAMP, ws, glu=k.glu_clamp_slot(limit, alpha))
        close(out, want, dtype, f"limit {limit}", tol=5e-5 if dtype == torch.float32 else 1e-2)
        assert k.glu_clamp_slot(limit, alpha) == k.glu_clamp_slot(limit, alpha) != k.glu_clamp_slot(limit + 1.0, alpha)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_the_clamped_gated_activation(dtype):
    T, ff, E = 19, 6, 3
    sums = rand(T, 2 * ff * E, seed=3) * 3.0
    wts = rand(T, E, seed=4).abs()
    g, u = sums[:, 0::2].double(), sums[:, 1::2].double()
    g, u = torch.clamp(g, max=1.25), torch.clamp(u, min=-1.25, max=1.25)
    want = g * plain_sigmoid(1.702 * g) * (u + 1.0)
    out = torch.empty(T, ff * E, dtype=dtype, device="cuda")
    kernels().act_weight(out, sums.cuda(), None, ff * E, "clamped_glu", 1.25, 1.702)
    close(out, want, dtype, "dense")
    kernels().act_weight(out, sums.cuda(), wts.cuda(), ff, "clamped_glu", 1.25, 1.702)
    close(out, want * wts.double().repeat_interleave(ff, dim=1), dtype, "times the experts' weights")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("q_rank,rank,rot", [(7, 9, 2), (40, 24, 8), (128, 96, 32), (200, 256, 64), (1500, 448, 64)])
def test_the_latent_vectors_and_the_rotated_key_part(q_rank, rank, rot, dtype):
    T, page, pages, eps = 11, 4, 5, 1e-5
    sums = rand(T, q_rank + rank + rot + 3, seed=rank)
    qw, cw = 1.0 + rand(q_rank, seed=1) * 0.1, 1.0 + rand(rank, seed=2) * 0.1
    positions = torch.tensor([0, 1, 2, 3, 700, 701, 5, 6, 7, 8, 9], dtype=torch.int32)
    slot_map = torch.tensor([4, 5, 6, 7, 0, 1, 13, 14, 15, 16, 17], dtype=torch.int32)
    freq, gain = plain_frequencies({"dims": rot, "base": 100.0, "scaling": BENT})
    width = rank + rot
    kc, vc = torch.zeros(pages * page * width, dtype=dtype, device="cuda"), torch.zeros(pages * page * width, dtype=dtype, device="cuda")
    cq = torch.empty(T, q_rank, dtype=dtype, device="cuda")
    kernels().latent_finish(sums.cuda(), cq, q_rank, rank, cw.cuda(), eps, slot_map.cuda(), kc, vc, page, pages, True, q_weight=qw.cuda(),
                            rotated=(rot, positions.cuda(), freq.float().cuda(), gain))
    s = sums.double()
    close(cq, plain_rmsnorm(s[:, :q_rank], qw.double(), eps), dtype, "the queries' latent vector")
    c = plain_rmsnorm(s[:, q_rank:q_rank + rank], cw.double(), eps)
    part = plain_rotate(s[:, q_rank + rank:q_rank + width].view(T, 1, rot), positions.tolist(), freq, gain, "pairs")[:, 0]
    want = torch.cat([c, part], dim=1)
    rows = kc.view(pages * page, width).cpu()[slot_map.long()]
    cols = vc.view(pages, width, page).cpu().permute(0, 2, 1).reshape(pages * page, width)[slot_map.long()]
    tol = 3e-5 if dtype == torch.float32 else 1e-2       # (angles of 700 turns in 32-bit)
    close(rows, want, dtype, "as rows", tol=tol)
    close(cols, want, dtype, "as columns", tol=tol)


def test_the_norm_over_the_whole_projection_and_the_mix_of_values():
    T, qc, kc_, vc_ = 9, 30, 12, 10
    sums = rand(T, qc + kc_ + vc_ + 2, seed=5)
    qw, kw = 1.0 + rand(qc, seed=1) * 0.1, 1.0 + rand(kc_, seed=2) * 0.1
    first, lam = rand(T, vc_, seed=3), torch.tensor([0.3])
    s = sums.double()
    x = sums.cuda()
    keep = torch.empty(T, vc_, device="cuda")
    kernels().qkv_whole(x, qc, kc_, vc_, qw.cuda(), kw.cuda(), 1e-5, keep=keep)
    close(x[:, :qc], plain_rmsnorm(s[:, :qc], qw.double(), 1e-5), torch.float32, "q")
    close(x[:, qc:qc + kc_], plain_rmsnorm(s[:, qc:qc + kc_], kw.double(), 1e-5), torch.float32, "k")
    assert torch.equal(keep.cpu(), sums[:, qc + kc_:qc + kc_ + vc_]) and torch.equal(x[:, qc + kc_:].cpu(), sums[:, qc + kc_:])
    x = sums.cuda()
    kernels().qkv_whole(x, qc, kc_, vc_, None, None, 0.0, first=first.cuda(), lam=lam.cuda())
    close(x[:, qc + kc_:qc + kc_ + vc_], 0.7 * s[:, qc + kc_:qc + kc_ + vc_] + 0.3 * first.double(), torch.float32, "mixed values")
    assert torch.equal(x[:, :qc + kc_].cpu(), sums[:, :qc + kc_]) and torch.equal(x[:, -2:].cpu(), sums[:, -2:])


# ---- every mechanism alone ------------------------------------------------------------------------------------------

ALONE = {
    "memory: narrow keys": mlstm(3, 5, 9, cap=3.0),
    "memory: one head, wide": mlstm(1, 130, 20, cap=20.0, mlp=dense(12, 0.5)),
    "memory: heads of 64": mlstm(2, 64, 64),
    "latent: any sizes": latent(3, 5, 2, 7, 9, 4, 0.4, base=30.0, scaling=BENT),
    "latent: a vector of 56 and 8": latent(4, 16, 8, 8, 56, 70, 0.3),
    "latent: a vector of 96 and 32": latent(8, 32, 32, 16, 96, 24, 0.2, scaling={"factor": 8.0, "original": 64, "fast": 4.0, "slow": 0.5}),
    "latent: a vector of 192 and 64": latent(2, 24, 64, 40, 192, 33, 0.15),
    "attention: narrow, three to a key head": attention(6, 2, 10, 6, 0.3, rot_dims=4, base=20.0),
    "attention: heads of 64, all rotated": attention(4, 2, 64, 64, 0.125, rot_dims=64),
    "attention: heads of 32, values of 96, no rotation": attention(3, 3, 32, 96, 0.2),
    "experts beside a shared one": mlstm(1, 4, 4, mlp=moe(7, 3, 9, limit=0.6, scale=2.5, shared=(5, 2.0))),
    "all experts chosen": attention(2, 1, 8, 8, 0.3, rot_dims=8, mlp=moe(3, 3, 6, shared=None)),
    "one expert of many": latent(2, 8, 4, 8, 12, 10, 0.3, mlp=moe(16, 1, 8, scale=0.7)),
}


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("which", list(ALONE))
def test_one_layer_of_each_kind(which, dtype):
    cfg = one_layer(ALONE[which], width=48 if "64" in which or "96" in which else 40)
    typed, tensors = make_model(cfg, seed=1, calm_router=dtype == "bfloat16")
    requests = {f"r{i}": random_tokens(cfg["vocab"], n, i) for i, n in enumerate([37, 1, 2, 70])}
    run_regimes(cfg, typed, tensors, dtype, 4 if "narrow" in which or "any" in which else 16, requests,
                {"whole": whole(requests), "decoded": tail_decoded(requests, tail=5), "token by token": tail_decoded(requests, tail=1000),
                 "portions": portions(requests, (2, 3, 30)), "mixed": mixed(requests, live=3, prefill_sizes=(3, 2, 9))})


# ---- whole models in every regime -----------------------------------------------------------------------------------

@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("which", list(CONFIGS))
def test_replay_regimes(which, dtype):
    cfg = CONFIGS[which]
    typed, tensors = make_model(cfg, seed=3, calm_router=dtype == "bfloat16")
    lengths = [1, 2, 23, 70, 131, 40, 17]          # more requests than slots: slots and pages are used again
    requests = {f"r{i}": random_tokens(cfg["vocab"], n, 10 + i) for i, n in enumerate(lengths)}
    run_regimes(cfg, typed, tensors, dtype, PAGE_SIZE[which], requests,
                {"whole": whole(requests), "decoded": tail_decoded(requests, tail=32), "portions": portions(requests),
                 "portions of two and three": portions(requests, (2, 3)), "mixed": mixed(requests, live=4),
                 "mixed, two live": mixed(requests, live=2, prefill_sizes=(2, 31, 4))})


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_batch_of_unequal_requests_equals_each_alone(dtype):
    cfg = CONFIGS["odd"]
    typed, tensors = make_model(cfg, seed=5, calm_router=dtype == "bfloat16")
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

def scaled(t, name, factor):
    t[name] = (t[name].double() * factor).to(torch.bfloat16)


def marked_model(kind, shape, mark=7, width=48, vocab=50):
    """One layer in which the key of token `mark` stands out for every query, wherever it stands.  The mixer's input
    holds a one at feature 0 (the norm's weight there is 0, its bias 1) and the queries read nothing else, so every
    query is the same vector.  In a latent layer it is, for each head, the marked token's unrotated key scaled so
    that its score is `loudness`, with nothing in the rotated part.  In an attention layer the last feature of a head,
    which no rotation touches, reads what only the marked token's row of the token table has."""
    loudness = shape.get("loudness", 14.0)
    if kind == "latent":
        cfg = one_layer(latent(shape["heads"], shape["dim"], shape["rot"], shape["vdim"], shape["rank"], shape["q_rank"], 1.0), width=width, vocab=vocab)
    else:
        cfg = one_layer(attention(shape["heads"], shape["kv_heads"], shape["dim"], shape["vdim"], 1.0, rot_dims=shape["rot_dims"]), width=width, vocab=vocab)

    def change(t):
        d = lambda n: t[n].double()
        t["l0.norm1.b"][0], t["l0.norm1"][0] = 1.0, 0.0
        H, dim = shape["heads"], shape["dim"]
        if kind == "latent":
            h = plain_layernorm(d("embed")[mark], d("l0.norm1"), d("l0.norm1.b"), 1e-5)
            r, rank = shape["rot"], shape["rank"]
            c = (d("l0.mix.dkv") @ h)[:rank]
            c = plain_rmsnorm(c, d("l0.mix.dkv.norm"), 1e-5).to(torch.bfloat16).double()
            key = (d("l0.mix.uk") @ c).view(H, dim)
            wdq = torch.zeros(shape["q_rank"], width, dtype=torch.float64)
            wdq[:, 0] = 1.0                                   # the queries' latent vector is the same for every token
            t["l0.mix.dq"] = wdq.to(torch.bfloat16)
            cq = plain_rmsnorm(torch.ones(shape["q_rank"], dtype=torch.float64), d("l0.mix.dq.norm"), 1e-5)
            target = torch.zeros(H, dim + r, dtype=torch.float64)
            target[:, :dim] = loudness * key / (key * key).sum(-1, keepdim=True)
            t["l0.mix.uq"] = (target.reshape(-1, 1) * cq[None, :] / (cq * cq).sum()).to(torch.bfloat16)
            t["l0.mix.sink"] = torch.full_like(t["l0.mix.sink"], -2.0)
            scaled(t, "l0.mix.uv", 8.0)
        else:
            G = shape["kv_heads"]
            assert shape["rot_dims"] < dim
            # (features 1 and 2 of the token table are zero but for the marked token's feature 1; the layer norm takes the
            # same mean off both, so their difference is nothing for every other token, also after rounding)
            t["embed"][:, 1:3] = 0.0
            t["embed"][mark, 1] = 8.0
            t["l0.norm1"][1:3], t["l0.norm1.b"][1:3] = 1.0, 0.0
            wk = d("l0.mix.k")
            for g in range(G):
                wk[g * dim + dim - 1] = 0.0
                wk[g * dim + dim - 1, 1], wk[g * dim + dim - 1, 2] = 30.0, -30.0
            t["l0.mix.k"] = wk.to(torch.bfloat16)
            wq = torch.zeros(H * dim, width, dtype=torch.float64)
            wq[dim - 1::dim, 0] = 1.0
            t["l0.mix.q"] = wq.to(torch.bfloat16)
            h = plain_layernorm(d("embed")[mark], d("l0.norm1"), d("l0.norm1.b"), 1e-5)
            key = plain_rmsnorm(d("l0.mix.k") @ h, d("l0.mix.k.norm"), 1e-5).view(G, dim)
            q = plain_rmsnorm(wq[:, 0], None, 1e-5).view(H, dim)       # before its weight
            nw = torch.zeros(H * dim, dtype=torch.float64)
            nw[dim - 1::dim] = loudness / (float(q[0, dim - 1]) * float(key[:, dim - 1].mean()))
            t["l0.mix.q.norm"] = nw.to(torch.bfloat16)
            scaled(t, "l0.mix.v", 64.0)
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


MARKED = {"latent, any sizes": ("latent", dict(heads=3, dim=10, rot=2, vdim=6, rank=12, q_rank=5, loudness=40.0)),
          "latent, a vector of 56 and 8": ("latent", dict(heads=4, dim=16, rot=8, vdim=16, rank=56, q_rank=20)),
          "latent, a vector of 96 and 32": ("latent", dict(heads=4, dim=32, rot=32, vdim=24, rank=96, q_rank=64)),
          "latent, a vector of 192 and 64": ("latent", dict(heads=2, dim=64, rot=64, vdim=32, rank=192, q_rank=16)),
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
@pytest.mark.parametrize("rank,rot,heads", [(10, 2, 3), (56, 8, 4), (96, 32, 8), (192, 64, 4)])
def test_a_sink_that_outweighs_the_keys(rank, rot, heads, dtype):
    """Sinks of +5 (first head: nearly all of the weight), -5 (hardly any) and between: left out, counted twice, scaled
    or given to the wrong head, each moves the logits by far more than rounding does."""
    cfg = one_layer(latent(heads, 16, rot, 16, rank, 24, 0.25), width=48)

    def change(t):
        t["l0.mix.sink"] = torch.linspace(5.0, -5.0, heads).to(torch.bfloat16)
        scaled(t, "l0.mix.uv", 8.0)
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
def test_values_that_are_mostly_the_first_layers(dtype):
    """Three mixing layers whose lambdas are 0.9, -0.5 and 0.6 (the first layer's is not used): values taken from the
    wrong layer, from the layer before instead of the first, or mixed with the first layer's own lambda move the logits
    by far more than rounding does."""
    cfg = config(40, 61, [attention(4, 2, 8, 6, 0.4, rot_dims=8, v_mix=True), mlstm(2, 4, 4), attention(2, 2, 16, 6, 0.3, rot_dims=4, v_mix=True),
                          attention(4, 1, 8, 12, 0.3, v_mix=False), attention(2, 2, 8, 6, 0.5, rot_dims=None, v_mix=True, mlp=dense(20))])

    def change(t):
        for layer, lam in ((0, 0.9), (2, -0.5), (4, 0.6)):
            t[f"l{layer}.mix.vmix"] = torch.tensor(lam, dtype=torch.bfloat16)
            scaled(t, f"l{layer}.mix.v", 16.0)
    typed, tensors = make_model(cfg, seed=19, change=change)
    requests = {"a": random_tokens(61, 75, 1), "b": random_tokens(61, 2, 2), "c": random_tokens(61, 20, 3)}
    exact = reference(cfg, tensors, requests)
    other = dict(tensors)
    other["l0.mix.vmix"] = torch.tensor(0.0, dtype=torch.bfloat16)
    assert torch.equal(reference(cfg, other, requests)["a"], exact["a"])          # the first layer's own lambda is not used
    for layer in (2, 4):
        other = dict(tensors)
        other[f"l{layer}.mix.vmix"] = torch.tensor(0.0, dtype=torch.bfloat16)
        assert float((reference(cfg, other, requests)["a"] - exact["a"]).abs().max()) / float(exact["a"].abs().max()) > 0.05
    allowed = allowed_error(dtype, cfg, tensors, requests, exact)
    assert allowed < 0.03
    run_regimes(cfg, typed, tensors, dtype, 4, requests,
                {"whole": whole(requests), "decoded": tail_decoded(requests, tail=9), "portions": portions(requests, (2, 7, 3)),
                 "mixed": mixed(requests, live=3, prefill_sizes=(3, 2, 9))}, allowed)


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_memory_that_keeps_its_first_token(dtype):
    """Forget gates near one, and an input gate that only a marked token opens (its row of the token table alone has the
    feature the gate reads): 300 tokens after the marked one the read-out is still what it wrote, in every regime, also
    when the request's slot was another request's before.  Then the same memory with gates whose logarithms are all
    small, where the running maximum stays where it started."""
    cfg = one_layer(mlstm(2, 8, 8, cap=8.0), width=32, vocab=40)

    def marked(t):
        t["embed"][:, 1] = 0.0
        t["embed"][7, 1] = 8.0
        t["l0.norm1"][1], t["l0.norm1.b"][1] = 1.0, 0.0
        wi = torch.zeros_like(t["l0.mix.i"])
        wi[:, 1] = 3.0
        t["l0.mix.i"] = wi
        t["l0.mix.i.b"] = torch.full_like(t["l0.mix.i.b"], -6.0)
        t["l0.mix.f.b"] = torch.full_like(t["l0.mix.f.b"], 8.0)
        scaled(t, "l0.mix.f", 0.2)

    def small(t):
        t["l0.mix.i.b"] = torch.full_like(t["l0.mix.i.b"], -7.5)
        t["l0.mix.f.b"] = torch.full_like(t["l0.mix.f.b"], -1.0)
        scaled(t, "l0.mix.i", 0.2)
        scaled(t, "l0.mix.f", 0.2)
    for change in (marked, small):
        typed, tensors = make_model(cfg, seed=23, change=change)
        requests = {"a": sequence_with_mark(40, 300, 0, 7, 1), "b": random_tokens(40, 1, 2), "c": sequence_with_mark(40, 90, 2, 7, 3)}
        exact = reference(cfg, tensors, requests)
        if change is marked:
            assert shows(cfg, tensors, requests["a"], 0, 299) > 0.05
        run_regimes(cfg, typed, tensors, dtype, 16, requests,
                    {"whole": whole(requests), "decoded": tail_decoded(requests, tail=40), "token by token": tail_decoded(requests, tail=1000),
                     "portions": portions(requests, (2, 70, 3, 64)), "mixed": mixed(requests, live=3, prefill_sizes=(40, 2, 7))})


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_slot_used_again_starts_from_nothing(dtype):
    cfg = CONFIGS["plain"]
    typed, tensors = make_model(cfg, seed=4, calm_router=dtype == "bfloat16")
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
    typed, tensors = make_model(cfg, seed=6, calm_router=dtype == "bfloat16")
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
    cfg = config(64, 40, [attention(2, 1, 32, 32, 0.2, rot_dims=16, v_mix=True, mlp=moe(4, 2, 24, shared=(8, 1.0))),
                          latent(4, 8, 8, 12, 56, 20, 0.3, scaling=BENT, mlp=dense(16)), mlstm(2, 16, 16, mlp=dense(24)),
                          attention(2, 1, 32, 32, 0.2, rot_dims=32, v_mix=True)])
    typed, tensors = make_model(cfg, seed=12, calm_router=dtype == "bfloat16")
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
    mixed_shape = None
    for _ in range(r.randint(2, 6)):
        mlp = r.choice([None, dense(8 * r.randint(2, 12), r.choice([0.5, 1.0, 7.0])), dense(r.randint(5, 70)),
                        moe(r.randint(2, 9), 1, r.randint(3, 40), shared=None), moe(r.choice([4, 8, 12]), r.randint(2, 4), 8 * r.randint(1, 6),
                                                                                 limit=r.choice([0.5, 1.5]), scale=r.uniform(0.5, 3.0), shared=(r.randint(4, 40), 1.0))])
        kind = r.choice(["mlstm", "latent", "attention"])
        if kind == "mlstm":
            layers.append(mlstm(r.choice([1, 2, 3, 4]), r.choice([4, 12, 32, 48, 64, 100]), r.choice([4, 12, 32, 63, 64]), cap=r.choice([2.0, 15.0, 40.0]), mlp=mlp))
        elif kind == "latent":
            rot = r.choice([2, 4, 8, 16, 32, 64])
            layers.append(latent(r.choice([1, 2, 3, 4, 8, 12]), r.choice([4, 8, 20, 32, 64]), rot, r.choice([4, 12, 32, 64]),
                                 r.choice([8, 20, 32, 64, 96, 128, 192]) - r.choice([0, 0, rot % 8]), r.choice([6, 24, 64, 100]), r.uniform(0.05, 0.5),
                                 base=r.choice([100.0, 10000.0, 500000.0]), scaling=r.choice([None, BENT, {"factor": 6.0, "original": 256, "fast": 16.0, "slow": 0.5}]), mlp=mlp))
        else:
            kv = r.choice([1, 2, 3])
            dim = r.choice([8, 20, 32, 64, 128])
            vdim = r.choice([dim, dim, 4 * r.randint(1, 10)])
            v_mix = r.random() < 0.6
            if v_mix and mixed_shape is None:
                mixed_shape = (kv, vdim)
            elif v_mix:
                kv, vdim = mixed_shape
            layers.append(attention(kv * r.choice([1, 2, 4]), kv, dim, vdim, r.uniform(0.05, 0.5), rot_dims=r.choice([None, 0, dim // 2 // 2 * 2, dim]),
                                    base=r.choice([100.0, 10000.0, 1000000.0]), v_mix=v_mix, mlp=mlp))
    return config(width, r.randint(30, 200), layers, eps=r.choice([1e-5, 1e-6, 1e-3]))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("seed", range(10))
def test_configurations_drawn_at_random(seed, dtype):
    cfg = random_configuration(seed)
    typed, tensors = make_model(cfg, seed=seed, calm_router=dtype == "bfloat16")
    requests = {f"r{i}": random_tokens(cfg["vocab"], n, 70 + i) for i, n in enumerate([150, 3, 66, 1, 35])}
    run_regimes(cfg, typed, tensors, dtype, 16, requests,
                {"whole": whole(requests), "decoded": tail_decoded(requests, tail=36), "portions": portions(requests, (2, 70, 3, 33)),
                 "mixed": mixed(requests, live=3)})


# ---- generation through the scheduler --------------------------------------------------------------------------------

def plain_greedy(cfg, tensors, prompt, n):
    toks, margins = list(prompt), []
    for _ in range(n):
        row = plain_gokosun_logits(cfg, tensors, toks)[-1]
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
    folder = make_folder(tmp_path, cfg, seed=11, calm_router=True)
    typed, tensors = make_model(cfg, seed=11, calm_router=True)
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
