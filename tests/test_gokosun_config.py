"""The Gokosun configuration, what the model asks of weights and cache, the plain decoder's own invariants, and the
engine's host logic on the emulated kernels (CPU)."""
from __future__ import annotations

import copy
import math

import pytest
import torch

from emulated_kernels import EmulatedKernels
from gokosun_cases import BENT, CONFIGS, attention, check_rows, config, dense, latent, make_folder, make_model, mlstm, moe, one_layer, reference
from llm_rs_amd import ConfigError, Engine, FixedState, GokosunConfig, Model, PagedKV, config_from_dict, load_config, use_kernels
from llm_rs_amd.engine.trace import TraceReplayer
from llm_rs_amd.parts.rope import rope_gain, rope_inv_freq
from plain_gokosun import (plain_attention, plain_clamped_glu, plain_experts, plain_frequencies, plain_gokosun_logits, plain_latent_attention,
                           plain_layernorm, plain_mlstm, plain_mlstm_gates, plain_mlstm_head, plain_rotate, plain_route, plain_softmax_rows)
from replay_cases import collect, live_token_need, mixed, portions, random_tokens, tail_decoded, whole


def test_the_registry_finds_the_architecture():
    cfg = config_from_dict(CONFIGS["odd"])
    assert isinstance(cfg, GokosunConfig) and cfg.to_dict() == CONFIGS["odd"]


@pytest.mark.parametrize("path", [("vocab",), ("width",), ("norm", "eps"), ("layers", 0, "type"), ("layers", 0, "mixer", "vdim"),
                                  ("layers", 0, "mixer", "scale"), ("layers", 0, "mixer", "rot", "base"), ("layers", 0, "mixer", "rot", "dims"),
                                  ("layers", 1, "mixer", "gate_cap"), ("layers", 2, "mixer", "kv_rank"), ("layers", 2, "mixer", "q_rank"),
                                  ("layers", 2, "mixer", "rot_dim"), ("layers", 2, "mixer", "rot"), ("layers", 2, "mixer", "rot", "scaling", "fast"),
                                  ("layers", 1, "mlp", "ff"), ("layers", 1, "mlp", "limit"), ("layers", 0, "mlp", "router", "top"),
                                  ("layers", 0, "mlp", "router", "scale"), ("layers", 0, "mlp", "expert", "limit"),
                                  ("layers", 0, "mlp", "shared", "ff")])
def test_a_missing_key_is_named(path):
    d = copy.deepcopy(CONFIGS["odd"])
    at = d
    for key in path[:-1]:
        at = at[key]
    del at[path[-1]]
    with pytest.raises(ConfigError, match=str(path[-1])):
        GokosunConfig.from_dict(d).model_spec()


def test_what_a_file_may_leave_out():
    d = copy.deepcopy(CONFIGS["plain"])
    del d["layers"][2]["mixer"]["kv_heads"], d["layers"][3]["mixer"]["rot"], d["layers"][3]["mixer"]["v_mix"], d["layers"][2]["mlp"]["shared"]
    spec = GokosunConfig.from_dict(d).model_spec()
    assert spec.layers[2].mixer.params["num_kv_heads"] == 4
    assert spec.layers[3].mixer.params["position"] is None and spec.layers[3].mixer.params["value_mix"] is None
    assert spec.layers[2].mixer.params["value_mix"] == "first" and spec.layers[2].feed_forward.params["shared"] is None
    assert spec.ignorable_tensors == ("l3.mix.vmix",)


def test_what_does_not_fit_is_refused():
    for change in (lambda d: d["layers"][0].update(type="lightning"), lambda d: d["layers"][0]["mixer"].update(kv_heads=4),
                   lambda d: d["layers"][1]["mlp"].update(kind="sparse"), lambda d: d["layers"][0]["mixer"]["rot"].update(dims=7),
                   lambda d: d["layers"][0]["mixer"]["rot"].update(dims=12), lambda d: d["layers"][2]["mixer"].update(kv_rank=0),
                   lambda d: d["layers"][2]["mixer"]["rot"].update(dims=4), lambda d: d["layers"][1]["mixer"].update(gate_cap=0.0),
                   lambda d: d["layers"][0]["mlp"]["router"].update(top=6), lambda d: d["layers"][1]["mlp"].update(limit=0.0),
                   lambda d: d["layers"][4]["mixer"].update(vdim=7), lambda d: d["norm"].update(eps=0.0)):
        d = copy.deepcopy(CONFIGS["odd"])
        change(d)
        with pytest.raises(ConfigError):
            GokosunConfig.from_dict(d).model_spec()


def test_who_gives_its_values_and_who_takes_them():
    spec = GokosunConfig.from_dict(CONFIGS["odd"]).model_spec()
    assert [layer.mixer.params.get("value_mix") for layer in spec.layers] == ["first", None, None, None, "later", None]
    assert spec.ignorable_tensors == ("l3.mix.vmix",)
    assert all(layer.block == "parallel" and layer.feed_forward_norm is None for layer in spec.layers)
    assert spec.layers[3].feed_forward is None and [r.layer for r in spec.schedule] == list(range(6))


def test_tensors_and_cache_needs():
    typed, tensors = make_model(CONFIGS["odd"], seed=1)
    model = Model(typed.model_spec(), torch.float32, "cpu")
    want = model.tensors()
    assert set(want) == set(tensors)
    assert want["l0.mix.q.norm"].shape == (60,) and want["l0.mix.k.norm"].shape == (20,) and want["l0.mix.vmix"].shape == ()
    assert want["l2.mix.dq"].shape == (11, 46) and want["l2.mix.uq"].shape == (21, 11) and want["l2.mix.dkv"].shape == (11, 46)
    assert want["l2.mix.uk"].shape == (15, 9) and want["l2.mix.sink"].shape == (3,) and want["l1.mix.i.b"].shape == (3,)
    assert want["l0.mlp.e4.gate"].shape == (7, 46) and want["l0.mlp.correction"].shape == (5,) and want["l0.mlp.shared.down"].shape == (46, 9)
    assert "l3.mix.vmix" not in want and "l4.mlp.shared.gate" not in want and want["final.norm.b"].shape == (46,)
    needs = [need for need, _ in model.cache_needs()]
    assert needs[0] == PagedKV(2, 10, 0, 6, 0)
    assert needs[1] == FixedState((3 * (7 + 1) * 5 + 4,), torch.float32)         # S with n as one more column, then room for the maxima
    assert needs[2] == PagedKV(1, 9 + 2)                                          # the latent vector and the rotated key part
    assert needs[5] == FixedState((1 * (4 + 1) * 13 + 4,), torch.float32)


def test_weights_come_back_as_the_file_had_them():
    for which in ("odd", "plain"):
        typed, tensors = make_model(CONFIGS[which], seed=2)
        model = Model(typed.model_spec(), torch.float32, "cpu")
        model.load(tensors)
        back = model.weights()
        assert set(back) == set(tensors)
        for name, t in tensors.items():
            assert torch.equal(back[name].float().reshape(t.shape), t.float()), name


def test_a_folder_is_read_by_its_architecture(tmp_path):
    folder = make_folder(tmp_path, CONFIGS["plain"], seed=3)
    assert isinstance(load_config(folder), GokosunConfig)


# ---- the plain decoder's mechanisms, worked out by hand ------------------------------------------------------------------

def test_plain_layer_norm_takes_the_mean_off_and_divides_by_the_deviation():
    x = torch.tensor([[1.0, 3.0, 5.0, 7.0]], dtype=torch.float64)
    y = plain_layernorm(x, torch.tensor([1.0, 1.0, 2.0, 1.0], dtype=torch.float64), torch.tensor([0.0, 0.5, 0.0, 0.0], dtype=torch.float64), 1e-12)
    s = math.sqrt(5.0)          # the mean of the squared deviations 9, 1, 1, 9
    assert torch.allclose(y, torch.tensor([[-3 / s, -1 / s + 0.5, 2 / s, 3 / s]], dtype=torch.float64), atol=1e-9)
    assert torch.allclose(plain_layernorm(x + 100.0, torch.ones(4).double(), torch.zeros(4).double(), 1e-12),
                          plain_layernorm(x, torch.ones(4).double(), torch.zeros(4).double(), 1e-12))


def test_plain_rotation_pairs():
    x = torch.arange(1.0, 9.0, dtype=torch.float64).view(1, 1, 8)
    freq = torch.tensor([math.pi / 2, math.pi], dtype=torch.float64)           # at position 1: a quarter turn, a half turn
    half = plain_rotate(x, [1], freq, 1.0, "half")[0, 0]
    assert torch.allclose(half, torch.tensor([-3.0, -2.0, 1.0, -4.0, 5.0, 6.0, 7.0, 8.0], dtype=torch.float64), atol=1e-9)
    pairs = plain_rotate(x, [1], freq, 2.0, "pairs")[0, 0]
    assert torch.allclose(pairs, torch.tensor([-4.0, 2.0, -6.0, -8.0, 5.0, 6.0, 7.0, 8.0], dtype=torch.float64), atol=1e-9)
    assert torch.equal(plain_rotate(x, [0], freq, 1.0, "half"), x)


def test_bent_frequencies_and_the_engines_table_agree():
    for dims, base, sc in ((6, 100.0, BENT), (16, 500000.0, {"factor": 2.0, "original": 2048, "fast": 32.0, "slow": 1.0}), (8, 10000.0, None)):
        freq, gain = plain_frequencies({"dims": dims, "base": base, "scaling": sc})
        scaling = None if sc is None else {"rope_type": "ramp", **sc}
        assert torch.allclose(rope_inv_freq(dims, base, scaling).double(), freq, rtol=1e-6)
        assert abs(rope_gain(scaling) - gain) < 1e-12
        if sc is None:
            assert gain == 1.0 and abs(float(freq[1]) - base ** (-2.0 / dims)) < 1e-12
    freq, gain = plain_frequencies({"dims": 6, "base": 100.0, "scaling": BENT})
    assert abs(gain - (0.1 * math.log(4.0) + 1.0)) < 1e-12
    assert abs(float(freq[0]) - 1.0) < 1e-12 and abs(float(freq[2]) - 100.0 ** (-4.0 / 6.0) / 4.0) < 1e-12      # the fastest kept, the slowest divided


def test_plain_sink_only_enlarges_the_denominator():
    s = torch.tensor([[[0.0, float("-inf")], [1.0, 2.0]]], dtype=torch.float64)
    p = plain_softmax_rows(s, torch.tensor([0.0], dtype=torch.float64))
    assert torch.allclose(p[0, 0], torch.tensor([0.5, 0.0], dtype=torch.float64))
    e1, e2 = math.e, math.e ** 2
    assert torch.allclose(p[0, 1], torch.tensor([e1 / (1 + e1 + e2), e2 / (1 + e1 + e2)], dtype=torch.float64))
    assert torch.allclose(plain_softmax_rows(s)[0, 1].sum(), torch.tensor(1.0, dtype=torch.float64))


def test_plain_matrix_memory_by_hand():
    """Two tokens of one head with one key channel and one value channel: the numbers of the recurrence written out."""
    q, k, v = torch.tensor([[1.0], [2.0]], dtype=torch.float64), torch.tensor([[3.0], [0.5]], dtype=torch.float64), torch.tensor([[2.0], [4.0]], dtype=torch.float64)
    i, f = torch.tensor([1.0, -3.0], dtype=torch.float64), torch.tensor([-0.5, -0.1], dtype=torch.float64)
    out, (S, n, m) = plain_mlstm_head(q, k, v, i, f)
    # token 0: m = max(-0.5 + 0, 1) = 1; S = exp(-1.5) 0 + exp(0) 3 * 2 = 6; n = 3; o = 6 / (max(3, exp(-1)) + 1e-6)
    assert abs(float(out[0, 0]) - 6.0 / (3.0 + 1e-6)) < 1e-12
    # token 1: m = max(-0.1 + 1, -3) = 0.9; keep = exp(-0.1 + 1 - 0.9) = 1; take = exp(-3.9); S = 6 + take 2; n = 3 + take 0.5
    take = math.exp(-3.9)
    assert abs(float(m) - 0.9) < 1e-12 and abs(float(S[0, 0]) - (6.0 + 2.0 * take)) < 1e-12 and abs(float(n[0]) - (3.0 + 0.5 * take)) < 1e-12
    assert abs(float(out[1, 0]) - 2.0 * (6.0 + 2.0 * take) / (2.0 * (3.0 + 0.5 * take) + 1e-6)) < 1e-12
    # the maximum starts at zero, not at minus infinity: a first token with small gates is weighed by exp(i), not by 1
    out, (S, n, m) = plain_mlstm_head(q[:1], k[:1], v[:1], torch.tensor([-5.0], dtype=torch.float64), torch.tensor([-2.0], dtype=torch.float64))
    assert float(m) == -2.0 and abs(float(S[0, 0]) - 6.0 * math.exp(-3.0)) < 1e-12
    assert abs(float(out[0, 0]) - 6.0 * math.exp(-3.0) / (math.exp(2.0) + 1e-6)) < 1e-12          # the floor exp(-m) is the larger
    # a state handed on continues exactly
    whole, _ = plain_mlstm_head(q, k, v, i, f)
    first, state = plain_mlstm_head(q[:1], k[:1], v[:1], i[:1], f[:1])
    second, _ = plain_mlstm_head(q[1:], k[1:], v[1:], i[1:], f[1:], state)
    assert torch.equal(torch.cat([first, second]), whole)


def test_plain_gates_are_bent_into_the_cap():
    h = torch.tensor([[100.0], [-100.0], [0.0]], dtype=torch.float64)
    w = {"i": torch.ones(2, 1).double(), "i.b": torch.tensor([0.0, 1.0], dtype=torch.float64), "f": torch.ones(2, 1).double(), "f.b": torch.zeros(2).double()}
    i, f = plain_mlstm_gates(h, w, 4.0)
    assert abs(float(i[0, 0]) - 4.0) < 1e-9 and abs(float(i[1, 0]) + 4.0) < 1e-9 and abs(float(i[2, 1]) - 4.0 * math.tanh(0.25)) < 1e-12
    assert abs(float(f[0, 0]) + math.log1p(math.exp(-4.0))) < 1e-9 and abs(float(f[1, 0]) + 4.0 + math.log1p(math.exp(-4.0))) < 1e-9
    assert abs(float(f[2, 0]) + math.log(2.0)) < 1e-12


def test_plain_activation_clamps_before_it_gates():
    w = {"gate": torch.tensor([[1.0], [1.0]], dtype=torch.float64), "up": torch.tensor([[1.0], [-1.0]], dtype=torch.float64), "down": torch.eye(2).double()}
    y = plain_clamped_glu(torch.tensor([[5.0]], dtype=torch.float64), w, 2.0)
    sig = 1.0 / (1.0 + math.exp(-1.702 * 2.0))
    assert torch.allclose(y, torch.tensor([[2.0 * sig * 3.0, 2.0 * sig * -1.0]], dtype=torch.float64), atol=1e-12)      # g = 2, u = 2 and -2
    y = plain_clamped_glu(torch.tensor([[-5.0]], dtype=torch.float64), w, 2.0)                                          # the gate has no lower limit
    sig = 1.0 / (1.0 + math.exp(1.702 * 5.0))
    assert torch.allclose(y, torch.tensor([[-5.0 * sig * -1.0, -5.0 * sig * 3.0]], dtype=torch.float64), atol=1e-12)


def test_plain_router_chooses_with_the_correction_and_weighs_without_it():
    w = {"router": torch.tensor([[2.0], [1.0], [0.0], [-1.0]], dtype=torch.float64), "correction": torch.tensor([-1.0, 0.0, 0.0, 1.0], dtype=torch.float64)}
    chosen, weights = plain_route(torch.tensor([[1.0]], dtype=torch.float64), w, 2, 3.0)
    s = [1.0 / (1.0 + math.exp(-z)) for z in (2.0, 1.0, 0.0, -1.0)]
    assert sorted(chosen[0].tolist()) == [1, 3]                  # scores 0.88, 0.73, 0.5, 0.27 become -0.12, 0.73, 0.5, 1.27
    got = dict(zip(chosen[0].tolist(), weights[0].tolist()))
    assert abs(got[1] - 3.0 * s[1] / (s[1] + s[3])) < 1e-12 and abs(got[3] - 3.0 * s[3] / (s[1] + s[3])) < 1e-12


def test_plain_experts_of_one_are_the_expert_itself_beside_the_shared_one():
    cfg = one_layer(mlstm(1, 2, 2, mlp=moe(1, 1, 3, scale=1.0, shared=(2, 1.0))), width=6, vocab=9)
    _, tensors = make_model(cfg, seed=4)
    w = {n[len("l0.mlp."):]: t.double() for n, t in tensors.items() if n.startswith("l0.mlp.")}
    h = torch.randn(5, 6, dtype=torch.float64, generator=torch.Generator().manual_seed(1))
    one = plain_clamped_glu(h, {k[3:]: v for k, v in w.items() if k.startswith("e0.")}, 1.5)
    shared = plain_clamped_glu(h, {k[7:]: v for k, v in w.items() if k.startswith("shared.")}, 1.0)
    assert torch.allclose(plain_experts(h, w, cfg["layers"][0]["mlp"]), one + shared, atol=1e-12)


def test_plain_latent_attention_of_one_token_is_its_value_under_the_sink():
    cfg = one_layer(latent(2, 4, 2, 3, 5, 6, 0.5, scaling=BENT), width=8, vocab=9)
    _, tensors = make_model(cfg, seed=5)
    w = {n[len("l0.mix."):]: t.double() for n, t in tensors.items() if n.startswith("l0.mix.")}
    m = cfg["layers"][0]["mixer"]
    h = torch.randn(1, 8, dtype=torch.float64, generator=torch.Generator().manual_seed(2))
    cq = h @ w["dq"].T
    cq = cq / torch.sqrt((cq * cq).mean() + 1e-5) * w["dq.norm"]
    q = (cq @ w["uq"].T).view(2, 6)
    low = (h @ w["dkv"].T)[0]
    c = low[:5] / torch.sqrt((low[:5] * low[:5]).mean() + 1e-5) * w["dkv.norm"]
    gain = 0.1 * math.log(4.0) + 1.0            # at position 0 nothing turns, but cosine is still enlarged
    out = torch.zeros(2, 3, dtype=torch.float64)
    for head in range(2):
        key = w["uk"].view(2, 4, 5)[head] @ c
        score = (q[head, :4] @ key + (q[head, 4:] * gain) @ (low[5:] * gain)) * 0.5
        p = math.exp(float(score)) / (math.exp(float(score)) + math.exp(float(w["sink"][head])))
        out[head] = p * (w["uv"].view(2, 3, 5)[head] @ c)
    assert torch.allclose(plain_latent_attention(h, w, m, 1e-5), out.reshape(1, 6) @ w["o"].T, atol=1e-10)


def test_plain_attention_norms_the_whole_projection_and_mixes_values():
    cfg = config(8, 9, [attention(2, 1, 4, 3, 0.5, rot_dims=2, v_mix=True), attention(2, 1, 4, 3, 0.5, rot_dims=None, v_mix=True)])
    _, tensors = make_model(cfg, seed=6)
    w = {n[len("l1.mix."):]: t.double() for n, t in tensors.items() if n.startswith("l1.mix.")}
    m = cfg["layers"][1]["mixer"]
    h = torch.randn(1, 8, dtype=torch.float64, generator=torch.Generator().manual_seed(3))
    v_first = torch.randn(1, 1, 3, dtype=torch.float64, generator=torch.Generator().manual_seed(4))
    out, v = plain_attention(h, w, m, 1e-5, v_first)
    lam = float(w["vmix"])
    mixed = (1.0 - lam) * (h @ w["v"].T).view(1, 1, 3) + lam * v_first
    assert torch.allclose(v, mixed, atol=1e-12)
    assert torch.allclose(out, mixed[0, 0].repeat(2).view(1, 6) @ w["o"].T, atol=1e-12)          # one token sees itself alone
    alone, v_alone = plain_attention(h, w, m, 1e-5, None)                                        # the first such layer mixes nothing
    assert torch.allclose(v_alone, (h @ w["v"].T).view(1, 1, 3), atol=1e-12)
    # the norm runs over all heads at once: a second head ten times as loud takes the first head's share
    q = h @ w["q"].T
    assert not torch.allclose((q / torch.sqrt((q * q).mean() + 1e-5)).view(2, 4)[0],
                              q.view(2, 4)[0] / torch.sqrt((q.view(2, 4)[0] ** 2).mean() + 1e-5))


def test_the_stream_takes_both_halves_of_a_layer_from_one_norm():
    cfg = CONFIGS["odd"]
    _, tensors = make_model(cfg, seed=7)
    seen = []
    logits = plain_gokosun_logits(cfg, tensors, [3, 1, 4, 1, 5], after_layer=lambda i, x: seen.append(x.clone()))
    assert len(seen) == 6 and logits.shape == (5, 97)
    x0 = tensors["embed"].double()[torch.tensor([3, 1, 4, 1, 5])]
    n = plain_layernorm(x0, tensors["l0.norm1"].double(), tensors["l0.norm1.b"].double(), 1e-5)
    w = {k[len("l0.mix."):]: t.double() for k, t in tensors.items() if k.startswith("l0.mix.")}
    ff = {k[len("l0.mlp."):]: t.double() for k, t in tensors.items() if k.startswith("l0.mlp.")}
    mix, _ = plain_attention(n, w, cfg["layers"][0]["mixer"], 1e-5, None)
    assert torch.allclose(seen[0], x0 + (mix + plain_experts(n, ff, cfg["layers"][0]["mlp"])), atol=1e-12)


# ---- the engine's host logic on the emulated kernels ---------------------------------------------------------------

def replay_cpu(typed, tensors, dtype, page_size, steps, max_requests=4):
    with use_kernels(EmulatedKernels()):
        eng = Engine(typed, tensors, dtype=dtype, device="cpu", page_size=page_size, num_pages=max(-(-live_token_need(steps, 64) // page_size), 1),
                     max_requests=max_requests)
        rep = TraceReplayer.for_engine(eng)
        outputs = []
        for step in steps:
            out = rep.step(step)
            outputs.append(None if out is None else torch.from_numpy(out.copy()))
        core = eng.cache.core
        assert core.slots_in_use() == 0 and all(core.pages_free(g) == core.pages_total(g) for g in range(core.n_groups))
    return collect(steps, outputs)


@pytest.mark.parametrize("which", ["odd", "plain"])
def test_replay_regimes_on_the_host_logic(which):
    cfg = CONFIGS[which]
    typed, tensors = make_model(cfg, seed=3)
    lengths = [1, 2, 23, 50, 40, 17]            # more requests than slots: slots and pages are used again
    requests = {f"r{i}": random_tokens(cfg["vocab"], n, 10 + i) for i, n in enumerate(lengths)}
    exact = reference(cfg, tensors, requests)
    for name, steps in {"whole": whole(requests), "decoded": tail_decoded(requests, tail=12), "portions": portions(requests, (2, 3, 7)),
                        "mixed": mixed(requests, live=3)}.items():
        check_rows(replay_cpu(typed, tensors, "float32", {"odd": 4, "plain": 16}[which], steps), exact, requests, 3e-5, name)


def test_a_layer_of_each_kind_alone_on_the_host_logic():
    for layer in (attention(3, 1, 8, 5, 0.4, rot_dims=4, base=50.0, v_mix=True, mlp=dense(12)), latent(5, 4, 6, 6, 7, 3, 0.3, scaling=BENT),
                  mlstm(2, 6, 3, cap=5.0, mlp=moe(3, 2, 4, shared=(5, 1.0))), attention(2, 2, 6, 6, 0.5, rot_dims=None)):
        cfg = one_layer(layer)
        typed, tensors = make_model(cfg, seed=5)
        requests = {"a": random_tokens(cfg["vocab"], 21, 1), "b": random_tokens(cfg["vocab"], 6, 2)}
        exact = reference(cfg, tensors, requests)
        for name, steps in {"whole": whole(requests), "portions": portions(requests, (2, 5, 3)), "mixed": mixed(requests, live=2)}.items():
            check_rows(replay_cpu(typed, tensors, "float32", 4, steps), exact, requests, 3e-5, f"{layer['type']} {name}")
