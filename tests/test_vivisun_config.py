"""The Vivisun configuration, what the model asks of weights and cache, the plain decoder's own invariants, and the
engine's host logic on the emulated kernels (CPU)."""
from __future__ import annotations

import copy
import math

import pytest
import torch

from emulated_kernels import EmulatedKernels
from llm_rs_amd import ConfigError, Engine, FixedState, Model, PagedKV, VivisunConfig, config_from_dict, load_config, use_kernels
from llm_rs_amd.engine.trace import TraceReplayer
from llm_rs_amd.parts.rope import rope_gain, rope_inv_freq
from plain_vivisun import (plain_attention, plain_bent_frequencies, plain_causal_conv, plain_dyt, plain_latent_attention,
                           plain_rotate_half, plain_schedule, plain_softmax_rows, plain_vivisun_logits)
from replay_cases import collect, live_token_need, mixed, portions, random_tokens, tail_decoded, whole
from vivisun_cases import BENT, CONFIGS, attention, check_rows, config, dense, latent, make_folder, make_model, one_layer, reference


def test_the_registry_finds_the_architecture():
    cfg = config_from_dict(CONFIGS["odd"])
    assert isinstance(cfg, VivisunConfig) and cfg.to_dict() == CONFIGS["odd"]


@pytest.mark.parametrize("path", [("vocab",), ("width",), ("norm", "eps"), ("layers", 0, "type"), ("layers", 0, "mixer", "vdim"),
                                  ("layers", 0, "mixer", "scale"), ("layers", 0, "mixer", "rot", "base"), ("layers", 0, "mixer", "rot", "dims"),
                                  ("layers", 0, "mixer", "rot", "scaling", "fast"), ("layers", 1, "mixer", "kv_rank"),
                                  ("layers", 1, "mixer", "heads"), ("layers", 0, "mlp", "ff"), ("loop", "times")])
def test_a_missing_key_is_named(path):
    d = copy.deepcopy(CONFIGS["odd"])
    at = d
    for key in path[:-1]:
        at = at[key]
    del at[path[-1]]
    with pytest.raises(ConfigError, match=str(path[-1])):
        VivisunConfig.from_dict(d).model_spec()


def test_what_a_file_may_leave_out():
    d = copy.deepcopy(CONFIGS["plain"])
    del d["layers"][1]["mixer"]["kv_heads"], d["layers"][2]["mixer"]["conv"], d["layers"][2]["mixer"]["rot"], d["loop"]
    spec = VivisunConfig.from_dict(d).model_spec()
    assert spec.layers[1].mixer.params["num_kv_heads"] == 4
    assert spec.layers[2].mixer.params["conv"] == 0 and spec.layers[2].mixer.params["position"] is None
    assert [r.layer for r in spec.schedule] == [0, 1, 2] and not any(r.add_embedding for r in spec.schedule)


def test_what_does_not_fit_is_refused():
    for change in (lambda d: d["layers"][0].update(type="lightning"), lambda d: d["layers"][0]["mixer"].update(kv_heads=4),
                   lambda d: d["layers"][1]["mlp"].update(kind="moe"), lambda d: d["layers"][0]["mixer"]["rot"].update(dims=7),
                   lambda d: d["layers"][0]["mixer"]["rot"].update(dims=12), lambda d: d["layers"][1]["mixer"].update(kv_rank=0),
                   lambda d: d["loop"].update(stop=5), lambda d: d["loop"].update(start=3, stop=2), lambda d: d["loop"].update(times=0),
                   lambda d: d["norm"].update(eps=0.0)):
        d = copy.deepcopy(CONFIGS["odd"])
        change(d)
        with pytest.raises(ConfigError):
            VivisunConfig.from_dict(d).model_spec()


@pytest.mark.parametrize("n,loop", [(4, None), (4, (1, 4, 2)), (4, (0, 4, 3)), (5, (2, 3, 4)), (3, (0, 1, 1)), (3, (1, 1, 5)), (2, (0, 2, 2))])
def test_the_order_of_runs(n, loop):
    layers = [latent(1, 4, 4, 4, 0.5) for _ in range(n)]
    spec = VivisunConfig.from_dict(config(8, 9, layers, loop)).model_spec()
    got = [(r.layer, r.add_embedding) for r in spec.schedule]
    want = plain_schedule(n, None if loop is None else {"start": loop[0], "stop": loop[1], "times": loop[2]})
    assert got == want
    if loop is not None and loop[2] > 1 and loop[1] > loop[0]:
        a, b, times = loop
        assert len(got) == n + (times - 1) * (b - a) and sum(again for _, again in got) == times - 1
        assert all(layer == a for layer, again in got if again)
    assert all(r.cache_of is None for r in spec.schedule)            # every pass has a cache of its own


def test_tensors_and_cache_needs():
    typed, tensors = make_model(CONFIGS["odd"], seed=1)
    model = Model(typed.model_spec(), torch.float32, "cpu")
    want = model.tensors()
    assert set(want) == set(tensors)
    assert want["l0.mix.q.conv"].shape == (60, 3) and want["l0.mix.g"].shape == (36, 46) and want["l0.mix.q.norm"].shape == (10,)
    assert want["l1.mix.g"].shape == (3, 46) and want["l1.mix.sink"].shape == (3,) and want["l1.mix.uk"].shape == (15, 9)
    assert want["l1.mix.uv"].shape == (21, 9) and want["l1.mix.dkv.norm"].shape == (9,) and want["final.norm.alpha"].shape == ()
    assert "l2.mlp.up" not in want and "l2.norm2" not in want            # a layer without a feed-forward reads no second norm
    needs = [need for need, _ in model.cache_needs()]
    assert len(needs) == 8
    assert needs[0] == (PagedKV(2, 10, 0, 6, 0), FixedState((2 * (60 + 20 + 12),), torch.float32))       # pages, and conv - 1 rows of q | k | v
    assert needs[1] == PagedKV(1, 9) and needs[3] == needs[1]           # only the latent vector is cached, once for all heads
    assert needs[2] == PagedKV(2, 12, 0, 20, 0)                          # one tap: nothing to remember
    assert needs[7] == PagedKV(1, 17)


def test_weights_come_back_as_the_file_had_them():
    typed, tensors = make_model(CONFIGS["odd"], seed=2)
    model = Model(typed.model_spec(), torch.float32, "cpu")
    model.load(tensors)
    back = model.weights()
    assert set(back) == set(tensors)
    for name, t in tensors.items():
        assert torch.equal(back[name].float().reshape(t.shape), t.float()), name


def test_a_folder_is_read_by_its_architecture(tmp_path):
    folder = make_folder(tmp_path, CONFIGS["plain"], seed=3)
    assert isinstance(load_config(folder), VivisunConfig)


# ---- the plain decoder's mechanisms, worked out by hand ------------------------------------------------------------------

def test_plain_dyt_sums_nothing_over_the_row():
    x = torch.tensor([[0.0, 1.0, -2.0]], dtype=torch.float64)
    y = plain_dyt(x, torch.tensor([2.0, 2.0, 2.0]).double(), torch.tensor([0.5, 0.0, 0.0]).double(), torch.tensor(0.5).double())
    assert torch.allclose(y, torch.tensor([[0.5, 2 * math.tanh(0.5), 2 * math.tanh(-1.0)]]).double())
    x2 = x.clone()
    x2[0, 2] = 100.0                                                  # another feature's value moves nothing else
    assert torch.equal(plain_dyt(x2, torch.ones(3).double(), torch.zeros(3).double(), torch.tensor(1.0).double())[0, :2],
                       plain_dyt(x, torch.ones(3).double(), torch.zeros(3).double(), torch.tensor(1.0).double())[0, :2])


def test_plain_conv_weighs_the_current_token_last_and_starts_from_zeros():
    u = torch.tensor([[1.0], [10.0], [100.0], [1000.0]], dtype=torch.float64)
    y = plain_causal_conv(u, torch.tensor([[3.0, 2.0, 1.0]], dtype=torch.float64))
    assert y.flatten().tolist() == [1.0, 12.0, 123.0, 1230.0]


def test_plain_rotation_pairs_a_feature_with_the_one_half_way_on():
    x = torch.zeros(1, 1, 6, dtype=torch.float64)
    x[0, 0, 0] = 1.0                                                  # feature 0 pairs with feature 2 when four features turn
    y = plain_rotate_half(x, [1], torch.tensor([math.pi / 2, 0.0], dtype=torch.float64), 2.0)
    assert torch.allclose(y[0, 0], torch.tensor([0.0, 0.0, 2.0, 0.0, 0.0, 0.0], dtype=torch.float64), atol=1e-12)
    x = torch.zeros(1, 1, 6, dtype=torch.float64)
    x[0, 0, 1], x[0, 0, 5] = 1.0, 7.0                                 # a zero frequency only enlarges; what is not turned passes
    y = plain_rotate_half(x, [9], torch.tensor([math.pi / 2, 0.0], dtype=torch.float64), 2.0)
    assert torch.allclose(y[0, 0], torch.tensor([0.0, 2.0, 0.0, 0.0, 0.0, 7.0], dtype=torch.float64), atol=1e-12)


def test_bent_frequencies_and_the_engines_table_agree():
    for dims, base, sc in ((6, 100.0, BENT), (32, 500.0, BENT), (24, 10000.0, {"factor": 16.0, "original": 128, "fast": 32.0, "slow": 1.0}),
                           (8, 50.0, None), (4, 10.0, {"factor": 2.0, "original": 4096, "fast": 4.0, "slow": 2.0})):
        freq, gain = plain_bent_frequencies({"dims": dims, "base": base, "scaling": sc})
        scaling = None if sc is None else {"rope_type": "ramp", **sc}
        assert torch.allclose(rope_inv_freq(dims, base, scaling).double(), freq, rtol=1e-6)
        assert abs(rope_gain(scaling) - gain) < 1e-12
        plain = torch.tensor([base ** (-2.0 * i / dims) for i in range(dims // 2)], dtype=torch.float64)
        if sc is None:
            assert gain == 1.0 and torch.equal(freq, plain)
        else:
            assert gain == 0.1 * math.log(sc["factor"]) + 1.0
            assert bool((freq <= plain * (1 + 1e-12)).all()) and bool((freq >= plain / sc["factor"] * (1 - 1e-12)).all())


def test_plain_sink_only_enlarges_the_denominator():
    s = torch.tensor([[[0.0, float("-inf")], [1.0, 2.0]]], dtype=torch.float64)
    p = plain_softmax_rows(s, torch.tensor([0.0], dtype=torch.float64))
    assert torch.allclose(p[0, 0], torch.tensor([0.5, 0.0], dtype=torch.float64))
    e1, e2 = math.exp(1.0), math.exp(2.0)
    assert torch.allclose(p[0, 1], torch.tensor([e1 / (e1 + e2 + 1.0), e2 / (e1 + e2 + 1.0)], dtype=torch.float64))
    assert torch.allclose(plain_softmax_rows(s)[0, 1].sum(), torch.tensor(1.0, dtype=torch.float64))


def test_plain_latent_attention_of_one_token_is_its_value_under_gate_and_sink():
    g = torch.Generator().manual_seed(0)
    D, H, dk, dv, R = 6, 2, 3, 4, 5
    w = {"q": torch.randn(H * dk, D, generator=g), "dkv": torch.randn(R, D, generator=g), "dkv.norm": torch.rand(R, generator=g) + 0.5,
         "uk": torch.randn(H * dk, R, generator=g), "uv": torch.randn(H * dv, R, generator=g), "sink": torch.tensor([0.3, -1.0]),
         "g": torch.randn(H, D, generator=g), "o": torch.eye(H * dv)}
    w = {k: v.double() for k, v in w.items()}
    h = torch.randn(1, D, generator=g).double()
    m = {"heads": H, "dim": dk, "vdim": dv, "kv_rank": R, "scale": 0.7}
    c = h @ w["dkv"].T
    c = c / torch.sqrt((c * c).mean() + 1e-5) * w["dkv.norm"]
    v = (c @ w["uv"].T).view(H, dv)
    s = ((h @ w["q"].T).view(H, dk) * (c @ w["uk"].T).view(H, dk)).sum(-1) * 0.7
    p = torch.exp(s) / (torch.exp(s) + torch.exp(w["sink"]))
    gate = 1.0 / (1.0 + torch.exp(-(h @ w["g"].T)))[0]
    assert torch.allclose(plain_latent_attention(h, w, m, 1e-5)[0], (v * (p * gate)[:, None]).reshape(-1), rtol=1e-10)


def test_plain_attention_of_one_token_is_its_gated_value():
    g = torch.Generator().manual_seed(1)
    D, H, G, dk, dv, K = 5, 4, 2, 6, 3, 3
    w = {"q": torch.randn(H * dk, D, generator=g), "k": torch.randn(G * dk, D, generator=g), "v": torch.randn(G * dv, D, generator=g),
         "q.conv": torch.randn(H * dk, K, generator=g), "k.conv": torch.randn(G * dk, K, generator=g), "v.conv": torch.randn(G * dv, K, generator=g),
         "q.norm": torch.ones(dk), "k.norm": torch.ones(dk), "g": torch.randn(H * dv, D, generator=g), "o": torch.eye(H * dv)}
    w = {k: v.double() for k, v in w.items()}
    h = torch.randn(1, D, generator=g).double()
    m = {"heads": H, "kv_heads": G, "dim": dk, "vdim": dv, "scale": 0.3, "conv": K, "rot": {"dims": 4, "base": 10.0, "scaling": None}}
    v = ((h @ w["v"].T)[0] * w["v.conv"][:, K - 1]).view(G, dv).repeat_interleave(H // G, dim=0).reshape(-1)       # the first token sees zeros before it
    gate = 1.0 / (1.0 + torch.exp(-(h @ w["g"].T)))[0]
    assert torch.allclose(plain_attention(h, w, m, 1e-5)[0], v * gate, rtol=1e-10)


def test_the_embeddings_come_again_before_every_further_pass():
    cfg = config(12, 20, [latent(2, 3, 3, 4, 0.5, mlp=dense(8)), latent(1, 4, 2, 3, 0.5)], loop=(0, 2, 3))
    typed, tensors = make_model(cfg, seed=4)
    seen = []
    plain_vivisun_logits(cfg, tensors, [3, 1, 4], after_run=lambda r, x: seen.append(x.clone()))
    assert len(seen) == 6
    once = copy.deepcopy(cfg)
    once["loop"] = None
    first = []
    plain_vivisun_logits(once, tensors, [3, 1, 4], after_run=lambda r, x: first.append(x.clone()))
    assert torch.equal(seen[0], first[0]) and torch.equal(seen[1], first[1])             # the first pass is the plain stack


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
    for layer in (attention(3, 1, 8, 5, 0.4, conv=5, rot_dims=4, base=50.0, scaling=BENT, mlp=dense(12)), latent(5, 4, 6, 7, 0.3),
                  attention(2, 2, 6, 6, 0.5, conv=0, rot_dims=None)):
        cfg = one_layer(layer, loop=(0, 1, 2))
        typed, tensors = make_model(cfg, seed=5)
        requests = {"a": random_tokens(cfg["vocab"], 21, 1), "b": random_tokens(cfg["vocab"], 6, 2)}
        exact = reference(cfg, tensors, requests)
        for name, steps in {"whole": whole(requests), "portions": portions(requests, (2, 5, 3)), "mixed": mixed(requests, live=2)}.items():
            check_rows(replay_cpu(typed, tensors, "float32", 4, steps), exact, requests, 3e-5, f"{layer['type']} {name}")
