"""Pigodra without a GPU: the plain implementation's mechanisms against closed forms worked
out by hand, the configuration reader, the plan, the checkpoint layout, and the cache's
bookkeeping for a window that keeps its first keys."""
import json
import math
import os

import pytest
import torch

import gpt_fast_amd as gfa
import plain_pigodra as P
from gpt_fast_amd.cache.store import KVNeed, StateNeed
from gpt_fast_amd.config.pigodra import ConfigError, PigodraConfig
from gpt_fast_amd.config.registry import architecture_of
from pigodra_cases import CASES, make_folder


# --------------------------------------------------------------------------- the plain pieces
def test_visibility_by_hand():
    see = P.visible(8, 3, 2)
    assert see[7].tolist() == [True, True, False, False, False, True, True, True]
    assert see[4].tolist() == [True, True, True, True, True, False, False, False]
    assert see[2].tolist() == [True, True, True, False, False, False, False, False]
    assert P.visible(5, None, 0)[4].all()
    assert P.visible(6, 2, 0)[5].tolist() == [False, False, False, False, True, True]


def test_norm_around_zero_and_eps_inside_the_root():
    x = torch.tensor([[3.0, -4.0]], dtype=P.F)
    got = P.rms_norm_around_zero(x, torch.tensor([0.0, 1.0], dtype=P.F), 0.5)
    r = math.sqrt(12.5 + 0.5)
    assert torch.allclose(got, torch.tensor([[3 / r, -8 / r]], dtype=P.F))


def test_gelu_tanh_values():
    z = torch.tensor([0.0, 1.0, -2.0], dtype=P.F)
    want = [0.0, 0.5 * (1 + math.tanh(math.sqrt(2 / math.pi) * 1.044715)),
            -1.0 * (1 + math.tanh(math.sqrt(2 / math.pi) * (-2 - 0.044715 * 8)))]
    assert torch.allclose(P.gelu_tanh(z), torch.tensor(want, dtype=P.F))


def test_rotation_keeps_lengths_is_relative_and_leaves_the_rest():
    torch.manual_seed(0)
    x = torch.randn(6, 2, 10, dtype=P.F)
    y = P.rotate_pairs(x, torch.arange(6), 6, 100.0, 2.0)
    assert torch.equal(y[..., 6:], x[..., 6:]) and torch.allclose(y[0], x[0])
    assert torch.allclose(y[..., :6].norm(dim=-1), x[..., :6].norm(dim=-1))
    # the dot product of two rotated rows depends on the distance only
    a, b = torch.randn(1, 1, 6, dtype=P.F), torch.randn(1, 1, 6, dtype=P.F)
    d1 = (P.rotate_pairs(a, torch.tensor([9]), 6, 100.0, 2.0) * P.rotate_pairs(b, torch.tensor([4]), 6, 100.0, 2.0)).sum()
    d2 = (P.rotate_pairs(a, torch.tensor([25]), 6, 100.0, 2.0) * P.rotate_pairs(b, torch.tensor([20]), 6, 100.0, 2.0)).sum()
    assert torch.allclose(d1, d2)
    # pair i turns by p * base^(-2i/dims) / factor: the second pair at position 3
    one = torch.zeros(1, 1, 4, dtype=P.F)
    one[0, 0, 2] = 1.0
    ang = 3 * 100.0 ** (-2 / 4) / 2.0
    got = P.rotate_pairs(one, torch.tensor([3]), 4, 100.0, 2.0)[0, 0]
    assert torch.allclose(got, torch.tensor([0, 0, math.cos(ang), math.sin(ang)], dtype=P.F))


def test_memory_cell_equals_the_sum_over_all_pairs():
    torch.manual_seed(1)
    T, H, dk, dv = 60, 3, 5, 7
    q, k = torch.randn(T, H, dk, dtype=P.F), torch.randn(T, H, dk, dtype=P.F)
    v = torch.randn(T, H, dv, dtype=P.F)
    ig = torch.randn(T, H, dtype=P.F) * 4
    fg = torch.nn.functional.logsigmoid(torch.randn(T, H, dtype=P.F) * 4)
    whole, _ = P.matrix_memory_cell(q, k, v, ig, fg)
    assert torch.allclose(whole, P.matrix_memory_all_pairs(q, k, v, ig, fg), atol=1e-11)
    # carried state: two portions equal the whole
    a, st = P.matrix_memory_cell(q[:23], k[:23], v[:23], ig[:23], fg[:23])
    b, _ = P.matrix_memory_cell(q[23:], k[23:], v[23:], ig[23:], fg[23:], st)
    assert torch.allclose(torch.cat([a, b]), whole, atol=1e-12)


def test_memory_cell_first_token_by_hand():
    # one head, one key and one value element: S = exp(i - m) k v, m = max(f + 0, i)
    q, k, v = (torch.tensor([[[x]]], dtype=P.F) for x in (2.0, 3.0, 5.0))
    for i, f in ((1.5, -0.2), (-3.0, -0.1)):
        o, (S, n, m) = P.matrix_memory_cell(q, k, v, torch.tensor([[i]], dtype=P.F),
                                            torch.tensor([[f]], dtype=P.F))
        mm = max(f, i)
        s = math.exp(i - mm) * 15.0
        nn = math.exp(i - mm) * 3.0
        assert math.isclose(float(m), mm) and math.isclose(float(S), s)
        assert math.isclose(float(o), s * 2.0 / (max(abs(nn * 2.0), math.exp(-mm)) + 1e-6))


def test_differential_attention_reduces_to_one_softmax_when_lambda_vanishes():
    torch.manual_seed(2)
    T, D = 9, 12
    m = {"heads": 2, "kv_heads": 1, "dim": 4, "vdim": 6, "diff": 0.0, "scale": 0.5,
         "mask": {"size": 4, "keep_first": 1}, "rot": {"dims": 0, "base": 1.0}}
    w = {"q": torch.randn(16, D, dtype=P.F), "k": torch.randn(8, D, dtype=P.F),
         "v": torch.randn(6, D, dtype=P.F), "g": torch.zeros(2, D, dtype=P.F),
         "o": torch.eye(12, dtype=P.F), "lq1": torch.zeros(4, dtype=P.F), "lk1": torch.zeros(4, dtype=P.F),
         "lq2": torch.zeros(4, dtype=P.F), "lk2": torch.zeros(4, dtype=P.F)}          # lambda = 1 - 1 + 0
    h = torch.randn(T, D, dtype=P.F)
    got = P.differential_attention(h, w, "", m, 1e-9).view(T, 2, 6)
    q = (h @ w["q"].T).view(T, 2, 2, 4)
    k = (h @ w["k"].T).view(T, 1, 2, 4)
    v = (h @ w["v"].T)
    s = (q[:, 1, 0] @ k[:, 0, 0].T) * 0.5
    a = torch.softmax(s.masked_fill(~P.visible(T, 4, 1), -math.inf), -1) @ v
    want = P.unit_rms(a, 1e-9) * 0.5                         # gate: sigmoid(0)
    assert torch.allclose(got[:, 1], want, atol=1e-12)


# --------------------------------------------------------------------------- configuration
def test_config_reader_round_trip_and_errors():
    for name, raw in CASES.items():
        c = PigodraConfig.from_dict(raw)
        assert PigodraConfig.from_dict(c.to_dict()) == c
        assert architecture_of(raw).names[0] == "Pigodra"
    bad = json.loads(json.dumps(CASES["A"]))
    bad["layers"][0]["type"] = "conv"
    with pytest.raises(ConfigError):
        PigodraConfig.from_dict(bad)
    bad = json.loads(json.dumps(CASES["A"]))
    del bad["layers"][1]["mixer"]["vdim"]
    with pytest.raises(ConfigError):
        PigodraConfig.from_dict(bad)
    bad = json.loads(json.dumps(CASES["A"]))
    bad["layers"][0]["mixer"]["kv_heads"] = 4
    with pytest.raises(ConfigError):
        PigodraConfig.from_dict(bad)


def test_plan_takes_every_size_from_the_configuration():
    arch = architecture_of(CASES["B"])
    c = arch.read_config(CASES["B"])
    plan = arch.plan(c)
    assert plan.dim == 104 and plan.vocab_size == 211 and plan.embedding_scale is None
    kinds = [l.mixer.kind for l in plan.layers]
    assert kinds == ["matrix_memory", "differential_attention", "matrix_memory", "differential_attention"]
    m0, a1, m2, a3 = (l.mixer for l in plan.layers)
    assert (m0.n_heads, m0.key_dim, m0.value_dim, m0.gate_cap) == (1, 24, 40, None)
    assert (a1.n_heads, a1.n_kv_heads, a1.head_dim, a1.value_dim) == (4, 1, 24, 24)
    assert (a1.window, a1.keep_first, a1.scale, a1.lam_init) == (7, 0, 0.3, 0.1)
    assert a1.position.rotary_dim == 8 and a1.position.scaling_dict() == {"rope_type": "linear", "factor": 1.5}
    assert (a3.window, a3.keep_first, a3.scale) == (90, 70, None)
    assert plan.layers[0].feed_forward is None and plan.layers[2].feed_forward.hidden == 52
    assert plan.layers[2].feed_forward.activation == "gelu_tanh"
    assert all(l.mixer_norm.weight_offset == 1.0 and l.mixer_norm.eps == 1e-6 for l in plan.layers)
    assert arch.plan(arch.read_config(CASES["A"])).embedding_scale == 1.7
    # no rotation at all
    t = arch.plan(arch.read_config(CASES["T"]))
    assert t.layers[0].mixer.position.kind == "none" and t.layers[0].mixer.window is None


def test_linear_frequency_scaling():
    from gpt_fast_amd.parts.position import FREQUENCY_SCALINGS, rotary_frequencies
    f = rotary_frequencies(8, 100.0)
    assert torch.allclose(FREQUENCY_SCALINGS["linear"](f, factor=4.0), f / 4.0)
    assert torch.allclose(f, torch.tensor([100.0 ** (-2 * i / 8) for i in range(4)]))


def test_checkpoint_layout_joins_what_reads_the_same_input(tmp_path):
    folder = make_folder(tmp_path, "A", seed=5, dtype="float32")
    arch, c = gfa.read_model_folder(folder)
    from gpt_fast_amd.weights.bindings import load_parameters
    params = load_parameters(folder, arch.layouts(c), "float32", None)
    _, w = P.load_folder(folder)
    got = params["l1.mix.w_in"].double()
    want = torch.cat([w["l1.mix." + n] for n in ("q", "k", "v", "g", "i", "f")])
    assert torch.equal(got, want)
    assert torch.equal(params["l1.mix.gate_bias"].double(), torch.cat([w["l1.mix.i.b"], w["l1.mix.f.b"]]))
    got = params["l0.mix.w_in"].double()
    assert torch.equal(got, torch.cat([w["l0.mix." + n] for n in ("q", "k", "v", "g")]))
    assert got.shape[0] == 6 * 2 * 16 + 2 * 2 * 16 + 2 * 32 + 6
    assert torch.equal(params["l0.mlp.w13"].double(), torch.cat([w["l0.mlp.gate"], w["l0.mlp.up"]]))
    assert "l3.mlp.w13" not in params and "l3.norm2.weight" not in params
    # a missing and a misshapen tensor are both named
    from gpt_fast_amd.weights.bindings import WeightsError
    from gpt_fast_amd.weights.safetensors_io import write_safetensors
    broken = {k: v.float() for k, v in w.items() if k != "l2.mix.lq2"}
    broken["l1.mix.i.b"] = torch.zeros(4)
    write_safetensors(os.path.join(folder, "model.safetensors"), broken)
    with pytest.raises(WeightsError) as e:
        load_parameters(folder, arch.layouts(c), "float32", None)
    assert "l2.mix.lq2" in str(e.value) and "l1.mix.i.b" in str(e.value)


def test_cache_needs_of_the_mixers():
    from gpt_fast_amd.parts.base import Runtime
    from gpt_fast_amd.parts.model import DecoderModel
    arch = architecture_of(CASES["B"])
    model = DecoderModel(arch.plan(arch.read_config(CASES["B"])), Runtime(torch.float32, "cpu"))
    needs = model.cache_needs()
    assert needs[0] == StateNeed((1 * (24 * 40 + 24 + 1),), "float32")
    assert needs[1] == KVNeed(1, 48, 7, 24, 0)
    assert needs[2] == StateNeed((5 * (20 * 12 + 20 + 1),), "float32")
    assert needs[3] == KVNeed(3, 40, 90, 40, 70)


def test_window_gives_pages_back_but_keeps_the_first_keys_pages():
    from gpt_fast_amd.cache.store import Cache
    need = KVNeed(1, 8, window=70, value_dim=4, keep_first=65)     # kept keys reach into page 1
    cache = Cache([need, KVNeed(1, 8, window=70, value_dim=4, keep_first=0)], [None, None],
                  max_tokens=64 * 8, max_sequences=2, dtype=torch.float32, device="cpu")
    s = cache.acquire()
    cache.extend(s, 300)
    assert cache.page_list(0, s) == cache.page_list(1, s) == [0, 1, 2, 3, 4]
    cache.extend(s, 1)            # position 300 sees keys from 231: pages 0..2 are out of reach
    assert cache.page_list(0, s) == [0, 1, -1, 3, 4]
    assert cache.page_list(1, s) == [-1, -1, -1, 3, 4]
    cache.check()
    for _ in range(200):
        cache.extend(s, 1)
    assert cache.page_list(0, s)[:2] == [0, 1] and cache.page_list(1, s)[:2] == [-1, -1]
    assert sum(p >= 0 for p in cache.page_list(0, s)) <= 2 + 3
    cache.check()
    cache.release(s)
    assert cache.groups[0].pages.free == 8 and cache.groups[1].pages.free == 8
