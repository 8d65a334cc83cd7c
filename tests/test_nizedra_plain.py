"""CPU tests of the Nizedra architecture: its configuration, plan, checkpoint layout and cache
needs, and the plain implementation of tests/plain_nizedra.py against closed forms and
invariants that pin how each equation is read."""
import json
import math
import os

import pytest
import torch

import plain_nizedra as P
from nizedra_cases import CASES, make_folder

F = torch.float64


# --------------------------------------------------------------------------- configuration
def _arch():
    import gpt_fast_amd as gfa
    return gfa.architecture("Nizedra")


@pytest.mark.parametrize("name", sorted(CASES))
def test_config_plan_and_order(name):
    arch = _arch()
    raw = CASES[name]
    cfg = arch.read_config(raw)
    assert arch.read_config(arch.config_dict(cfg)) == cfg
    plan = arch.plan(cfg)
    want = P.run_order(raw)
    assert [(r.layer, r.enter is not None) for r in plan.order] == want
    kinds = {"lightning": "decayed_memory", "latent_attention": "latent_attention",
             "attention": "mixed_heads_attention"}
    for spec, layer in zip(plan.layers, raw["layers"]):
        assert spec.arrangement == "sandwich_norm"
        assert spec.mixer.kind == kinds[layer["type"]]
        assert (spec.feed_forward is None) == (layer["mlp"] is None)
        if layer["mlp"] is not None:
            assert spec.feed_forward.kind == "dense" and spec.feed_forward.hidden == layer["mlp"]["ff"]
    # the input mix is one part, whatever the number of passes
    enters = {id(r.enter) for r in plan.order if r.enter is not None}
    assert len(enters) == (1 if raw.get("loop") and raw["loop"]["times"] else 0)


def test_config_errors_name_the_place():
    arch = _arch()
    from gpt_fast_amd.config.nizedra import ConfigError
    bad = json.loads(json.dumps(CASES["A"]))
    bad["layers"][1]["mixer"]["decay"] = [0.5]
    with pytest.raises(ConfigError, match=r"layers\[1\]"):
        arch.read_config(bad)
    bad = json.loads(json.dumps(CASES["A"]))
    bad["layers"][2]["type"] = "convolution"
    with pytest.raises(ConfigError, match="convolution"):
        arch.read_config(bad)
    bad = json.loads(json.dumps(CASES["A"]))
    bad["loop"]["stop"] = 9
    with pytest.raises(ConfigError, match="loop"):
        arch.read_config(bad)
    bad = json.loads(json.dumps(CASES["B"]))
    bad["layers"][3]["mixer"]["kv_heads"] = 3
    with pytest.raises(ConfigError, match="kv_heads"):
        arch.read_config(bad)


@pytest.mark.parametrize("name", sorted(CASES))
def test_model_folder_tensors_and_sizes_from_their_shapes(tmp_path, name):
    """A written folder holds exactly the layout's tensors; its config.json does not say how
    many rows the distance tables have, the checkpoint does; the cache has an entry per run."""
    import gpt_fast_amd as gfa
    from gpt_fast_amd.cache.store import KVNeed, StateNeed
    from gpt_fast_amd.parts.base import Runtime
    from gpt_fast_amd.parts.model import DecoderModel
    from gpt_fast_amd.weights.bindings import load_parameters
    folder = make_folder(tmp_path, name, seed=1)
    raw, w = P.load_folder(folder)
    assert all("bias_rows" not in l["mixer"] for l in raw["layers"])
    arch, cfg = gfa.read_model_folder(folder)
    for i, l in enumerate(raw["layers"]):
        if l["type"] == "attention":
            assert cfg.layers[i].mixer.bias_rows == w[f"l{i}.mix.rel"].shape[0] == CASES[name]["layers"][i]["mixer"]["bias_rows"]
    layout = arch.bindings(cfg)
    names = {s.name for b in layout.bindings for s in b.sources}
    assert names == set(w)
    assert ("loop.in" in names) == (raw.get("loop") is not None)
    params = load_parameters(folder, arch.layouts(cfg), "float32", None)
    model = DecoderModel(arch.plan(cfg), Runtime(torch.float32, "cpu"))
    model.bind(params)
    needs = model.cache_needs()
    order = P.run_order(raw)
    assert len(needs) == len(order)
    for need, (i, _) in zip(needs, order):
        m = raw["layers"][i]["mixer"]
        if raw["layers"][i]["type"] == "lightning":
            assert need == StateNeed((m["heads"] * m["dim"] * m["vdim"],), "float32")
        elif raw["layers"][i]["type"] == "latent_attention":
            assert need == KVNeed(1, m["kv_rank"] + m["rot_dim"], (m.get("mask") or {}).get("size"), m["kv_rank"])
        else:
            assert need == KVNeed(m["kv_heads"], m["dim"], None, m["vdim"])
    # a wrong shape is reported with the tensor's name
    from gpt_fast_amd.weights.bindings import WeightsError
    other = json.loads(json.dumps(CASES[name]))
    other["width"] += 8
    with pytest.raises(WeightsError, match="embed"):
        load_parameters(folder, arch.layouts(arch.read_config(other)), "float32", None)


def test_a_loop_without_a_pass_needs_no_matrix_and_tolerates_one(tmp_path):
    import gpt_fast_amd as gfa
    from gpt_fast_amd.weights.bindings import load_parameters
    from gpt_fast_amd.weights.safetensors_io import write_safetensors
    from nizedra_cases import write_model
    for loop in ({"start": 1, "stop": 1, "times": 2}, {"start": 0, "stop": 2, "times": 0}):
        raw = {**CASES["B"], "loop": loop}
        folder = write_model(str(tmp_path / f"empty{loop['times']}"), raw, 3)
        arch, cfg = gfa.read_model_folder(folder)
        plan = arch.plan(cfg)
        assert all(r.enter is None for r in plan.order)
        assert [r.layer for r in plan.order] == [i for i, _ in P.run_order(raw)]
        params = load_parameters(folder, arch.layouts(cfg), "float32", None)
        assert "loop.in" not in params
        # ... and with the matrix in the file
        _, w = P.load_folder(folder)
        w["loop.in"] = torch.zeros(raw["width"], 2 * raw["width"])
        write_safetensors(os.path.join(folder, "model.safetensors"), {k: v.float() for k, v in w.items()})
        assert "loop.in" not in load_parameters(folder, arch.layouts(cfg), "float32", None)


def test_cache_entries_of_a_looped_layer_are_apart(tmp_path):
    import gpt_fast_amd as gfa
    from gpt_fast_amd.cache.store import Cache
    from gpt_fast_amd.parts.base import Runtime
    from gpt_fast_amd.parts.model import DecoderModel
    arch = _arch()
    cfg = arch.read_config(CASES["A"])
    model = DecoderModel(arch.plan(cfg), Runtime(torch.float32, "cpu"))
    cache = Cache(model.cache_needs(), model.cache_borrow(), max_tokens=256, max_sequences=2,
                  dtype=torch.float32, device="cpu")
    seen = set()
    for e in cache.entries:
        assert e is not None and (e.group_id, e.index) not in seen
        seen.add((e.group_id, e.index))
    assert len(seen) == len(P.run_order(CASES["A"])) == 1 + 3 * 2 + 1
    # a window below a page gives pages back while a sequence grows
    slot = cache.acquire()
    cache.extend(slot, 200)
    cache.extend(slot, 1)
    windowed = [g for _, g in cache.kv_groups if g.need.window is not None][0]
    assert windowed.held[slot][0] == -1 and windowed.held[slot][-1] >= 0
    cache.release(slot)
    cache.check()


# --------------------------------------------------------------------------- the plain pieces
def test_xielu_pieces():
    z = torch.linspace(-6, 6, 241, dtype=F)
    for p, q in ((0.7, -1.3), (0.0, 0.0), (-3.0, 2.0)):
        y = P.xielu(z, p, q)
        assert float(P.xielu(torch.zeros(1, dtype=F), p, q)) == 0.0
        # continuous with slope 1/2 at zero from both sides
        h = 1e-6
        up = float(P.xielu(torch.tensor([h], dtype=F), p, q)) / h
        down = float(P.xielu(torch.tensor([-h], dtype=F), p, q)) / -h
        assert abs(up - 0.5) < 1e-5 and abs(down - 0.5) < 1e-5
        a, b = math.log1p(math.exp(p)), 0.5 + math.log1p(math.exp(q))
        assert torch.allclose(y[z > 0], a * z[z > 0] ** 2 + z[z > 0] / 2)
        neg = z[z <= 0]
        assert torch.allclose(y[z <= 0], b * (torch.exp(neg) - 1 - neg) + neg / 2)


def test_distance_bucket_rows():
    # exact rows, then logarithmic steps, the last row from the far distance on
    assert [P.distance_bucket(n, 8, 50) for n in range(6)] == [0, 1, 2, 3, 4, 4]
    assert P.distance_bucket(49, 8, 50) == 7 and P.distance_bucket(50, 8, 50) == 7
    assert P.distance_bucket(10 ** 6, 8, 50) == 7
    for rows, far in ((8, 50), (6, 9), (32, 2000), (7, 300)):
        half = rows // 2
        got = [P.distance_bucket(n, rows, far) for n in range(int(far) + 5)]
        assert got[:half] == list(range(half)) and got[half] == half
        assert all(a <= b for a, b in zip(got, got[1:])) and max(got) == rows - 1
        # the step from row r to r + 1 lies at half * (far / half) ** ((r + 1 - half) / (rows - half))
        for r in range(half, rows - 1):
            edge = half * (far / half) ** ((r + 1 - half) / (rows - half))
            n = math.ceil(edge)
            if n - edge > 1e-9:
                assert P.distance_bucket(n, rows, far) >= r + 1 > P.distance_bucket(n - 1, rows, far) \
                    or n - 1 < half


def test_rotation_is_relative_and_leaves_the_rest():
    torch.manual_seed(0)
    x, y = torch.randn(1, 3, 12, dtype=F), torch.randn(1, 3, 12, dtype=F)
    def dot(px, py):
        a = P.rotate_pairs(x, torch.tensor([px]), 8, 500.0)
        b = P.rotate_pairs(y, torch.tensor([py]), 8, 500.0)
        return (a * b).sum(-1)
    assert torch.allclose(dot(7, 3), dot(104, 100))
    assert not torch.allclose(dot(7, 3), dot(7, 4))
    r = P.rotate_pairs(x, torch.tensor([5]), 8, 500.0)
    assert torch.equal(r[..., 8:], x[..., 8:])
    # the pair (2i, 2i+1) turns by p * base^(-2i/dims): the first pair by p itself
    one = torch.zeros(1, 1, 4, dtype=F)
    one[0, 0, 0] = 1.0
    r = P.rotate_pairs(one, torch.tensor([2]), 4, 100.0)
    assert torch.allclose(r[0, 0, :2], torch.tensor([math.cos(2.0), math.sin(2.0)], dtype=F))
    one = torch.zeros(1, 1, 4, dtype=F)
    one[0, 0, 2] = 1.0
    r = P.rotate_pairs(one, torch.tensor([2]), 4, 100.0)
    assert torch.allclose(r[0, 0, 2:], torch.tensor([math.cos(0.2), math.sin(0.2)], dtype=F))


def test_decayed_memory_is_a_sum_over_earlier_tokens():
    torch.manual_seed(1)
    T, H, dk, dv = 40, 3, 5, 7
    q, k, v = (torch.randn(T, H, d, dtype=F) for d in (dk, dk, dv))
    decay = torch.tensor([0.5, 0.9, 0.999], dtype=F)
    o, S = P.decayed_memory_cell(q, k, v, decay)
    t, s = torch.arange(T)[:, None], torch.arange(T)[None, :]
    for h in range(H):
        wts = torch.where(s <= t, decay[h] ** (t - s).clamp_min(0).to(F), torch.zeros((), dtype=F))
        assert torch.allclose(o[:, h], ((q[:, h] @ k[:, h].T) * wts) @ v[:, h])
    # carried on from a state: the same as one run
    o1, S1 = P.decayed_memory_cell(q[:25], k[:25], v[:25], decay)
    o2, S2 = P.decayed_memory_cell(q[25:], k[25:], v[25:], decay, S1)
    assert torch.allclose(torch.cat([o1, o2]), o) and torch.allclose(S2, S)


def _random_weights(cfg_layer, width, prefix, seed):
    torch.manual_seed(seed)
    m = cfg_layer["mixer"]
    w = {}
    if cfg_layer["type"] == "latent_attention":
        H, d, dr, dv, R, Q = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"], m["q_rank"]
        shapes = {"dq": (Q, width), "dq.norm": (Q,), "uq": (H * (d + dr), Q), "dkv": (R + dr, width),
                  "dkv.norm": (R,), "uk": (H * d, R), "uv": (H * dv, R), "o": (width, H * dv)}
    else:
        H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        shapes = {"q": (H * d, width), "q.b": (H * d,), "k": (G * d, width), "k.b": (G * d,),
                  "v": (G * dv, width), "v.b": (G * dv,), "rel": (m["bias_rows"], H), "talk": (H, H),
                  "temp": (H,), "o": (width, H * dv), "o.b": (width,)}
    for n, s in shapes.items():
        w[prefix + n] = torch.randn(*s, dtype=F) * (0.3 if len(s) == 2 else 1.0)
    return w


def test_latent_attention_equals_attention_in_the_latents_space():
    """Keys and values expanded per head, as the plain function does, give what one kv head
    whose key is [latent, rotated part] and whose value is the latent gives, with the query
    carried through w_uk and the result through w_uv."""
    layer = CASES["A"]["layers"][0]
    m = layer["mixer"]
    w = _random_weights(layer, 96, "x.", 3)
    h = torch.randn(60, 96, dtype=F)
    want = P.latent_attention(h, w, "x.", m, 1e-5)
    T, H, d, dr, dv, R = 60, m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    pos = torch.arange(T)
    cq = P.rms_norm(h @ w["x.dq"].T, w["x.dq.norm"], 1e-5)
    q = (cq @ w["x.uq"].T).view(T, H, d + dr)
    dkv = h @ w["x.dkv"].T
    c = P.rms_norm(dkv[:, :R], w["x.dkv.norm"], 1e-5)
    key = torch.cat([c, P.rotate_pairs(dkv[:, R:], pos, m["rot"]["dims"], m["rot"]["base"])], -1)
    q_rot = P.rotate_pairs(q[..., d:], pos, m["rot"]["dims"], m["rot"]["base"])
    i, j = pos[:, None], pos[None, :]
    see = (j <= i) & (i - j < m["mask"]["size"])
    heads = []
    for hh in range(H):
        q_lat = q[:, hh, :d] @ w["x.uk"].view(H, d, R)[hh]
        s = (torch.cat([q_lat, q_rot[:, hh]], -1) @ key.T) * m["scale"]
        a = torch.softmax(s.masked_fill(~see, -math.inf), -1)
        heads.append((a @ c) @ w["x.uv"].view(H, dv, R)[hh].T)
    assert torch.allclose(torch.cat(heads, -1) @ w["x.o"].T, want, atol=1e-10)
    # the window: the token at 40 sees 17 .. 40 and nothing before
    h2 = h.clone()
    h2[:17 - 0] += 1.0
    far = P.latent_attention(h2, w, "x.", m, 1e-5)
    assert torch.allclose(far[40:41], want[40:41], atol=1e-10) and not torch.allclose(far[39:40], want[39:40], atol=1e-6)


def test_mixed_heads_attention_order_of_its_steps():
    layer = CASES["A"]["layers"][2]
    m = dict(layer["mixer"])
    w = _random_weights(layer, 96, "x.", 4)
    h = torch.randn(30, 96, dtype=F)
    base = P.softmax_attention(h, w, "x.", m, 1e-5)
    # the scale does not multiply the bias: without a scale the bias alone still decides
    flat = P.softmax_attention(h, w, "x.", {**m, "scale": 0.0}, 1e-5)
    w0 = {**w, "x.rel": torch.zeros_like(w["x.rel"])}
    uniform = P.softmax_attention(h, w0, "x.", {**m, "scale": 0.0}, 1e-5)
    assert not torch.allclose(flat, uniform, atol=1e-6)
    # ... and with neither, every head averages its kv head's values so far
    T, H, G, dv = 30, m["heads"], m["kv_heads"], m["vdim"]
    v = (h @ w["x.v"].T + w["x.v.b"]).view(T, G, dv)
    mean = torch.cumsum(v, 0) / torch.arange(1, T + 1, dtype=F)[:, None, None]
    want = mean[:, [hh // (H // G) for hh in range(H)]].reshape(T, H * dv) @ w["x.o"].T + w["x.o.b"]
    assert torch.allclose(uniform, want, atol=1e-10)
    # the mix stands before the softmax: swapping two rows of it swaps which values two heads
    # of different kv heads weigh with which scores; with the identity nothing is mixed
    eye = {**w, "x.talk": torch.eye(H, dtype=F)}
    alone = P.softmax_attention(h, eye, "x.", m, 1e-5)
    assert not torch.allclose(alone, base, atol=1e-6)
    # q and k are normed: their size does not matter (but for eps), v's does
    big = {**w, "x.q": w["x.q"] * 7, "x.q.b": w["x.q.b"] * 7}
    assert torch.allclose(P.softmax_attention(h, big, "x.", m, 1e-12), P.softmax_attention(h, w, "x.", m, 1e-12), atol=1e-8)
    # the cap bounds a score before the bias is added
    hot = P.softmax_attention(h, {**w, "x.temp": w["x.temp"] * 1e6}, "x.", m, 1e-5)
    assert torch.isfinite(hot).all()


def test_whole_model_run_order_and_first_tokens(tmp_path):
    """The stream after every run; a looped layer's passes have states of their own; the
    prompt's first token alone equals the first row of a longer prompt (causal everywhere)."""
    for name in ("A", "C", "O"):
        folder = make_folder(tmp_path, name, seed=2)
        cfg, w = P.load_folder(folder)
        toks = [5, 9, 2, 77, 31, 8, 64, 3, 19, 20, 21, 40]
        outs = []
        full = P.forward(w, cfg, toks, outs)
        assert len(outs) == len(P.run_order(cfg))
        assert torch.allclose(P.forward(w, cfg, toks[:1]), full[:1], atol=1e-9)
        assert torch.allclose(P.forward(w, cfg, toks[:7]), full[:7], atol=1e-9)
        assert P.greedy_generate(w, cfg, toks[:4], 3) == P.greedy_generate(w, cfg, toks[:4], 5)[:3]
