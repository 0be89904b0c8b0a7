"""Lusolix without a GPU: configuration, tensor declarations, what the layers ask of the cache manager, and the plain
implementation's mechanisms pinned against special cases that reduce to something known."""
from __future__ import annotations

import copy
import math

import pytest
import torch

from lusolix_cases import P, Q, R
from plain import lusolix_plain as L


# ----------------------------------------------------------------------------------------------- configuration

def test_config_reads_every_size_and_constant():
    from tokenmill_amd.config import LusolixConfig
    from tokenmill_amd.config.registry import architecture_name, get_architecture
    assert architecture_name(P) == "Lusolix" and get_architecture("Lusolix").name == "Lusolix"
    cfg = LusolixConfig.from_dict(P)
    assert (cfg.vocab_size, cfg.hidden_size, cfg.max_position_embeddings, cfg.norm_eps, cfg.residual_mult, cfg.conv_taps) == \
        (211, 96, 320, 3e-5, 0.5, 3)
    assert [l.mlp and l.mlp["kind"] for l in cfg.layers] == ["moe", "dense", None, "moe"]
    assert cfg.layers[0].mlp == {"kind": "moe", "ff": 40, "experts": 5, "top": 2} and cfg.layers[1].mlp == {"kind": "dense", "ff": 136}
    assert cfg.layers[1].mixer["rot"] == {"base": 5e5, "dims": 4} and cfg.layers[1].mixer["mask"]["size"] == 50
    assert "mask" not in cfg.layers[2].mixer
    cfg = LusolixConfig.from_dict(Q)
    assert cfg.conv_taps == 1 and cfg.residual_mult == 1.0 and "rot" not in cfg.layers[2].mixer
    bare = copy.deepcopy(Q)
    bare.pop("canon"), bare.pop("residual_mult")
    cfg = LusolixConfig.from_dict(bare)
    assert cfg.conv_taps == 0 and cfg.residual_mult == 1.0


@pytest.mark.parametrize("edit,match", [
    (lambda c: c.pop("norm"), "norm"),
    (lambda c: c.pop("width"), "width"),
    (lambda c: c["layers"][0].update(type="attention"), "type"),
    (lambda c: c["layers"][1]["mixer"].pop("kv_rank"), "kv_rank"),
    (lambda c: c["layers"][1]["mixer"].pop("scale"), "scale"),
    (lambda c: c["layers"][1]["mixer"]["rot"].update(dims=10), "rot.dims"),
    (lambda c: c["layers"][1]["mixer"]["rot"].update(dims=3), "rot.dims"),
    (lambda c: c["layers"][1]["mlp"].update(kind="routed"), "kind"),
    (lambda c: c["layers"][1]["mlp"].pop("ff"), "ff"),
    (lambda c: c["layers"][0]["mlp"]["router"].update(top=6), "experts"),
    (lambda c: c["layers"][0]["mlp"]["router"].pop("experts"), "experts"),
    (lambda c: c["layers"][0]["mixer"]["mask"].update(size=0), "mask.size"),
    (lambda c: c["canon"].update(taps=17), "taps"),
])
def test_config_refuses_what_the_model_cannot_be(edit, match):
    from tokenmill_amd.config import ConfigError, LusolixConfig
    raw = copy.deepcopy(P)
    edit(raw)
    with pytest.raises(ConfigError, match=match):
        LusolixConfig.from_dict(raw)


def test_tensor_names_shapes_and_caches():
    from tokenmill_amd.config import LusolixConfig
    from tokenmill_amd.models.lusolix import build_lusolix
    from tokenmill_amd.parts import KVCacheSpec, LayerCacheSpec, StateSpec
    model = build_lusolix(LusolixConfig.from_dict(P))
    specs = model.tensor_specs()
    assert specs["embed"].shape == (211, 96) and specs["pos"].shape == (320, 96) and "head" not in specs
    assert specs["final.norm"].shape == (96,) and specs["final.norm.b"].shape == (96,)
    assert specs["l0.norm1"].shape == (96,) and specs["l0.norm1.b"].shape == (96,) and specs["l0.canon1"].shape == (96, 3)
    assert specs["l0.rg1"].shape == (96, 96) and specs["l0.rg1.b"].shape == (96,) and specs["l0.rg2.b"].shape == (96,)
    assert specs["l0.mix.dq"].shape == (40, 96) and specs["l0.mix.dq.norm"].shape == (40,) and specs["l0.mix.uq"].shape == (3 * 32, 40)
    assert specs["l0.mix.dkv"].shape == (36 + 12, 96) and specs["l0.mix.dkv.norm"].shape == (36,)
    assert specs["l0.mix.uk"].shape == (3 * 20, 36) and specs["l0.mix.uv"].shape == (3 * 24, 36)
    assert specs["l0.mix.g"].shape == (3, 96) and specs["l0.mix.o"].shape == (96, 3 * 24)
    assert specs["l0.mlp.table"].shape == (211, 2) and specs["l0.mlp.table"].kind == "int"
    assert specs["l0.mlp.e4.gate"].shape == (40, 96) and specs["l0.mlp.e4.down"].shape == (96, 40) and "l0.mlp.e5.up" not in specs
    assert specs["l1.mlp.up"].shape == (136, 96) and specs["l1.mlp.down"].shape == (96, 136) and specs["l1.mlp.act"].shape == (4,)
    assert "l1.mlp.up.b" not in specs and "l2.norm2" not in specs and "l2.rg2" not in specs and "l2.mlp.up" not in specs
    # pages for one row of latent + rotated channels per token, no value pool, and the convolution's rows beside them
    c = model.cache_specs()
    assert c[0] == LayerCacheSpec(KVCacheSpec(1, 48, 24, values=False), StateSpec((2, 96), None))
    assert c[2].kv == KVCacheSpec(1, 24, None, values=False) and c[3].kv.window == 7
    assert c[0].kv.value_dim == 0
    # a checkpoint may carry the second norm and gate of a layer without a feed-forward; nothing else may be unknown
    assert "l2.rg2" in model.ignorable and "l2.norm2.b" in model.ignorable and not any(n.startswith("l1.") for n in model.ignorable)
    # one tap: nothing to remember
    model = build_lusolix(LusolixConfig.from_dict(Q))
    assert model.cache_specs()[0] == KVCacheSpec(1, 120, 33, values=False)
    assert build_lusolix(LusolixConfig.from_dict(R)).cache_specs()[1].state == StateSpec((4, 72), None)


def test_random_tables_name_different_experts_and_models_are_written_and_read_back(tmp_path):
    from safetensors.torch import load_file
    from tokenmill_amd.config.registry import load_config
    from tokenmill_amd.weights import write_random_model
    d = write_random_model(P, tmp_path / "m", seed=3)
    arch, cfg = load_config(d)
    assert type(cfg).__name__ == "LusolixConfig"
    w = load_file(str(d / "model.safetensors"))
    assert set(w) == set(arch.build_model(cfg).tensor_specs())
    for name, experts, top in (("l0.mlp.table", 5, 2), ("l3.mlp.table", 7, 3)):
        t = w[name]
        assert t.dtype == torch.int32 and tuple(t.shape) == (211, top) and int(t.min()) >= 0 and int(t.max()) < experts
        assert all(len(set(row.tolist())) == top for row in t)
        assert len(set(map(tuple, t.tolist()))) > 3


def test_pools_hold_no_values_and_the_convolution_state_beside_the_pages():
    from tokenmill_amd.cache.pool import CachePools
    from tokenmill_amd.config import LusolixConfig
    from tokenmill_amd.models.lusolix import build_lusolix
    model = build_lusolix(LusolixConfig.from_dict(P))
    pools = CachePools(model, 6, 8, 3, torch.bfloat16, "cpu")
    assert len(pools.groups) == 4 and all(v is None for v in pools.v)
    assert tuple(pools.k[0].shape) == (1, 6, 8, 1, 48)
    assert sorted(pools.states) == [0, 1, 2, 3] and tuple(pools.states[0].shape) == (4, 2, 96) and pools.states[0].dtype == torch.bfloat16
    assert pools.views[1].state is pools.states[1] and pools.views[1].v is None and pools.views[1].k.shape[-1] == 80
    assert CachePools.bytes_per_token(model, torch.bfloat16) == 2 * (48 + 80 + 24 + 50)


# ----------------------------------------------------------------------------------------------- the plain mechanisms

def test_plain_layer_norm_and_convolution_are_the_library_routines():
    torch.manual_seed(0)
    x, w, b = torch.randn(5, 33) * 3 + 2, torch.rand(33) + 0.5, torch.randn(33)
    assert torch.allclose(L.layer_norm(x, w, b, 1e-5), torch.nn.functional.layer_norm(x, (33,), w, b, 1e-5), atol=1e-5)
    h, k = torch.randn(12, 7), torch.randn(7, 4)
    out, last = L.short_conv(h, k)
    ref = torch.nn.functional.conv1d(torch.nn.functional.pad(h.T[None], (3, 0)), k[:, None, :], groups=7)[0].T
    assert torch.allclose(out, h + ref, atol=1e-5) and torch.equal(last, h[-3:])
    # cut anywhere, also into pieces shorter than the taps, the state carries what is needed
    a, st = L.short_conv(h[:1], k)
    b2, st = L.short_conv(h[1:3], k, st)
    c, st = L.short_conv(h[3:], k, st)
    assert torch.allclose(torch.cat([a, b2, c]), out, atol=1e-6) and torch.equal(st, h[-3:])
    one, none = L.short_conv(h, k[:, :1])
    assert torch.allclose(one, h * (1 + k[:, 0])) and none.shape == (0, 7)


def test_plain_rotation_turns_neighbours_and_depends_on_distance_only():
    torch.manual_seed(1)
    v = torch.randn(6, 2, 10)
    pos = torch.tensor([0, 1, 5, 40, 41, 300])
    r = L.rotate_interleaved(v, pos, 1e4, 6)
    assert torch.equal(r[0], v[0]) and torch.equal(r[..., 6:], v[..., 6:])
    assert torch.allclose(r.norm(dim=-1), v.norm(dim=-1), atol=1e-5)
    # the first pair turns by the position itself (f_0 = 1)
    assert torch.allclose(r[1, 0, 0], v[1, 0, 0] * math.cos(1.0) - v[1, 0, 1] * math.sin(1.0), atol=1e-6)
    assert torch.allclose(r[1, 0, 1], v[1, 0, 1] * math.cos(1.0) + v[1, 0, 0] * math.sin(1.0), atol=1e-6)
    a, b = torch.randn(1, 6), torch.randn(1, 6)
    d1 = (L.rotate_interleaved(a, pos[3:4], 50.0, 6) * L.rotate_interleaved(b, pos[1:2], 50.0, 6)).sum()
    d2 = (L.rotate_interleaved(a, pos[4:5] + 59, 50.0, 6) * L.rotate_interleaved(b, pos[1:2] + 60, 50.0, 6)).sum()
    assert torch.allclose(d1, d2, atol=1e-4)


def _mixer_weights(m, width, seed):
    torch.manual_seed(seed)
    H, Dn, Dr, Dv, Lq, Lk = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["q_rank"], m["kv_rank"]
    shapes = {"dq": (Lq, width), "dq.norm": (Lq,), "uq": (H * (Dn + Dr), Lq), "dkv": (Lk + Dr, width), "dkv.norm": (Lk,),
              "uk": (H * Dn, Lk), "uv": (H * Dv, Lk), "g": (H, width), "o": (width, H * Dv)}
    return {"a." + k: (torch.rand(s) + 0.5 if k.endswith("norm") else torch.randn(s) * 0.3) for k, s in shapes.items()}


def test_plain_attention_by_hand_window_and_cut():
    m = dict(P["layers"][0]["mixer"])
    w = _mixer_weights(m, 30, 2)
    x = torch.randn(40, 30)
    pos = torch.arange(40)
    out, _ = L.latent_attention(x, pos, m, w, "a.", 1e-5, torch.float32)
    # position 30, head 1, by hand
    H, Dn, Dr, Dv, Lk = 3, 20, 12, 24, 36
    cq = L.rms_norm(x @ w["a.dq"].T, w["a.dq.norm"], 1e-5)
    qq = (cq @ w["a.uq"].T).view(40, H, Dn + Dr)
    low = x @ w["a.dkv"].T
    c = L.rms_norm(low[:, :Lk], w["a.dkv.norm"], 1e-5)
    kr = L.rotate_interleaved(low[:, Lk:], pos, 1e4, 12)
    qr = L.rotate_interleaved(qq[..., Dn:], pos, 1e4, 12)
    t, h = 30, 1
    keys = torch.cat([c @ w["a.uk"].view(H, Dn, Lk)[h].T, kr], 1)
    query = torch.cat([qq[t, h, :Dn], qr[t, h]])
    seen = list(range(t - 24 + 1, t + 1))                       # itself and the 23 before it
    p = torch.softmax(keys[seen] @ query * 0.2, 0)
    o = (p[:, None] * (c[seen] @ w["a.uv"].view(H, Dv, Lk)[h].T)).sum(0) * torch.sigmoid(x[t] @ w["a.g"][h])
    heads = torch.zeros(H * Dv)
    heads[h * Dv:(h + 1) * Dv] = o
    mine = w["a.o"] @ heads
    w0 = dict(w)
    w0["a.o"] = w["a.o"].clone()
    w0["a.o"][:, :Dv] = 0
    w0["a.o"][:, 2 * Dv:] = 0
    only_h, _ = L.latent_attention(x, pos, m, w0, "a.", 1e-5, torch.float32)
    assert torch.allclose(only_h[t], mine, atol=1e-4)
    # the rows seen earlier come back through ``seen``: cut in three
    a, st = L.latent_attention(x[:7], pos[:7], m, w, "a.", 1e-5, torch.float32)
    b, st = L.latent_attention(x[7:8], pos[7:8], m, w, "a.", 1e-5, torch.float32, st)
    c2, st = L.latent_attention(x[8:], pos[8:], m, w, "a.", 1e-5, torch.float32, st)
    assert torch.allclose(torch.cat([a, b, c2]), out, atol=1e-5)
    # without a window the first row is seen by all
    m2 = dict(m)
    m2.pop("mask")
    far, _ = L.latent_attention(x, pos, m2, w, "a.", 1e-5, torch.float32)
    assert torch.allclose(far[:24], out[:24], atol=1e-6) and not torch.allclose(far[24:], out[24:], atol=1e-4)


def test_plain_poly_norm_and_experts_by_hand():
    z = torch.tensor([[1.0, -2.0, 3.0, 0.5]])
    coef = torch.tensor([2.0, -1.0, 0.5, 0.25])
    want = 2 * z / z.pow(2).mean().sqrt() - z ** 2 / z.pow(4).mean().sqrt() + 0.5 * z ** 3 / z.pow(6).mean().sqrt() + 0.25
    assert torch.allclose(L.poly_norm(z, coef, 1e-12), want, atol=1e-5)
    torch.manual_seed(3)
    w = {"m.table": torch.tensor([[2, 0], [1, 2], [0, 1]], dtype=torch.int32)}
    for e in range(3):
        w[f"m.e{e}.gate"], w[f"m.e{e}.up"], w[f"m.e{e}.down"] = torch.randn(6, 10), torch.randn(6, 10), torch.randn(10, 6)
    x = torch.randn(4, 10)
    got = L.table_experts(x, torch.tensor([1, 1, 0, 2]), w, "m.", torch.float32)

    def expert(e, v):
        return w[f"m.e{e}.down"] @ (torch.nn.functional.silu(w[f"m.e{e}.gate"] @ v) * (w[f"m.e{e}.up"] @ v))
    assert torch.allclose(got[0], (expert(1, x[0]) + expert(2, x[0])) / 2, atol=1e-5)
    assert torch.allclose(got[2], (expert(2, x[2]) + expert(0, x[2])) / 2, atol=1e-5)
    assert torch.allclose(got[3], (expert(0, x[3]) + expert(1, x[3])) / 2, atol=1e-5)


@pytest.fixture(scope="module")
def drawn(tmp_path_factory):
    from safetensors.torch import load_file
    from tokenmill_amd.weights import write_random_model
    d = write_random_model(P, tmp_path_factory.mktemp("p"), seed=5, std=0.1, norm_std=0.1)
    return load_file(str(d / "model.safetensors"))


def test_plain_model_cut_into_calls_gives_the_whole(drawn):
    ids = torch.randint(0, 211, (70,)).tolist()
    whole = L.forward(P, drawn, ids)
    state: dict = {}
    parts = [L.forward(P, drawn, ids[a:b], start=a, state=state) for a, b in ((0, 1), (1, 3), (3, 40), (40, 41), (41, 70))]
    assert torch.allclose(torch.cat(parts), whole, atol=2e-5 * float(whole.abs().max()))


def test_plain_model_taken_apart(drawn):
    """With every output projection silent the model is the head on the final norm of the embedding's sum; with the gates'
    matrices silent a gate is the sigmoid of its bias; the residual multiplier scales what a layer adds."""
    ids = [5, 17, 200, 5]
    w = {k: v.clone() for k, v in drawn.items()}
    for i in range(4):
        w[f"l{i}.mix.o"].zero_()
    for name in list(w):
        if name.endswith(".down"):
            w[name].zero_()
    x = w["embed"].float()[ids] + w["pos"].float()[:4]
    want = L.layer_norm(x, w["final.norm"], w["final.norm.b"], 3e-5) @ w["embed"].float().T
    assert torch.allclose(L.forward(P, w, ids), want, atol=1e-5)
    one = copy.deepcopy(P)
    one["layers"] = one["layers"][2:3]                       # a layer without a feed-forward
    w1 = {k.replace("l2.", "l0."): v.clone() for k, v in drawn.items() if not k.startswith(("l0.", "l1.", "l3."))}
    w1["l0.rg1"].zero_()
    tr: list = []
    L.forward(one, w1, ids, trace=tr)
    x0 = w1["embed"].float()[ids] + w1["pos"].float()[:4]
    n = L.layer_norm(x0, w1["l0.norm1"], w1["l0.norm1.b"], 3e-5)
    u, _ = L.short_conv(n, w1["l0.canon1"])
    y, _ = L.latent_attention(u, torch.arange(4), one["layers"][0]["mixer"], w1, "l0.mix.", 3e-5, torch.float32)
    assert torch.allclose(tr[0], x0 + 0.5 * y * torch.sigmoid(w1["l0.rg1.b"].float()), atol=1e-5)
