"""Lusolix on the GPU against the plain implementation (``tests/plain/lusolix_plain.py``): every mechanism alone, then
whole models through the replay session and the engine: whole prompts, prefill + decoding, portions down to two
tokens, mixed batches with pages and state slots used again, rows at the edges of windows and pages, long decoding,
greedy generation through the scheduler."""
from __future__ import annotations

import json
import math

import pytest
import torch

from conftest import random_ids
from lusolix_cases import CASES, P, Q
from plain import lusolix_plain as L
from tolerances import F32_REL

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
DTS = [torch.float32, torch.bfloat16]
NAMES = {torch.float32: "float32", torch.bfloat16: "bfloat16"}


def q(x, dt):
    return x.to(dt).float()


def close(got, want, dt, what, bf16=2.0 ** -7):
    assert got.shape == want.shape and torch.isfinite(got).all(), f"{what}: shape or non-finite values"
    scale = float(want.abs().max())
    bound = (F32_REL if dt == torch.float32 else bf16) * max(scale, 1e-6)
    err = float((got - want).abs().max())
    assert err <= bound, f"{what}: max |diff| {err:.3e} > {bound:.3e} (largest value {scale:.3g})"


def ints(v):
    return torch.tensor(v, dtype=torch.int32, device=DEV)


# ----------------------------------------------------------------------------------------------- mechanisms alone

@pytest.mark.parametrize("dt", DTS)
@pytest.mark.parametrize("hidden", [72, 96, 1000, 4096])
def test_layer_norm_behind_a_gated_add(dt, hidden):
    from tokenmill_amd.parts import GatedAdd, LayerNorm, NormedInput, as_tensor
    torch.manual_seed(hidden)
    T, eps, mult = 6, 2e-5, 0.3
    norm = LayerNorm(hidden, eps, names=("", ".b"))
    w, b = q(torch.rand(hidden) + 0.5, dt), q(torch.randn(hidden), dt)
    norm.load({"n": w.to(dt).to(DEV), "n.b": b.to(dt).to(DEV)}, "n")
    resid = torch.randn(T, hidden) * 3 + 1.5
    y, g = q(torch.randn(T, hidden) * 5, dt), q(torch.randn(T, hidden) * 2, dt)
    r = resid.to(DEV)
    got = norm.add_norm(r, None, dt)
    close(got.float().cpu(), q(L.layer_norm(resid, w, b, eps), dt), dt, "norm alone", bf16=2.0 ** -8)
    assert torch.equal(r.cpu(), resid)
    want_sum = resid + mult * (y * torch.sigmoid(g))
    x = NormedInput(norm, r, y.to(dt).to(DEV), dt, delta_norm=GatedAdd(g.to(dt).to(DEV), mult))
    got = as_tensor(x)
    close(r.cpu(), want_sum, torch.float32, "residual after the gated add")
    close(got.float().cpu(), q(L.layer_norm(want_sum, w, b, eps), dt), dt, "norm of the sum", bf16=2.0 ** -8)
    r2 = resid.to(DEV)
    rows = ints([4, 0, 4, 1])
    got = norm.add_norm(r2, y.to(dt).to(DEV), dt, rows=rows, delta_norm=GatedAdd(g.to(dt).to(DEV), mult))
    close(got.float().cpu(), q(L.layer_norm(want_sum, w, b, eps), dt)[rows.cpu().long()], dt, "chosen rows", bf16=2.0 ** -8)
    assert torch.equal(r2.cpu(), resid)
    r3 = resid.to(DEV)
    GatedAdd(None, 2.0).add_normed(r3, y.to(dt).to(DEV))
    close(r3.cpu(), resid + 2.0 * y, torch.float32, "scaled add without a gate")
    r4 = resid.to(DEV)
    got = norm.add_norm(r4, y.to(dt).to(DEV), dt)
    close(r4.cpu(), resid + y, torch.float32, "plain add")
    close(got.float().cpu(), q(L.layer_norm(resid + y, w, b, eps), dt), dt, "norm behind a plain add", bf16=2.0 ** -8)


@pytest.mark.parametrize("dt", DTS)
@pytest.mark.parametrize("taps,width", [(1, 40), (2, 72), (4, 96), (5, 300), (16, 33)])
def test_short_convolution_whole_cut_and_beside_another_request(dt, taps, width):
    """A request's rows give the same numbers whole, cut anywhere (also into pieces shorter than the taps) and one by
    one, with another request's rows beside them; a slot that is used again starts from zeros."""
    from tokenmill_amd.hip import ops
    torch.manual_seed(taps * 100 + width)
    w = q(torch.randn(width, taps) * 0.5, dt)
    ha, hb = q(torch.randn(23, width), dt), q(torch.randn(9, width), dt)
    want_a, _ = L.short_conv(ha, w)
    want_b, _ = L.short_conv(hb, w)
    state = torch.full((3, max(taps - 1, 1), width), math.nan, dtype=dt, device=DEV)[:, :taps - 1]
    state = state.contiguous() if taps > 1 else None
    wd = w.to(dt).to(DEV)

    def run(pieces, walk=True):   # pieces: [(rows of a, rows of b)] per step; a in slot 2, b in slot 0; walk: one launch where rows are few
        if state is not None:
            state[2].zero_(), state[0].zero_()
        outs_a, outs_b, pa, pb = [], [], 0, 0
        for na, nb in pieces:
            h = torch.cat([ha[pa:pa + na], hb[pb:pb + nb]]).to(dt).to(DEV)
            seqs = [(na, 2)] * (na > 0) + [(nb, 0)] * (nb > 0)
            cu = [0]
            for n, _ in seqs:
                cu.append(cu[-1] + n)
            seq_of = [i for i, (n, _) in enumerate(seqs) for _ in range(n)]
            out = ops.short_conv(h, wd, state, ints(cu), ints([s for _, s in seqs]), ints(seq_of), len(seqs), torch.empty_like(h),
                                 most_rows=max(na, nb) if walk else 0)
            outs_a.append(out[:na].float().cpu())
            outs_b.append(out[na:].float().cpu())
            pa, pb = pa + na, pb + nb
        return torch.cat(outs_a), torch.cat(outs_b)

    for pieces in ([(23, 9)], [(10, 0), (13, 9)], [(1, 2), (2, 1), (1, 1), (7, 2), (12, 3)], [(1, 1)] * 9 + [(1, 0)] * 14):
        a, b = run(pieces)
        close(a, q(want_a, dt), dt, f"request a in {len(pieces)} steps", bf16=2.0 ** -8)
        close(b, q(want_b, dt), dt, f"request b in {len(pieces)} steps", bf16=2.0 ** -8)
    first = run([(23, 9)])
    for pieces, walk in (([(5, 4), (18, 5)], True), ([(1, 1)] * 9 + [(1, 0)] * 14, True), ([(1, 1)] * 9 + [(1, 0)] * 14, False)):
        again = run(pieces, walk)
        assert torch.equal(first[0], again[0]) and torch.equal(first[1], again[1]), "a cut changes bits"


@pytest.mark.parametrize("dt", DTS)
@pytest.mark.parametrize("F", [60, 136, 1000, 5000])
def test_poly_norm(dt, F):
    from tokenmill_amd.hip import ops
    torch.manual_seed(F)
    z = torch.randn(5, F) * 2
    z[0] *= 1e-3                    # a row so small that eps matters
    coef = torch.tensor([0.7, -0.4, 0.25, 0.1])
    out = ops.poly_norm(z.to(DEV), coef.to(DEV), torch.empty((5, F), dtype=dt, device=DEV), 1e-5)
    close(out.float().cpu(), q(L.poly_norm(z, coef, 1e-5), dt), dt, "poly_norm", bf16=2.0 ** -8)


@pytest.mark.parametrize("dt", DTS)
@pytest.mark.parametrize("T,H,K,N", [(1, 3, 20, 36), (37, 2, 72, 8), (130, 5, 8, 100), (4, 1, 44, 40), (200, 3, 64, 96)])
def test_products_head_by_head(dt, T, H, K, N):
    from tokenmill_amd.hip import ops
    torch.manual_seed(T + H)
    pad_a, pad_c = (6, 4) if K % 8 else (8, 8)
    a = q(torch.randn(T, H * (K + pad_a)), dt)
    b = q(torch.randn(H, K, N) * 0.3, dt)
    gate = torch.randn(T, H + 3)
    c = torch.full((T, H * (N + pad_c)), 7.0, dtype=dt, device=DEV)
    ops.heads_matmul(a.to(dt).to(DEV), K + pad_a, b.to(dt).to(DEV), c, N + pad_c, gate=gate.to(DEV)[:, 2:])
    want = torch.einsum("thk,hkn->thn", a.view(T, H, K + pad_a)[..., :K], b) * torch.sigmoid(gate[:, 2:2 + H])[:, :, None]
    got = c.float().cpu().view(T, H, N + pad_c)
    close(got[..., :N], q(want, dt), dt, "per-head product")
    assert bool((got[..., N:] == 7.0).all()), "wrote beyond a head's columns"
    if dt == torch.bfloat16 and K % 8 == 0:
        # the matrix unit, from the matrices as [H, N, K]; a row alone gives the bits it has among the others
        ad, wd = a.to(dt).to(DEV), b.transpose(1, 2).contiguous().to(dt).to(DEV)
        assert ops.heads_matmul_mfma_takes(ad, K + pad_a, wd)
        c2 = torch.full((T, H * (N + pad_c)), 7.0, dtype=dt, device=DEV)
        ops.heads_matmul_mfma(ad, K + pad_a, wd, c2, N + pad_c, gate=gate.to(DEV)[:, 2:])
        got2 = c2.float().cpu().view(T, H, N + pad_c)
        close(got2[..., :N], q(want, dt), dt, "per-head product on the matrix unit")
        assert bool((got2[..., N:] == 7.0).all()), "wrote beyond a head's columns"
        one = torch.zeros((1, H * (N + pad_c)), dtype=dt, device=DEV)
        ops.heads_matmul_mfma(ad[T // 2:T // 2 + 1], K + pad_a, wd, one, N + pad_c, gate=gate.to(DEV)[T // 2:T // 2 + 1, 2:])
        assert torch.equal(one.float().cpu().view(H, N + pad_c)[:, :N], got2[T // 2, :, :N])
        # the channels behind a head's inputs go behind its outputs in the same launch, the first four rotated by position
        from tokenmill_amd.parts import RotaryEmbedding
        table = RotaryEmbedding(6, 1e4, 64, rotary_dim=4, interleaved=True)
        table.build_tables(DEV)
        pos = torch.arange(T) % 64
        c3 = torch.full((T, H * (N + pad_c)), 7.0, dtype=dt, device=DEV)
        ops.heads_matmul_mfma(ad, K + pad_a, wd, c3, N + pad_c, tail=6, cos=table.cos, sin=table.sin, positions=pos.to(torch.int32).to(DEV))
        got3 = c3.float().cpu().view(T, H, N + pad_c)
        plain = torch.einsum("thk,hkn->thn", a.view(T, H, K + pad_a)[..., :K], b)
        close(got3[..., :N], q(plain, dt), dt, "per-head product beside a rotated tail")
        turned = L.rotate_interleaved(a.view(T, H, K + pad_a)[..., K:K + 6], pos, 1e4, 4)
        close(got3[..., N:N + 6], q(turned, dt), dt, "the rotated tail", bf16=2.0 ** -8)
        assert bool((got3[..., N + 6:] == 7.0).all()), "wrote beyond the tail"


def _experts_fixture(dt, width, ff, experts, top, vocab, seed):
    from tokenmill_amd.parts import TableRoutedExperts
    torch.manual_seed(seed)
    part = TableRoutedExperts(width, ff, experts, top, vocab)
    w = {}
    for name, spec in part.tensor_specs("m.").items():
        if spec.kind == "int":
            w[name] = torch.rand(vocab, experts).argsort(1)[:, :top].to(torch.int32)
        else:
            w[name] = q(torch.randn(spec.shape) * 0.2, dt)
    part.load({k: (v.to(DEV) if v.dtype == torch.int32 else v.to(dt).to(DEV)) for k, v in w.items()}, "m.")
    return part, w


@pytest.mark.parametrize("dt", DTS)
@pytest.mark.parametrize("width,ff,experts,top,T", [(96, 40, 5, 2, 77), (80, 16, 3, 3, 9), (80, 52, 4, 1, 1), (72, 32, 9, 2, 200), (64, 24, 40, 4, 3),
                                                      (96, 40, 5, 2, 300), (80, 16, 3, 3, 60)])
def test_experts_by_table(dt, width, ff, experts, top, T):
    from types import SimpleNamespace
    vocab = 50
    part, w = _experts_fixture(dt, width, ff, experts, top, vocab, width + T)
    ids = torch.randint(0, vocab, (T,))
    ids[: min(T, 5)] = ids[0]                                    # the same id several times: the same experts
    x = q(torch.randn(T, width), dt)
    step = SimpleNamespace(token_ids=ids.to(torch.int32).to(DEV), num_seqs=1)
    got = part.forward(x.to(dt).to(DEV), step).float().cpu()
    close(got, q(L.table_experts(x, ids, w, "m.", dt), dt), dt, "experts")
    # a row alone gives the bits it has in the batch
    one = part.forward(x[3 % T:3 % T + 1].to(dt).to(DEV), SimpleNamespace(token_ids=ids[3 % T:3 % T + 1].to(torch.int32).to(DEV), num_seqs=1))
    assert torch.equal(one.float().cpu()[0], got[3 % T])


def test_experts_refuse_a_table_that_names_no_expert():
    from tokenmill_amd.parts import TableRoutedExperts
    part, w = _experts_fixture(torch.float32, 32, 8, 3, 2, 10, 0)
    bad = dict(w)
    bad["m.table"] = w["m.table"].clone()
    bad["m.table"][4, 1] = 3
    with pytest.raises(ValueError, match="outside"):
        TableRoutedExperts(32, 8, 3, 2, 10).load({k: v.to(DEV) for k, v in bad.items()}, "m.")
    bad["m.table"][4] = torch.tensor([1, 1])
    with pytest.raises(ValueError, match="twice"):
        TableRoutedExperts(32, 8, 3, 2, 10).load({k: v.to(DEV) for k, v in bad.items()}, "m.")


# ----------------------------------------------------------------------------------------------- the attention

def _attention_fixture(dt, H, Dn, Dr, Dv, Lq, Lk, rot_dims, window, hidden=64, page=8, pages=80, max_pos=640, base=1e4, scale=0.3, std=0.3):
    from tokenmill_amd.cache import CacheManager
    from tokenmill_amd.cache.pool import CachePools
    from tokenmill_amd.engine.runner import ModelRunner
    from tokenmill_amd.parts import LatentAttention, RotaryEmbedding
    from test_gpu_parts import OneLayer
    rotary = RotaryEmbedding(Dr, base, max_pos, rotary_dim=rot_dims, interleaved=True) if rot_dims else None
    attn = LatentAttention(hidden, H, Dn, Dr, Dv, Lq, Lk, scale, 1e-5, rotary=rotary, window=window)
    w = {}
    for name, spec in attn.tensor_specs("a.").items():
        w[name] = q((torch.rand(spec.shape) + 0.5) if spec.init == "ones" else torch.randn(spec.shape) * std, dt)
    attn.load({k: v.to(dt).to(DEV) for k, v in w.items()}, "a.")
    attn.prepare(True)
    pools = CachePools(OneLayer(attn), pages, page, 4, dt, DEV)
    assert pools.v[0] is None and tuple(pools.k[0].shape[2:]) == (page, 1, Lk + Dr)
    manager = CacheManager(pools.group_specs, pages, page, 4)

    class Shell:
        device = torch.device(DEV)
        head = type("H", (), {"vocab": 10})()

        def program(self, views, tune=None):
            return None
    runner = ModelRunner.__new__(ModelRunner)
    ModelRunner.__init__(runner, Shell(), pools, max_pos)
    m = {"heads": H, "dim": Dn, "rot_dim": Dr, "vdim": Dv, "q_rank": Lq, "kv_rank": Lk, "scale": scale}
    if rot_dims:
        m["rot"] = {"base": base, "dims": rot_dims}
    if window:
        m["mask"] = {"size": window}
    return attn, w, m, pools, manager, runner


def _run_cuts(attn, pools, manager, runner, x, cuts, dt, rid="a"):
    from tokenmill_amd.engine.runner import StepEntry
    outs, start, rc = [], 0, None
    for n in cuts:
        if rc is None:
            rc = manager.allocate(rid, n)
        else:
            manager.append(rc, start + n)
        ctx, _ = runner.prepare([StepEntry(rc, start, [0] * n, [])])
        outs.append(attn.forward(x[start:start + n].to(dt).to(DEV), ctx, pools.views[0]).float().cpu())
        start += n
        manager.release_behind_window(rc, start)
    manager.free(rc)
    return torch.cat(outs)


@pytest.mark.parametrize("dt", DTS)
@pytest.mark.parametrize("H,Dn,Dr,Dv,Lq,Lk,rot,window", [(3, 20, 12, 24, 40, 36, 12, 24), (2, 16, 8, 8, 24, 72, 4, 50),
                                                         (5, 8, 4, 12, 56, 20, 4, None), (1, 28, 6, 40, 16, 44, 0, 7),
                                                         (4, 64, 32, 64, 96, 128, 32, 100), (2, 32, 32, 32, 64, 320, 32, 70),
                                                         (20, 16, 16, 16, 48, 264, 8, None)])
def test_latent_attention_whole_in_portions_and_token_by_token(dt, H, Dn, Dr, Dv, Lq, Lk, rot, window):
    # wide heads with wide weights give scores of several tens, where one rounding of a query moves the softmax by per cents
    attn, w, m, pools, manager, runner = _attention_fixture(dt, H, Dn, Dr, Dv, Lq, Lk, rot, window, std=0.3 if Dn < 64 and Lk < 256 else 0.1)
    torch.manual_seed(H * 10 + Dn)
    T = 150
    x = q(torch.randn(T, 64), dt)
    want, _ = L.latent_attention(x, torch.arange(T), m, w, "a.", 1e-5, dt)
    want = q(want, dt)
    for cuts in ([T], [2, 5, 40, 1, 1, 64, 37], [3] + [1] * (T - 3)):
        got = _run_cuts(attn, pools, manager, runner, x, cuts, dt)
        close(got, want, dt, f"cuts {cuts[:4]}..", bf16=2.0 ** -6)
    assert manager.num_free_pages == manager.num_pages


@pytest.mark.parametrize("dt", DTS)
@pytest.mark.parametrize("window,page,H", [(24, 8, 5), (17, 16, 20), (33, 4, 70), (64, 32, 16)])
def test_rows_just_inside_and_just_outside_the_window_show(dt, window, page, H):
    """Cached rows whose latent is one channel set to one (row j sets channel j % Lk) and whose scores are all equal: a
    token's result is then, channel by channel, how many visible rows set that channel, over the number of visible rows.
    One row too many or too few, at the window's far edge or at the token itself, changes both."""
    from tokenmill_amd.hip import ops
    Lk, Dr = 40, 8
    Dk = Lk + Dr
    n = 90
    pool = torch.zeros((n // page + 2, page, 1, Dk), dtype=dt, device=DEV)
    table = torch.randperm(n // page + 2)[: -(-n // page)].to(torch.int32)          # pages in no order
    flat = pool.view(-1, Dk)
    for j in range(n):
        flat[int(table[j // page]) * page + j % page, j % Lk] = 1.0
    qa = torch.zeros((n, H * Dk), dtype=dt, device=DEV)                              # every score is zero
    out = torch.empty((n, H * Lk), dtype=dt, device=DEV)
    tab = table.view(1, -1).to(DEV)
    ops.attn_latent(qa, out, pool, tab, ints([0] * n), ints(list(range(n))), H, Lk, Dk, 0.3, window)
    results = {"a wavefront a pair": out.float().cpu().view(n, H, Lk)}
    if dt == torch.bfloat16:
        # the matrix-unit kernel: the same rows as prompt tiles (the last one not full, one that starts inside a page), then as
        # single tokens
        assert ops.attn_latent_mfma_takes(dt, Lk, Dk, H)
        cuts = [(0, 16), (16, 16), (32, 5), (37, 16), (53, 16), (69, 16), (85, 5)]
        tiles = torch.tensor([[0, a, k, a] for a, k in cuts], dtype=torch.int32, device=DEV)
        tiled = torch.full_like(out, math.nan)
        ops.attn_latent_mfma(qa, tiled, pool, tab, tiles, ints([0] * n), ints(list(range(n))), 0, 0, H, Lk, Dk, 0.3, window)
        results["prompt tiles on the matrix unit"] = tiled.float().cpu().view(n, H, Lk)
        alone = torch.full_like(out, math.nan)
        ops.attn_latent_mfma(qa, alone, pool, tab, None, ints([0] * n), ints(list(range(n))), 0, n, H, Lk, Dk, 0.3, window, most_context=n)
        results["single tokens on the matrix unit"] = alone.float().cpu().view(n, H, Lk)
    for how, got in results.items():
        for p in range(n):
            lo = max(0, p - window + 1)
            want = torch.zeros(Lk)
            for j in range(lo, p + 1):
                want[j % Lk] += 1.0 / (p - lo + 1)
            for h in range(H):
                close(got[p, h], q(want, dt), dt, f"{how}: position {p} head {h}", bf16=2.0 ** -7)


@pytest.mark.parametrize("dt", DTS)
def test_one_far_row_among_hundreds_dominates(dt):
    """No window: a token near position 600 whose query points at one early row gets that row's latent back."""
    from tokenmill_amd.hip import ops
    H, Lk, Dr, page = 3, 24, 8, 16
    Dk = Lk + Dr
    n = 600
    torch.manual_seed(4)
    rows = q(torch.randn(n, Dk) * 0.1, dt)
    rows[13, Lk + 2] = 8.0                       # the far row stands out in one rotated channel
    pool = torch.zeros((n // page + 1, page, 1, Dk), dtype=dt, device=DEV)
    pool.view(-1, Dk)[:n] = rows.to(dt).to(DEV)
    table = torch.arange(n // page + 1, dtype=torch.int32).view(1, -1).to(DEV)
    qa = torch.zeros((2, H * Dk), dtype=dt, device=DEV)
    qa.view(2, H, Dk)[:, 1, Lk + 2] = 8.0        # head 1 asks for it
    out = torch.empty((2, H * Lk), dtype=dt, device=DEV)
    ops.attn_latent(qa, out, pool, table, ints([0, 0]), ints([598, 599]), H, Lk, Dk, 1.0, 0)
    got = out.float().cpu().view(2, H, Lk)
    close(got[:, 1], rows[13, :Lk].expand(2, Lk), dt, "the far row", bf16=2.0 ** -6)
    close(got[1, 0], q(rows[:600, :Lk].mean(0), dt), dt, "a head that asks for nothing sees the mean", bf16=2.0 ** -4)
    ops.attn_latent(qa, out, pool, table, ints([0, 0]), ints([598, 599]), H, Lk, Dk, 1.0, 586)
    got = out.float().cpu().view(2, H, Lk)
    close(got[0, 1], rows[13, :Lk], dt, "row 13 is the window's last for position 598", bf16=2.0 ** -6)
    assert float((got[1, 1] - rows[13, :Lk]).abs().max()) > 0.05, "row 13 is outside the window of position 599"
    if dt == torch.bfloat16:
        # the matrix unit: the two tokens alone (their rows in chunks over several blocks, merged), then as a prompt tile
        tile = torch.tensor([[0, 0, 2, 598]], dtype=torch.int32, device=DEV)
        for tiles, window in ((None, 0), (None, 586), (tile, 0), (tile, 586)):
            out.fill_(math.nan)
            ops.attn_latent_mfma(qa, out, pool, table, tiles, ints([0, 0]), ints([598, 599]), 0, 2, H, Lk, Dk, 1.0, window, most_context=600)
            got = out.float().cpu().view(2, H, Lk)
            close(got[0, 1], rows[13, :Lk], dt, "the far row, matrix unit", bf16=2.0 ** -6)
            if window:
                assert float((got[1, 1] - rows[13, :Lk]).abs().max()) > 0.05, "row 13 is outside the window of position 599"
            else:
                close(got[1, 1], rows[13, :Lk], dt, "the far row, matrix unit", bf16=2.0 ** -6)
                close(got[1, 0], q(rows[:600, :Lk].mean(0), dt), dt, "the mean, matrix unit", bf16=2.0 ** -4)


# ----------------------------------------------------------------------------------------------- whole models

@pytest.fixture(scope="module")
def models(tmp_path_factory):
    """name -> (folder, config, plain weights)."""
    from safetensors.torch import load_file
    from tokenmill_amd.weights.random_init import write_random_model
    out = {}
    for name, (cfg, seed, std, norm_std) in CASES.items():
        d = tmp_path_factory.mktemp(f"lusolix{name}")
        write_random_model(cfg, d, seed=seed, std=std, norm_std=norm_std)
        out[name] = (d, cfg, load_file(str(d / "model.safetensors")))
    return out


_plain_cache: dict = {}


def plain_logits(models, name, ids, dt):
    key = (name, tuple(ids), dt)
    if key not in _plain_cache:
        _, cfg, w = models[name]
        _plain_cache[key] = L.forward(cfg, w, ids, dt)
    return _plain_cache[key]


def check_rows(models, name, got, reqs, dt, what):
    """float32: 5e-5 of the largest logit. bfloat16: the engine may be twice as far from the plain bfloat16 run as that run
    is from the plain float32 run (both differ from it by the same roundings, falling differently), per request."""
    assert got, "no rows"
    for (rid, p), row in sorted(got.items()):
        want = plain_logits(models, name, reqs[rid], dt)
        if dt == torch.float32:
            bound = 2.5 * F32_REL * float(want.abs().max())
        else:
            bound = max(2.0 * float((want - plain_logits(models, name, reqs[rid], torch.float32)).abs().max()),
                        2.0 ** -7 * float(want.abs().max()))
        err = float((row - want[p]).abs().max())
        assert torch.isfinite(row).all() and err <= bound, f"{what}: request {rid} position {p}: {err:.3e} > {bound:.3e}"


def make_requests(name, lengths, seed):
    vocab = CASES[name][0]["vocab"]
    return {f"r{i}": random_ids(n, vocab, seed * 100 + i) for i, n in enumerate(lengths)}


def poison_freed_slots(session):
    slots, pools = session.manager.slots, session.pools
    plain_release = slots.release

    def release(slot):
        for t in pools.states.values():
            t[slot].fill_(math.nan)
        return plain_release(slot)

    slots.release = release


@pytest.mark.parametrize("dtype_name", ["float32", "bfloat16"])
@pytest.mark.parametrize("name,page", [("P", 16), ("Q", 8), ("R", 4), ("P", 64)])
def test_whole_decode_portions_mixed(models, name, page, dtype_name):
    from tokenmill_amd.replay import ReplaySession
    from test_gpu_replay import assert_all_given_back, mixed, poison_freed_pages, portions, prefill_then_decode, run_trace, whole
    dt = {"float32": torch.float32, "bfloat16": torch.bfloat16}[dtype_name]
    s = ReplaySession(models[name][0], dtype_name, 4 * 128, max_requests=4, page_size=page)
    taps = CASES[name][0]["canon"]["taps"]
    assert len(s.pools.states) == (len(CASES[name][0]["layers"]) if taps > 1 else 0) and all(v is None for v in s.pools.v)
    poison_freed_pages(s)
    poison_freed_slots(s)
    lengths = [1, 9, 26, 53, 120]
    reqs = make_requests(name, lengths, 1)
    got = run_trace(s, whole(reqs))
    assert len(got) == sum(lengths)
    check_rows(models, name, got, reqs, dt, "whole")
    assert_all_given_back(s)
    check_rows(models, name, run_trace(s, prefill_then_decode(reqs, tail=60)), reqs, dt, "prefill + decode")
    assert_all_given_back(s)
    steps = portions({k: v for k, v in reqs.items() if len(v) >= 2})
    assert min(len(e["tokens"]) for st in steps for e in st["entries"]) == 2
    check_rows(models, name, run_trace(s, steps), reqs, dt, "portions")
    assert_all_given_back(s)
    many = make_requests(name, [37, 64, 21, 90, 48, 33, 75, 18, 59, 44, 96, 27, 70, 52, 85, 40, 113, 66], 2)
    steps = mixed(many, seed=5)
    assert max(len(st["entries"]) for st in steps) == 4
    got = run_trace(s, steps)
    assert len(got) == sum(len(v) for v in many.values())
    check_rows(models, name, got, many, dt, "mixed")
    assert_all_given_back(s)
    assert s.manager.slots.num_free == s.manager.slots.num_slots


@pytest.mark.parametrize("dtype_name", ["float32", "bfloat16"])
def test_long_decoding_past_every_window_with_pages_given_back(models, dtype_name):
    """One token at a time from the third token on, to the model's last position: every window's far edge and every page
    edge is passed by decoded tokens; a windowed group gives the pages behind its window back on the way."""
    from tokenmill_amd.replay import ReplaySession
    from test_gpu_replay import assert_all_given_back, poison_freed_pages, run_trace
    dt = {"float32": torch.float32, "bfloat16": torch.bfloat16}[dtype_name]
    s = ReplaySession(models["P"][0], dtype_name, 320, max_requests=4, page_size=8)
    poison_freed_pages(s)
    n = 300
    ids = random_ids(n, 211, 77)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": ids[:3], "want": [0, 1, 2]}], "end": []}]
    steps += [{"step": p - 2, "entries": [{"id": "a", "tokens": [ids[p]], "want": [0]}], "end": ["a"] if p == n - 1 else []}
              for p in range(3, n)]
    got, held = {}, {}
    for st in steps:
        got.update(run_trace(s, [st]))
        if "a" in s.manager.live:
            for g, spec in enumerate(s.pools.groups):
                held[spec.window] = max(held.get(spec.window, 0), sum(p != -1 for p in s.manager.live["a"].tables[g]))
    check_rows(models, "P", got, {"a": ids}, dt, "long decoding")
    assert held[24] <= 24 // 8 + 1 and held[7] <= 2 and held[None] == -(-n // 8)
    assert_all_given_back(s)


def test_greedy_generation_through_the_engine_and_its_graphs(models):
    """The engine's own entry point: scheduler, chunked prefill, sampling, HIP graphs for the decode steps, decode steps
    queued ahead. Every token is the plain implementation's first choice at its place (or a near-tie with it), and all
    modes agree."""
    from tokenmill_amd import EngineConfig, LLMEngine, SamplingParams
    d, cfg, w = models["P"]
    prompts = [random_ids(n, 211, 500 + i) for i, n in enumerate([12, 3, 30, 7, 21, 16, 45, 25, 5, 18])]
    params = [SamplingParams(max_tokens=8 + 5 * (i % 4), ignore_eos=True) for i in range(len(prompts))]
    outs = {}
    for mode in ("eager", "graphs", "chunked", "ahead"):
        eng = LLMEngine(EngineConfig(model=str(d), dtype="float32", block_size=8, num_blocks=48, max_model_len=96,
                                     max_num_seqs=4, max_num_batched_tokens=32 if mode == "chunked" else 64, watermark=0.0,
                                     hip_graphs=mode != "eager", enable_chunked_prefill=mode == "chunked",
                                     pipeline_decode=mode == "ahead"))
        kinds = [type(p).__name__ for p in eng.runner.program.foreign_parts]
        assert kinds.count("LatentAttention") == 4 and kinds.count("TableRoutedExperts") == 2
        outs[mode] = eng.generate(prompts, params)
        if mode in ("graphs", "ahead"):
            assert eng.runner.graphs.stateful_ok and eng.runner.graphs.replays > 10
        assert (eng.stats["steps_ahead"] > 5) == (mode == "ahead")
        assert eng.cache.num_free_pages == eng.cache.num_pages
    tokens = {m: [list(o) for o in outs[m]] for m in outs}
    assert tokens["eager"] == tokens["graphs"] == tokens["chunked"] == tokens["ahead"]
    exempt = 0
    for prompt, toks in zip(prompts, tokens["eager"]):
        rows = L.forward(cfg, w, prompt + toks[:-1], torch.float32)[len(prompt) - 1:]
        for row, tok in zip(rows, toks):
            best = int(row.argmax())
            if tok != best:
                assert float(row[best] - row[tok]) <= 4 * F32_REL * float(row.abs().max()), "a token that is no near-tie"
                exempt += 1
    assert exempt <= 2


def test_command_line_generates_with_a_random_lusolix_model(tmp_path):
    import subprocess
    import sys
    from conftest import ROOT
    (tmp_path / "config.json").write_text(json.dumps(Q))
    r = subprocess.run([sys.executable, "-m", "tokenmill_amd.generate", "--random", str(tmp_path / "config.json"), "--prompt-ids",
                        "5,9,33,2;7,7", "--max-tokens", "6", "--max-model-len", "64", "--ignore-eos"], capture_output=True, text=True, cwd=ROOT, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    lines = [json.loads(ln) for ln in r.stdout.splitlines() if ln.startswith("{")]
    assert [len(ln["output_ids"]) for ln in lines] == [6, 6] and all(0 <= t < 150 for ln in lines for t in ln["output_ids"])
