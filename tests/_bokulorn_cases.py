"""The Bokulorn test cases, written once and run on a device: tests/test_bokulorn_cpu.py ("cpu", the
package's torch restatement of the kernels under the engine's host logic) and tests/test_bokulorn_gpu.py
("cuda", the HIP kernels)."""
from __future__ import annotations

import torch

from oracle import bokulorn_oracle as oracle
from tests import _bokulorn as K

F64 = torch.float64


def _dt(name):
    return {"float32": torch.float32, "bfloat16": torch.bfloat16}[name]


# ------------------------------------------------------------------------------- single mechanisms
def case_residual_norm(device, dtype):
    """One f32 residual: two sublayer outputs are added, the norm weight is applied as (offset + w)."""
    from light_vllm_amd import mix_ops
    g = torch.Generator().manual_seed(1)
    for T, W in ((7, 48), (3, 37), (5, 1000)):
        x = 5 * torch.randn(T, W, generator=g)
        y1, y2 = (torch.randn(T, W, generator=g).to(_dt(dtype)) for _ in range(2))
        w = 0.3 * torch.randn(W, generator=g)
        tol = 1e-5 if dtype == "float32" else 1e-2
        xd = x.clone().to(device)
        h = mix_ops.residual_add_norm(xd, y1.to(device), y2.to(device), w.to(device), 1.0, 1e-5, _dt(dtype))
        want_x = x.to(F64) + (y1.to(F64) + y2.to(F64))
        assert torch.allclose(xd.cpu().to(F64), want_x, rtol=1e-6, atol=1e-6), "the residual is f32"
        assert torch.allclose(h.cpu().to(F64), oracle.offset_rms_norm(want_x, w.to(F64), 1e-5), rtol=tol, atol=tol)
        xd = x.clone().to(device)                      # one output only; the norm alone leaves the residual untouched
        mix_ops.residual_add_norm(xd, y1.to(device), None, w.to(device), 1.0, 1e-5, _dt(dtype))
        assert torch.allclose(xd.cpu().to(F64), x.to(F64) + y1.to(F64), rtol=1e-6, atol=1e-6)
        xd = x.clone().to(device)
        h0 = mix_ops.residual_add_norm(xd, None, None, w.to(device), 1.0, 1e-5, _dt(dtype))
        assert torch.equal(xd.cpu(), x)
        assert torch.allclose(h0.cpu().to(F64), oracle.offset_rms_norm(x.to(F64), w.to(F64), 1e-5), rtol=tol, atol=tol)


def case_latent_prep_and_query(device, dtype):
    """Norms of both latents, the rotation of the positional parts at positions that continue a context
    across pages, rows of the cache by page table; a rotation over part of the positional entries and none."""
    from light_vllm_amd import mix_ops
    g = torch.Generator().manual_seed(2)
    for (H, Dn, Dr, dims, R, Rq, base) in ((3, 12, 8, 8, 24, 20, 5000.0), (1, 4, 6, 2, 70, 7, 100.0),
                                           (2, 8, 0, 0, 8, 8, 1.0), (5, 32, 16, 16, 32, 48, 10000.0)):
        page, ctx, T = 16, 29, 21                     # positions 29 .. 49: three pages
        table = [2, 0, 3, 1]
        ld = 3 + Rq + R + Dr + 2
        proj = torch.randn(T, ld, generator=g).to(_dt(dtype))
        qw, kw = 1 + 0.3 * torch.randn(Rq, generator=g), 1 + 0.3 * torch.randn(R, generator=g)
        inv_freq = mix_ops.rotary_inv_freq(max(dims, 2), base, device)
        cache = torch.zeros(5, page, R + Dr, dtype=_dt(dtype), device=device)
        step = K.make_step([T - 2, 2], [ctx, ctx + T - 2], [0, 1], [table, table], device)      # two portions, one sequence's rows
        cq = mix_ops.latent_prep(proj.to(device), 3, 3 + Rq, qw.to(device), kw.to(device), inv_freq, cache, step,
                                 Rq, R, Dr, dims, 1e-5).cpu().to(F64)
        p64 = proj.to(F64)
        pos = list(range(ctx, ctx + T))
        tol = 1e-5 if dtype == "float32" else 1e-2
        assert torch.allclose(cq, oracle.rms_norm(p64[:, 3:3 + Rq], qw.to(F64), 1e-5), rtol=tol, atol=tol)
        want_c = oracle.rms_norm(p64[:, 3 + Rq:3 + Rq + R], kw.to(F64), 1e-5)
        want_r = oracle.rotate(p64[:, 3 + Rq + R:3 + Rq + R + Dr], pos, dims, base) if Dr else p64[:, :0]
        for r in range(T):
            row = cache.cpu()[table[pos[r] // page], pos[r] % page].to(F64)
            assert torch.allclose(row, torch.cat([want_c[r], want_r[r]]), rtol=tol, atol=tol), (r, Dr)
        # queries: [absorbed part | rotated positional part] per head
        q = torch.randn(T, H * (Dn + Dr), generator=g).to(_dt(dtype))
        q_lat = torch.randn(H, T, R, generator=g).to(_dt(dtype))
        got = mix_ops.latent_q_finish(q.to(device), q_lat.to(device), inv_freq, step, H, Dn, Dr, R, dims).cpu().to(F64)
        got = got.view(T, H, R + Dr)
        for hh in range(H):
            assert torch.equal(got[:, hh, :R], q_lat[hh].to(F64))
            if Dr:
                want = oracle.rotate(q.to(F64).view(T, H, Dn + Dr)[:, hh, Dn:], pos, dims, base)
                assert torch.allclose(got[:, hh, R:], want, rtol=tol, atol=tol)


def _latent_rows(L, R, Dr, page, seed, dtype, device, beacons, strength=8.0):
    g = torch.Generator().manual_seed(seed)
    rows = 0.05 * torch.randn(L, R + Dr, generator=g)
    rows[:, :R] += torch.randn(L, R, generator=g) * 0.5 * (torch.arange(R) % 3 == 0)     # values worth telling apart
    e = torch.zeros(R + Dr); e[R + Dr - 1] = 1.0                                           # the beacon direction: last key entry
    for j in beacons:
        if 0 <= j < L:
            rows[j] = rows[j] + strength * e
    rows = rows.to(_dt(dtype)).to(torch.float32)
    num_pages = -(-L // page) + 3
    table = torch.randperm(num_pages, generator=g).tolist()[:-(-L // page)]
    cache = torch.zeros(num_pages, page, R + Dr, dtype=_dt(dtype))
    for j in range(L):
        cache[table[j // page], j % page] = rows[j].to(_dt(dtype))
    return rows, e, table, cache.to(device)


def case_latent_attention_beacons(device, dtype):
    """All heads attend to one cached row per token (keys: the whole row, values: its first entries) with
    plain causal softmax. A few beacon rows score far above the hundreds of others: the very first tokens,
    rows either side of page borders, one far back. Prompt-shaped, decode-shaped and portion-shaped launches."""
    from light_vllm_amd import mix_ops
    from light_vllm_amd.layers.latent_attention import NO_WINDOW
    for (H, R, Dr, page, L) in ((3, 24, 8, 16, 300), (1, 70, 6, 64, 333), (10, 9, 0, 16, 120),
                                (5, 32, 16, 16, 300), (4, 64, 0, 32, 410), (2, 160, 32, 64, 200),
                                (5, 320, 32, 64, 150)):              # a latent above 256: the vector kernel with four heads a workgroup
        beacons = [0, 1, page - 1, page, 2 * page + 1, 50]
        rows, e, table, cache = _latent_rows(L, R, Dr, page, L + H, dtype, device, beacons)
        g = torch.Generator().manual_seed(L)
        q = (0.3 * torch.randn(L, H, R + Dr, generator=g) + 4.0 * e).to(_dt(dtype)).to(torch.float32)
        scale = 0.7
        want = torch.stack([oracle.causal_softmax_attention(q[:, h].to(F64), rows.to(F64), rows[:, :R].to(F64), scale)
                            for h in range(H)], 1).reshape(L, H * R)
        # the test has teeth: the far beacon holds a good part of the weight of a late row
        s = (rows.to(F64) @ q[L - 1, 0].to(F64)) * scale
        assert torch.softmax(s, 0)[0] > 0.03          # against 1 / L for a key that does not stand out
        kc = cache.unsqueeze(2)
        vc = kc[..., :R]
        qd = q.reshape(L, H * (R + Dr)).to(_dt(dtype)).to(device)
        tol = 2e-4 if dtype == "float32" else 5e-2

        def run(step, qq):
            return mix_ops.window_pool_attention(qq.contiguous(), kc, vc, None, None, None, step, H, 1, R + Dr, R,
                                                 NO_WINDOW, 0, scale, has_sink=False)

        def check(got, idx, what):
            err = (got.cpu().to(F64) - want[idx]).abs().max().item()
            assert err <= tol * want.abs().max().item(), (what, H, R, Dr, page, err)

        check(run(K.make_step([L], [0], [0], [table], device), qd), list(range(L)), "prompt")
        idx = sorted({i for j in beacons for i in (j - 1, j, j + 1) if 0 <= i < L} | set(range(L - 20, L)))
        step = K.make_step([1] * len(idx), idx, [0] * len(idx), [table] * len(idx), device)
        check(run(step, qd[idx]), idx, "decode")
        few = idx[-3:]
        check(run(K.make_step([1] * 3, few, [0] * 3, [table] * 3, device), qd[few]), few, "decode, few sequences")
        check(run(K.make_step([2], [L - 2], [0], [table], device), qd[L - 2:]), [L - 2, L - 1], "two tokens behind a long context")
        a, b = page - 1, page + 1           # a portion of two tokens across a page border beside the start of a sequence
        step = K.make_step([b - a, 5], [a, 0], [0, 1], [table, table], device)
        check(run(step, torch.cat([qd[a:b], qd[:5]])), list(range(a, b)) + list(range(5)), "portions")


def case_softmax_without_sink(device, dtype):
    """Scores far below zero: without a sink the weights still sum to one (a running maximum that started at
    a sink's score of 0 would lose every term); with equal scores the result is the mean of the values."""
    from light_vllm_amd import mix_ops
    from light_vllm_amd.layers.latent_attention import NO_WINDOW
    for (R, Dr) in ((8, 4), (32, 16)):
        L, page, H = 70, 16, 2
        rows = torch.zeros(L, R + Dr)
        rows[:, R + Dr - 1] = 1.0
        rows[:, 0] = torch.arange(L, dtype=torch.float32) % 4
        cache = torch.zeros(5, page, R + Dr, dtype=_dt(dtype))
        for j in range(L):
            cache[j // page, j % page] = rows[j]
        kc = cache.to(device).unsqueeze(2)
        q = torch.zeros(L, H, R + Dr)
        q[:, :, R + Dr - 1] = -300.0
        step = K.make_step([L], [0], [0], [list(range(5))], device)
        got = mix_ops.window_pool_attention(q.reshape(L, -1).to(_dt(dtype)).to(device), kc, kc[..., :R], None, None, None,
                                            step, H, 1, R + Dr, R, NO_WINDOW, 0, 1.0, has_sink=False).cpu().float()
        want = torch.stack([rows[:i + 1, 0].mean() for i in range(L)])
        assert torch.allclose(got.view(L, H, R)[:, 0, 0], want, atol=2e-2 if dtype == "bfloat16" else 1e-5)
        one = K.make_step([1], [L - 1], [0], [list(range(5))], device)
        got1 = mix_ops.window_pool_attention(q[L - 1:].reshape(1, -1).to(_dt(dtype)).to(device), kc, kc[..., :R], None, None,
                                             None, one, H, 1, R + Dr, R, NO_WINDOW, 0, 1.0, has_sink=False).cpu().float()
        assert abs(got1.view(H, R)[1, 0].item() - want[-1].item()) <= (2e-2 if dtype == "bfloat16" else 1e-5)


def case_latent_out_gate(device, dtype):
    from light_vllm_amd import mix_ops
    g = torch.Generator().manual_seed(5)
    for H, Dv in ((3, 10), (1, 70), (4, 16)):
        T = 6
        o = torch.randn(H, T, Dv, generator=g).to(_dt(dtype))
        for per_channel in (False, True):
            gate = torch.randn(T, 2 + (H * Dv if per_channel else H), generator=g).to(_dt(dtype))
            got = mix_ops.latent_out_gate(o.to(device), gate.to(device)[:, 2:], per_channel).cpu().to(F64)
            s = torch.sigmoid(gate[:, 2:].to(F64))
            s = s.view(T, H, Dv) if per_channel else s.view(T, H, 1)
            want = (o.to(F64).permute(1, 0, 2) * s).reshape(T, H * Dv)
            tol = 1e-5 if dtype == "float32" else 1e-2
            assert torch.allclose(got, want, rtol=tol, atol=tol)


def case_channel_delta_portions(device, dtype):
    """The recurrence in which every key channel decays at its own rate, over one sequence cut into portions (also of
    one and two tokens) beside a second sequence in the same launches, on slots with stale contents."""
    from light_vllm_amd import mix_ops
    for (G, H, D, Dv, taps) in ((2, 4, 8, 12, 3), (1, 2, 40, 70, 1), (2, 2, 20, 6, 5), (1, 1, 130, 8, 2)):
        T0, T1 = 23, 9
        C = 2 * G * D + H * Dv
        ld = C + H + 3

        def inputs(seed, T):
            g = torch.Generator().manual_seed(seed)
            return torch.randn(T, ld, generator=g).to(_dt(dtype)), (2 * torch.randn(T, H * D, generator=g)).to(_dt(dtype))

        g = torch.Generator().manual_seed(D)
        conv_w = 0.6 * torch.randn(C, taps, generator=g)
        A_log, dt_bias = 0.5 * torch.randn(H, generator=g), 0.5 * torch.randn(H * D, generator=g)

        def want(proj, a):
            T = proj.shape[0]
            p = proj.to(F64)
            y = oracle.short_conv_silu(p[:, :C], conv_w.to(F64))
            q = oracle.unit(y[:, :G * D].view(T, G, D), 1e-6) * D ** -0.5
            k = oracle.unit(y[:, G * D:2 * G * D].view(T, G, D), 1e-6)
            v = y[:, 2 * G * D:].view(T, H, Dv)
            beta = torch.sigmoid(p[:, C:C + H])
            dec = torch.exp(-torch.exp(A_log.to(F64))[None, :, None] *
                            torch.nn.functional.softplus(a.to(F64) + dt_bias.to(F64)).view(T, H, D))
            rep = H // G
            return torch.stack([oracle.channel_delta_rule(q[:, h // rep], k[:, h // rep], v[:, h], beta[:, h], dec[:, h])
                                for h in range(H)], 1)

        (p0, a0), (p1, a1) = inputs(10 + D, T0), inputs(20 + D, T1)
        want0, want1 = want(p0, a0), want(p1, a1)
        slots = 3
        conv_buf = torch.full((slots, max(taps - 1, 1), C), 7.0).to(_dt(dtype)).to(device)
        conv_state = conv_buf[:, :taps - 1]
        state = torch.full((slots, H, D, Dv), 5.0, device=device)
        cuts0 = [0, 1, 3, 5, 12, 13, 21, 23]
        cuts1 = [0, 0, 0, 2, 2, 9, 9, 9]
        got0, got1 = [], []
        for s in range(len(cuts0) - 1):
            n0, n1 = cuts0[s + 1] - cuts0[s], cuts1[s + 1] - cuts1[s]
            lens, ctx, sl = [n0], [cuts0[s]], [2]
            rows, arows = [p0[cuts0[s]:cuts0[s + 1]]], [a0[cuts0[s]:cuts0[s + 1]]]
            if n1:
                lens.append(n1); ctx.append(cuts1[s]); sl.append(0)
                rows.append(p1[cuts1[s]:cuts1[s + 1]]); arows.append(a1[cuts1[s]:cuts1[s + 1]])
            step = K.make_step(lens, ctx, sl, [[0]] * len(lens), device)
            proj, a = torch.cat(rows).to(device), torch.cat(arows).to(device)
            qn, kn, v, beta, dec = mix_ops.delta_prep(proj, conv_w.to(device), conv_state, A_log.to(device),
                                                      dt_bias.to(device), step, G, H, D, Dv, taps, C, a, 1e-6,
                                                      decay_per_channel=True)
            assert dec.shape == (proj.shape[0], H, D)
            mix_ops.conv_state_update(proj, conv_state, step, C, taps)
            o = mix_ops.gated_delta_rule(qn, kn, v, beta, dec, state, step).cpu()
            got0.append(o[:n0])
            got1.append(o[n0:])
        tol = 2e-4 if dtype == "float32" else 3e-2
        for got, w in ((torch.cat(got0), want0), (torch.cat(got1), want1)):
            assert (got.to(F64) - w).abs().max().item() <= tol * w.abs().max().item(), (G, H, D, Dv, taps)


def case_channel_decay_acts_on_rows(device, dtype):
    """One key channel decays to nothing, the others keep everything: what was written along the first is
    gone at the next token, what was written along the others is still read."""
    from light_vllm_amd import mix_ops
    H = G = 1; D, Dv = 4, 3
    step = K.make_step([2], [0], [0], [[0]], device)
    kn = torch.tensor([[[1.0, 0, 0, 0]], [[0, 1.0, 0, 0]]], device=device)
    qn = torch.tensor([[[0.0, 0, 0, 0]], [[1.0, 1.0, 0, 0]]], device=device)
    v = torch.tensor([[[1.0, 2, 3]], [[10.0, 20, 30]]], device=device)
    beta = torch.ones(2, 1, device=device)
    dec = torch.ones(2, 1, D, device=device)
    dec[1, 0, 0] = 0.0
    state = torch.zeros(1, H, D, Dv, device=device)
    o = mix_ops.gated_delta_rule(qn, kn, v, beta, dec, state, step).cpu()
    assert torch.allclose(o[1, 0], torch.tensor([10.0, 20, 30]))
    dec[1, 0, 0] = 1.0
    o = mix_ops.gated_delta_rule(qn, kn, v, beta, dec, state, step).cpu()
    assert torch.allclose(o[1, 0], torch.tensor([11.0, 22, 33]))


def case_head_norm_gate_sigmoid(device, dtype):
    from light_vllm_amd import mix_ops
    g = torch.Generator().manual_seed(3)
    for H, Dv in ((4, 12), (2, 70)):
        o = torch.randn(5, H, Dv, generator=g)
        gate = torch.randn(5, H * Dv + 3, generator=g).to(_dt(dtype))
        w = 1 + 0.3 * torch.randn(Dv, generator=g)
        got = mix_ops.head_norm_gate(o.to(device), gate.to(device)[:, 3:], w.to(device), 1e-5, _dt(dtype), "sigmoid").cpu().to(F64)
        want = (oracle.rms_norm(o.to(F64), w.to(F64), 1e-5) * torch.sigmoid(gate[:, 3:].to(F64)).view(5, H, Dv)).reshape(5, -1)
        tol = 1e-5 if dtype == "float32" else 1e-2
        assert torch.allclose(got, want, rtol=tol, atol=tol)


def case_moe_route(device):
    """The correction moves the choice and not the weights; experts outside the kept groups are out even when
    every selection score inside them is negative; a block of experts is ranked by its top two; random cases against the oracle."""
    from light_vllm_amd import mix_ops

    def run(z, corr, top, groups, keep):
        ids, w, dense = mix_ops.moe_route(z.to(device), corr.to(device), top, groups, keep)
        return ids.cpu(), w.cpu(), dense.cpu()

    # the correction decides the choice, the weights are the plain scores
    z = torch.tensor([[2.0, 1.0, 0.0, -1.0]])
    ids, w, dense = run(z, torch.tensor([0.0, 0.0, 0.0, 5.0]), 2, 1, 1)
    assert sorted(ids[0].tolist()) == [0, 3]
    s = torch.sigmoid(z[0])
    assert torch.allclose(w[0].sum(), torch.tensor(1.0)) and abs(dense[0, 3] - s[3] / (s[0] + s[3])) < 1e-6
    # negative selection scores inside the one kept group still beat positive ones outside it
    z = torch.tensor([[-3.0, -4.0, 3.0, -9.0, 2.9, 2.8]])
    corr = torch.tensor([-1.0, -1.0, 0.0, 0.0, 0.0, 0.0])
    ids, w, dense = run(z, corr + torch.tensor([0, 0, -5.0, 0, -5.0, -5.0]), 2, 3, 1)
    assert sorted(ids[0].tolist()) == [0, 1], ids          # group 0: -0.95 - 0.98; group 1: -4.05 + 0; group 2: -4.05 - 4.06
    assert (dense[0, 2:] == 0).all()
    # a group with one very good expert loses against a group with two good ones
    z = torch.tensor([[6.0, -6.0, 1.5, 1.4]])
    ids, _, _ = run(z, torch.zeros(4), 1, 2, 1)
    assert ids[0].tolist() == [2]
    g = torch.Generator().manual_seed(6)
    for E, top, groups, keep in ((6, 2, 3, 2), (8, 3, 4, 2), (5, 1, 5, 2), (3, 3, 1, 1), (64, 6, 8, 3), (130, 8, 1, 1)):
        T = 33
        z = 2 * torch.randn(T, E, generator=g)
        corr = 0.5 * torch.randn(E, generator=g)
        ids, w, dense = run(z, corr, top, groups, keep)
        for t in range(T):
            chosen, weights = oracle.route(z[t].to(F64), corr.to(F64), top, groups, keep)
            assert ids[t].tolist() == chosen, (E, top, groups, keep, t)
            assert torch.allclose(w[t].to(F64), torch.tensor(weights, dtype=F64), atol=1e-6)
            assert torch.allclose(dense[t, chosen].to(F64), torch.tensor(weights, dtype=F64), atol=1e-6)
            assert int((dense[t] != 0).sum()) == top


def case_moe_ff(device, dtype):
    """The feed-forward module on its own weights against the expert-by-expert oracle: the masked form, and for
    sizes in multiples of 32 the gathered form (one token, a few, and enough for the large row tiles)."""
    from light_vllm_amd.layers import moe as moe_mod
    g = torch.Generator().manual_seed(7)
    cases = [(24, 12, 6, 2, 3, 2, 19, "masked"), (64, 32, 8, 3, 4, 2, 1, "gathered"), (64, 32, 8, 3, 4, 2, 19, "gathered"),
             (64, 32, 8, 3, 4, 2, 19, "masked"), (96, 64, 4, 1, 1, 1, 210, "gathered"), (32, 32, 16, 5, 1, 1, 333, "gathered"),
             (128, 64, 2, 1, 1, 1, 700, "gathered"), (192, 160, 3, 2, 1, 1, 500, "gathered"), (96, 96, 2, 2, 1, 1, 300, "gathered"),
             (64, 32, 8, 3, 4, 2, 19, "sorted"), (192, 160, 3, 2, 1, 1, 500, "sorted"), (32, 32, 16, 5, 1, 1, 333, "sorted")]
    for (W, Fe, E, top, groups, keep, T, kernel) in cases:
        if kernel in ("gathered", "sorted") and dtype != "bfloat16" and device != "cpu":
            continue                                  # the gathered kernels are bf16 only
        mlp = {"expert": {"ff": Fe}, "router": {"experts": E, "top": top, "groups": {"count": groups, "keep": keep}}}
        weights = {"router": 2 * torch.randn(E, W, generator=g) / W ** 0.5, "correction": 0.3 * torch.randn(E, generator=g)}
        for e in range(E):
            weights[f"e{e}.up"] = torch.randn(Fe, W, generator=g) / W ** 0.5
            weights[f"e{e}.down"] = torch.randn(W, Fe, generator=g) / Fe ** 0.5
        weights = {k: v.to(torch.bfloat16).float() for k, v in weights.items()}
        h = torch.randn(T, W, generator=g).to(_dt(dtype))
        old = torch.get_default_dtype()
        torch.set_default_dtype(_dt(dtype))
        try:
            moe = moe_mod.SparseMoE(W, Fe, E, top, groups, keep)
        finally:
            torch.set_default_dtype(old)
        with torch.no_grad():
            moe.router_weight.copy_(weights["router"])
            moe.correction.copy_(weights["correction"])
            for e in range(E):
                moe.up_weight[e * Fe:(e + 1) * Fe].copy_(weights[f"e{e}.up"])
                moe.down_weight[:, e * Fe:(e + 1) * Fe].copy_(weights[f"e{e}.down"])
        moe = moe.to(device)
        old_kernel, moe_mod.MOE_KERNEL = moe_mod.MOE_KERNEL, kernel
        try:
            with torch.inference_mode():
                got = moe(h.to(device)).cpu().to(F64)
        finally:
            moe_mod.MOE_KERNEL = old_kernel
        margins = [[] for _ in range(T)]
        want = oracle.moe_ff(h.to(F64), {k: v.to(F64) for k, v in weights.items()}, "", mlp, margins)
        rows = [t for t in range(T) if dtype == "float32" or not margins[t] or min(margins[t]) >= 1e-3]
        tol = 1e-4 if dtype == "float32" else 4e-2
        assert (got[rows] - want[rows]).abs().max().item() <= tol * want.abs().max().item(), (W, Fe, E, top, T, kernel)


# ------------------------------------------------------------------------------------- the engine
def _model(tmp_path, cfg, seed):
    weights = oracle.random_weights(cfg, seed)
    return K.write_model(tmp_path / f"m{seed}", cfg, weights), weights


def _oracle_logits(cfg, weights, prompts):
    return {i: oracle.forward(cfg, weights, t) for i, t in prompts.items()}


ROUTE_MARGIN = 0.03      # bf16 runs: a router decided by less than this (in score units) may choose otherwise after rounding


def _decided(cfg, weights, prompts, dtype):
    """id -> positions whose routing was no close call in the oracle (all of them for f32 runs). A token whose
    experts differ is another computation, not a rounding of this one, so bf16 comparisons leave those out."""
    out = {}
    for i, t in prompts.items():
        margins = []
        oracle.forward(cfg, weights, t, margins=margins)
        out[i] = [j for j, m in enumerate(margins) if dtype == "float32" or m >= ROUTE_MARGIN]
        assert len(out[i]) >= 0.3 * len(t), "too many close calls: pick another seed"
    return out


def case_layer_by_layer(device, tmp_path):
    """The f32 residual after every layer of a whole prompt, against the oracle: names the first layer that differs."""
    from light_vllm_amd.engine.trace_replay import TraceReplayer
    cfg = K.CFG_MAIN
    model_dir, weights = _model(tmp_path, cfg, 4)
    tokens = K.tokens_for(cfg, 27, 5)
    want = []
    oracle.forward(cfg, weights, tokens, want)
    rp = TraceReplayer(model_dir, "float32", 64, device=device, slots=2, page=16)
    try:
        model = rp.engine.model_runner.model
        model.layer_outputs = []
        rp.step([{"id": "a", "tokens": tokens, "want": []}], ["a"])
        got = [x.cpu() for x in model.layer_outputs]
    finally:
        rp.close()
    assert len(got) == len(cfg["layers"])
    for i, (a, b) in enumerate(zip(got, want)):
        assert (a.to(F64) - b).abs().max().item() <= 3e-4 * b.abs().max().item(), f"layer {i}"


def case_engine_schedules(device, dtype, tmp_path, cfg=None, seed=5):
    """Whole prompts, token-by-token decoding, portions down to two tokens and mixed batches of unequal
    requests give the logits of the whole-sequence oracle at every position: the first tokens and every
    page border included (pages of 16 tokens)."""
    cfg = cfg or K.CFG_MAIN
    model_dir, weights = _model(tmp_path, cfg, seed)
    prompts = {"a": K.tokens_for(cfg, 53, 1), "b": K.tokens_for(cfg, 21, 2), "c": K.tokens_for(cfg, 38, 3)}
    want = _oracle_logits(cfg, weights, prompts)
    decided = _decided(cfg, weights, prompts, dtype)
    schedules = {
        "whole": [[("a", 53)], [("b", 21)], [("c", 38)]],
        "decode": [[("a", 9)]] + [[("a", 1)]] * 44 + [[("b", 1)]] * 21,
        "portions": [[("a", n)] for n in (2, 3, 11, 2, 16, 1, 17, 1)] + [[("c", n)] for n in (16, 16, 2, 2, 2)],
        "mixed": [[("a", 5), ("b", 2)], [("a", 1), ("b", 7), ("c", 30)], [("c", 1), ("a", 20)], [("b", 12), ("a", 1)],
                  [("a", 26), ("c", 2)], [("c", 5)]],
    }
    for name, schedule in schedules.items():
        got = K.replay(model_dir, dtype, device, prompts, schedule, max_tokens=128, page=16, slots=3)
        for i, logits in got.items():
            rows = [j for j in decided[i] if j < len(logits)]
            if rows:
                err = K.rel_err(logits[rows], want[i][rows])
                assert err <= K.TOL[dtype], (name, i, err)


def case_engine_random_config(device, dtype, tmp_path, seed):
    """A drawn configuration, prompts of a few hundred tokens on pages of 64: whole, and cut into unequal portions beside
    single tokens of another request, against the oracle at every position."""
    cfg = K.random_config(seed)
    model_dir, weights = _model(tmp_path, cfg, seed)
    prompts = {"a": K.tokens_for(cfg, 210, seed), "b": K.tokens_for(cfg, 75, seed + 1)}
    want = _oracle_logits(cfg, weights, prompts)
    decided = _decided(cfg, weights, prompts, dtype)
    schedules = {
        "whole": [[("a", 210)], [("b", 75)]],
        "mixed": [[("a", 63)], [("a", 2), ("b", 70)], [("a", 100), ("b", 1)], [("a", 1), ("b", 1)], [("a", 44), ("b", 1)], [("b", 2)]],
    }
    for name, schedule in schedules.items():
        got = K.replay(model_dir, dtype, device, prompts, schedule, max_tokens=384, page=64, slots=2)
        for i, logits in got.items():
            rows = [j for j in decided[i] if j < len(logits)]
            err = K.rel_err(logits[rows], want[i][rows])
            assert err <= K.TOL[dtype], (seed, name, i, err, cfg)


def case_engine_reuse(device, dtype, tmp_path):
    """More requests than state slots and more tokens than pages: both are given back and used again,
    in another order, and a sequence that starts on a used slot and used pages starts from nothing."""
    cfg = K.CFG_MAIN
    model_dir, weights = _model(tmp_path, cfg, 6)
    prompts = {f"r{n}": K.tokens_for(cfg, length, 10 + n) for n, length in enumerate((30, 17, 33, 9, 26, 31))}
    want = _oracle_logits(cfg, weights, prompts)
    schedule = [[("r0", 30), ("r1", 10)], [("r1", 7), ("r2", 20)], [("r3", 9), ("r2", 13)], [("r4", 13)],
                [("r5", 15), ("r4", 13)], [("r5", 16)]]
    decided = _decided(cfg, weights, prompts, dtype)
    got = K.replay(model_dir, dtype, device, prompts, schedule, max_tokens=64, page=16, slots=2)   # 4 pages, 2 slots
    for i, logits in got.items():
        K.assert_close(logits[decided[i]], want[i][decided[i]], dtype, i)


def case_engine_long_decode(device, dtype, tmp_path):
    """Hundreds of single-token steps through the latent cache and the recurrent state."""
    cfg = K.CFG_MAIN
    model_dir, weights = _model(tmp_path, cfg, 7)
    prompts = {"a": K.tokens_for(cfg, 140, 21)}
    want = _oracle_logits(cfg, weights, prompts)
    got = K.replay(model_dir, dtype, device, prompts, [[("a", 3)]] + [[("a", 1)]] * 137, max_tokens=192, page=16, slots=1)
    K.assert_close(got["a"], want["a"], dtype, "long decode")


def case_generate(device, tmp_path, enforce_eager=True):
    """Greedy generation through LLM.generate: the scheduler admits, cuts prompts into portions under a small
    token budget, mixes them with decoding sequences, and every completion is the oracle's greedy continuation."""
    from light_vllm_amd.llm import LLM
    from light_vllm_amd.sampling_params import SamplingParams
    cfg = K.CFG_MAIN
    model_dir, weights = _model(tmp_path, cfg, 8)
    prompts = [K.tokens_for(cfg, n, 30 + n) for n in (19, 5, 33, 12, 8)]
    steps = 6
    llm = LLM(model_dir, dtype="float32", device=device, kvcache_block_size=16, max_num_seqs=3, max_cache_tokens=160,
              max_num_batched_tokens=24, long_prefill_token_threshold=10, max_model_len=64, enforce_eager=enforce_eager)
    assert llm.model_runner.enforce_eager == enforce_eager
    outs = llm.generate([list(p) for p in prompts], SamplingParams(temperature=0.0, max_tokens=steps, ignore_eos=True))
    llm.exit()
    for p, out in zip(prompts, outs):
        seq = list(p)
        for _ in range(steps):
            logits = oracle.forward(cfg, weights, seq)[-1]
            top2 = logits.topk(2).values
            assert (top2[0] - top2[1]).item() > 2e-4 * logits.abs().max().item(), "oracle tie: pick another seed"
            seq.append(int(logits.argmax()))
        assert out["token_ids"] == seq[len(p):]


def case_generate_bf16_graphs_like_eager(device, tmp_path):
    """bf16, sizes that take the matrix-core attention and the gathered experts: single-token steps replayed from
    hipGraphs (launch geometry fixed at its bound, padded rows) continue every prompt like eager steps do, wherever
    the oracle's choice of the next token is no close call."""
    from light_vllm_amd.llm import LLM
    from light_vllm_amd.sampling_params import SamplingParams
    cfg = K.CFG_WIDE
    model_dir, weights = _model(tmp_path, cfg, 12)
    prompts = [K.tokens_for(cfg, n, 70 + n) for n in (40, 9, 23)]
    steps = 8
    outs = {}
    for eager in (True, False):
        llm = LLM(model_dir, dtype="bfloat16", device=device, kvcache_block_size=16, max_num_seqs=4, max_cache_tokens=256,
                  max_num_batched_tokens=64, max_model_len=64, enforce_eager=eager)
        outs[eager] = [o["token_ids"] for o in llm.generate([list(p) for p in prompts],
                                                           SamplingParams(temperature=0.0, max_tokens=steps, ignore_eos=True))]
        llm.exit()
    compared = 0
    for p, a, b in zip(prompts, outs[True], outs[False]):
        seq = list(p)
        for x, y in zip(a, b):
            logits = oracle.forward(cfg, weights, seq)[-1]
            top2 = logits.topk(2).values
            if (top2[0] - top2[1]).item() < 0.05 * logits.std().item() or x != int(logits.argmax()):
                break                       # a close call (or bf16 already chose otherwise): the continuations part ways
            assert x == y, (seq[len(p):], a, b)
            compared += 1
            seq.append(x)
    assert compared >= steps, "too few decided tokens: pick another seed"
