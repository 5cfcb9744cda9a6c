"""The Kagalorn test cases, written once and run on a device: tests/test_kagalorn_cpu.py ("cpu") and
tests/test_kagalorn_gpu.py ("cuda", the HIP kernels)."""
from __future__ import annotations

import math

import torch

from oracle import kagalorn_oracle as oracle
from tests import _kagalorn as K

F64 = torch.float64


def _dt(name):
    return {"float32": torch.float32, "bfloat16": torch.bfloat16}[name]


# ------------------------------------------------------------------------------- single mechanisms
def case_hyper_connection_and_norm(device, dtype):
    from light_vllm_amd import mix_ops
    g = torch.Generator().manual_seed(1)
    for S, W, groups in ((3, 48, 3), (1, 40, 1), (4, 96, 2), (8, 64, 8)):
        T = 7
        x = torch.randn(T, S, W, generator=g)
        y = torch.randn(T, W, generator=g).to(_dt(dtype))
        mix, out_w, in_w = torch.randn(S, S, generator=g), torch.randn(S, generator=g), torch.randn(S, generator=g)
        nw = 1 + 0.3 * torch.randn(W, generator=g)
        xs = x.permute(1, 0, 2).to(F64)
        want_x = oracle.streams_write(xs, y.to(F64), mix.to(F64), out_w.to(F64))
        want_h = oracle.grouped_rms_norm(oracle.streams_read(want_x, in_w.to(F64)), nw.to(F64), groups, 1e-5)
        xd = x.clone().to(device)
        h = mix_ops.hc_update_norm(xd, y.to(device), mix.to(device), out_w.to(device), in_w.to(device), nw.to(device),
                                   groups, 1e-5, _dt(dtype))
        assert torch.allclose(xd.cpu().to(F64), want_x.permute(1, 0, 2), rtol=1e-5, atol=1e-5), "streams are f32"
        tol = 1e-5 if dtype == "float32" else 1e-2
        assert torch.allclose(h.cpu().to(F64), want_h, rtol=tol, atol=tol)
        # read-out alone (first sublayer) and write alone leave the other part untouched
        xd2 = x.clone().to(device)
        h0 = mix_ops.hc_update_norm(xd2, None, None, None, in_w.to(device), nw.to(device), groups, 1e-5, _dt(dtype))
        assert torch.equal(xd2.cpu(), x)
        want_h0 = oracle.grouped_rms_norm(oracle.streams_read(xs, in_w.to(F64)), nw.to(F64), groups, 1e-5)
        assert torch.allclose(h0.cpu().to(F64), want_h0, rtol=tol, atol=tol)


def case_clamped_glu(device, dtype):
    from light_vllm_amd import mix_ops
    g = torch.Generator().manual_seed(2)
    x = (3 * torch.randn(9, 2 * 20, generator=g)).to(_dt(dtype))
    for limit in (0.7, 2.0):
        got = mix_ops.clamped_glu(x.to(device), limit, 1.702).cpu().to(F64)
        gate, up = x[:, :20].to(F64).clamp(max=limit), x[:, 20:].to(F64).clamp(-limit, limit)
        want = gate * torch.sigmoid(1.702 * gate) * (up + 1)
        assert torch.allclose(got, want, rtol=1e-2 if dtype == "bfloat16" else 1e-5, atol=1e-2 if dtype == "bfloat16" else 1e-6)


def _delta_inputs(seed, T, G, H, D, Dv, taps, dtype):
    g = torch.Generator().manual_seed(seed)
    C = 2 * G * D + H * Dv
    ld = C + H * Dv + 2 * H
    proj = torch.randn(T, ld, generator=g).to(_dt(dtype))
    conv_w = 0.6 * torch.randn(C, taps, generator=g)
    A_log, dt_bias = 0.5 * torch.randn(H, generator=g), 0.5 * torch.randn(H, generator=g)
    return proj, conv_w, A_log, dt_bias, C


def _delta_oracle(proj, conv_w, A_log, dt_bias, G, H, D, Dv):
    T = proj.shape[0]
    C = 2 * G * D + H * Dv
    p = proj.to(F64)
    y = oracle.short_conv_silu(p[:, :C], conv_w.to(F64))
    q = oracle.unit(y[:, :G * D].view(T, G, D), 1e-6) * D ** -0.5
    k = oracle.unit(y[:, G * D:2 * G * D].view(T, G, D), 1e-6)
    v = y[:, 2 * G * D:].view(T, H, Dv)
    beta = torch.sigmoid(p[:, C + H * Dv:C + H * Dv + H])
    dec = torch.exp(-torch.exp(A_log.to(F64)) * torch.nn.functional.softplus(p[:, C + H * Dv + H:] + dt_bias.to(F64)))
    rep = H // G
    return torch.stack([oracle.delta_rule(q[:, h // rep], k[:, h // rep], v[:, h], beta[:, h], dec[:, h]) for h in range(H)], 1)


def case_delta_rule_portions(device, dtype):
    """The recurrence over one sequence cut into portions (also of one and two tokens) beside a second
    sequence in the same launches, slots used out of order; against the whole-sequence oracle."""
    from light_vllm_amd import mix_ops
    for (G, H, D, Dv, taps) in ((2, 4, 8, 12, 3), (1, 2, 40, 70, 1), (2, 2, 20, 6, 5), (1, 1, 130, 8, 2)):
        T0, T1 = 23, 9
        a = _delta_inputs(10 + D, T0, G, H, D, Dv, taps, dtype)
        b = _delta_inputs(20 + D, T1, G, H, D, Dv, taps, dtype)
        conv_w, A_log, dt_bias, C = a[1], a[2], a[3], a[4]
        want0 = _delta_oracle(a[0], conv_w, A_log, dt_bias, G, H, D, Dv)
        want1 = _delta_oracle(b[0], conv_w, A_log, dt_bias, G, H, D, Dv)
        slots = 3
        conv_buf = torch.full((slots, max(taps - 1, 1), C), 7.0).to(_dt(dtype)).to(device)   # stale values of an earlier owner
        conv_state = conv_buf[:, :taps - 1]
        state = torch.full((slots, H, D, Dv), 5.0, device=device)
        cuts0 = [0, 1, 3, 5, 12, 13, 21, 23]
        cuts1 = [0, 0, 0, 2, 2, 9, 9, 9]
        got0, got1 = [], []
        for s in range(len(cuts0) - 1):
            n0, n1 = cuts0[s + 1] - cuts0[s], cuts1[s + 1] - cuts1[s]
            lens, ctx, sl, rows = [n0], [cuts0[s]], [2], [a[0][cuts0[s]:cuts0[s + 1]]]
            if n1:
                lens.append(n1); ctx.append(cuts1[s]); sl.append(0); rows.append(b[0][cuts1[s]:cuts1[s + 1]])
            step = K.make_step(lens, ctx, sl, [[0]] * len(lens), device)
            proj = torch.cat(rows).to(device)
            qn, kn, v, beta, dec = mix_ops.delta_prep(proj, conv_w.to(device), conv_state, A_log.to(device),
                                                      dt_bias.to(device), step, G, H, D, Dv, taps, C + H * Dv,
                                                      proj[:, C + H * Dv + H:C + H * Dv + 2 * H], 1e-6)
            mix_ops.conv_state_update(proj, conv_state, step, C, taps)
            o = mix_ops.gated_delta_rule(qn, kn, v, beta, dec, state, step).cpu()
            got0.append(o[:n0])
            got1.append(o[n0:])
        tol = 2e-4 if dtype == "float32" else 3e-2
        for got, want in ((torch.cat(got0), want0), (torch.cat(got1), want1)):
            scale = want.abs().max().item()
            assert (got.to(F64) - want).abs().max().item() <= tol * scale, (G, H, D, Dv, taps)


def case_head_norm_gate(device, dtype):
    from light_vllm_amd import mix_ops
    g = torch.Generator().manual_seed(3)
    for H, Dv in ((4, 12), (2, 70), (1, 64)):
        o = torch.randn(5, H, Dv, generator=g)
        gate = torch.randn(5, H * Dv + 3, generator=g).to(_dt(dtype))
        w = 1 + 0.3 * torch.randn(Dv, generator=g)
        got = mix_ops.head_norm_gate(o.to(device), gate.to(device)[:, 3:], w.to(device), 1e-5, _dt(dtype)).cpu().to(F64)
        o64, g64 = o.to(F64), gate[:, 3:].to(F64).view(5, H, Dv)
        want = (o64 / torch.sqrt((o64 * o64).mean(-1, keepdim=True) + 1e-5) * w.to(F64) * g64 * torch.sigmoid(g64)).reshape(5, -1)
        tol = 1e-5 if dtype == "float32" else 1e-2
        assert torch.allclose(got, want, rtol=tol, atol=tol)


def _fill_cache(k, v, tables, page, num_pages, G, D, Dv, dtype, device):
    kc = torch.zeros(num_pages, page, G, D, dtype=_dt(dtype))
    vc = torch.zeros(num_pages, page, G, Dv, dtype=_dt(dtype))
    for j in range(k.shape[0]):
        kc[tables[j // page], j % page] = k[j].to(_dt(dtype))
        vc[tables[j // page], j % page] = v[j].to(_dt(dtype))
    return kc.to(device), vc.to(device)


def case_window_pool_beacons(device, dtype):
    """Keys far back, at page borders, just inside and just outside the window, and in pooled blocks
    that are just seen or not yet: a few beacon keys score far above the hundreds of others, so a
    window, block or page that is one off moves whole rows. Prompt-shaped launch (all positions at
    once), decode-shaped launch (single tokens of many contexts in one batch) and portions."""
    from light_vllm_amd import mix_ops
    for (H, G, D, Dv, window, P, page, L) in ((4, 2, 16, 8, 37, 5, 16, 300), (10, 1, 8, 70, 64, 16, 64, 333),
                                              (2, 2, 24, 4, 5, 21, 16, 120), (3, 3, 8, 8, 16, 0, 16, 90),
                                              # head sizes in multiples of 16: the matrix-core kernel in bf16
                                              (4, 2, 32, 16, 37, 5, 16, 300), (6, 2, 48, 32, 70, 12, 64, 410),
                                              (9, 1, 64, 80, 130, 7, 32, 333), (2, 2, 16, 16, 3, 0, 16, 90),
                                              (2, 1, 160, 144, 40, 9, 32, 200)):       # heads above 128: the wide instantiation
        g = torch.Generator().manual_seed(L)
        rep = H // G
        k = 0.05 * torch.randn(L, G, D, generator=g)
        v = torch.randn(L, G, Dv, generator=g)
        e = torch.zeros(D); e[1] = 1.0
        beacons = [0, 3, page - 1, page, 2 * page + 1, 50, L - window - 1]
        for j in beacons:
            if 0 <= j < L:
                k[j] = k[j] + 8.0 * e
        q = 0.3 * torch.randn(L, H, D, generator=g) + 4.0 * e
        k, v, q = (t.to(_dt(dtype)).to(torch.float32) for t in (k, v, q))     # what a cache of this dtype holds
        scale = 1.0
        want = torch.stack([oracle.window_pool_softmax_attention(q[:, h].to(F64), k[:, h // rep].to(F64),
                                                                 v[:, h // rep].to(F64), window, P, scale)
                            for h in range(H)], 1).reshape(L, H * Dv)
        # the test has teeth: a beacon just inside the window dominates its row, just outside it does not
        j = 50
        w_in = oracle.window_pool_softmax_attention(q[:, 0].to(F64), k[:, 0].to(F64), torch.eye(L, dtype=F64), window, 0, scale)
        assert w_in[j + window - 1, j] > 0.2 and w_in[j + window, j] == 0

        num_pages = -(-L // page) + 3
        perm = torch.randperm(num_pages, generator=g).tolist()
        table = perm[:-(-L // page)]
        kc, vc = _fill_cache(k, v, table, page, num_pages, G, D, Dv, dtype, device)
        pp = max(mix_ops.pooled_slots(page, P), 1)
        kp = torch.zeros(num_pages, pp, G, D, dtype=_dt(dtype), device=device)
        vp = torch.zeros(num_pages, pp, G, Dv, dtype=_dt(dtype), device=device)
        # pooled entries are made as the sequence grows, in portions that cut blocks and pages anywhere
        cuts = [0, 1, 2, 7, page + 3, 3 * page, 3 * page + 2, L]
        for a, b in zip(cuts[:-1], cuts[1:]):
            mix_ops.pool_update(kc, vc, kp, vp, K.make_step([b - a], [a], [0], [table], device), G, D, Dv, P)
        qd = q.reshape(L, H * D).to(_dt(dtype)).to(device)
        tol = 2e-4 if dtype == "float32" else 5e-2

        def check(got, rows, what):
            err = (got.cpu().to(F64) - want[rows]).abs().max().item()
            assert err <= tol * want.abs().max().item(), (what, H, G, D, Dv, window, P, page, err)

        got = mix_ops.window_pool_attention(qd, kc, vc, kp, vp, None, K.make_step([L], [0], [0], [table], device),
                                            H, G, D, Dv, window, P, scale, True)
        check(got, list(range(L)), "prompt")
        rows = sorted({i for j in beacons for i in (j, j + window - 1, j + window, j + window + P, j + window + 2 * P)
                       if 0 <= i < L} | {0, 1, L - 1} | set(range(L - 20, L)))
        step = K.make_step([1] * len(rows), rows, [0] * len(rows), [table] * len(rows), device)
        got = mix_ops.window_pool_attention(qd[rows].contiguous(), kc, vc, kp, vp, None, step, H, G, D, Dv, window, P, scale, True)
        check(got, rows, "decode")
        # few sequences: the matrix-core kernel then cuts each one's key tiles over several workgroups and merges
        few = rows[-3:]
        step = K.make_step([1] * len(few), few, [0] * len(few), [table] * len(few), device)
        got = mix_ops.window_pool_attention(qd[few].contiguous(), kc, vc, kp, vp, None, step, H, G, D, Dv, window, P, scale, True)
        check(got, few, "decode, few sequences")
        step = K.make_step([2], [L - 2], [0], [table], device)
        got = mix_ops.window_pool_attention(qd[L - 2:].contiguous(), kc, vc, kp, vp, None, step, H, G, D, Dv, window, P, scale, True)
        check(got, [L - 2, L - 1], "two tokens behind a long context")
        a, b = L // 3, L // 3 + 2       # a portion of two tokens in the middle, beside one that starts a sequence
        step = K.make_step([b - a, 5], [a, 0], [0, 1], [table, table], device)
        got = mix_ops.window_pool_attention(torch.cat([qd[a:b], qd[:5]]).contiguous(), kc, vc, kp, vp, None, step,
                                            H, G, D, Dv, window, P, scale, True)
        check(got, list(range(a, b)) + list(range(5)), "portions")


def case_sink_and_gate(device, dtype):
    """With all scores at zero the weights are 1 / (1 + n): the sink takes its share; without it 1 / n."""
    from light_vllm_amd import mix_ops
    H = G = 1; D, Dv, page, L, window = 8, 4, 16, 10, 4
    kc, vc = _fill_cache(torch.zeros(L, G, D), torch.ones(L, G, Dv), [0], page, 1, G, D, Dv, dtype, device)
    q = torch.randn(L, D).to(_dt(dtype)).to(device)
    step = K.make_step([L], [0], [0], [[0]], device)
    gate = torch.zeros(L, Dv, dtype=_dt(dtype), device=device)
    for sink, gated in ((True, False), (False, False), (True, True)):
        got = mix_ops.window_pool_attention(q, kc, vc, None, None, gate if gated else None, step, H, G, D, Dv, window, 0,
                                            1.0, sink).cpu().float()
        n = torch.tensor([min(i + 1, window) for i in range(L)], dtype=torch.float32)
        want = (n / (n + 1) if sink else torch.ones(L)) * (0.5 if gated else 1.0)
        assert torch.allclose(got, want[:, None].expand(L, Dv), atol=1e-2 if dtype == "bfloat16" else 1e-6)


def case_qk_norm_store(device, dtype):
    from light_vllm_amd import mix_ops
    g = torch.Generator().manual_seed(4)
    H, G, D, Dv, page = 3, 1, 8, 6, 16
    T = 21
    proj = torch.randn(T, H * D + G * D + G * Dv + 5, generator=g).to(_dt(dtype))
    qw, kw = 1 + 0.3 * torch.randn(H * D, generator=g), 1 + 0.3 * torch.randn(G * D, generator=g)
    kc = torch.zeros(4, page, G, D, dtype=_dt(dtype), device=device)
    vc = torch.zeros(4, page, G, Dv, dtype=_dt(dtype), device=device)
    table = [2, 0, 3]
    ctx = 14                      # the portion crosses from the first page into the second and third
    step = K.make_step([T], [ctx], [0], [table], device)
    pd = proj.to(device)
    a, b, c = H * D, H * D + G * D, H * D + G * D + G * Dv
    qn = mix_ops.qk_fullnorm_store(pd[:, :a], pd[:, a:b], pd[:, b:c], qw.to(device), kw.to(device), kc, vc, step,
                                   H, G, D, Dv, 1e-5).cpu().to(F64)
    p64 = proj.to(F64)
    tol = 1e-5 if dtype == "float32" else 1e-2
    wq = p64[:, :a] / torch.sqrt((p64[:, :a] ** 2).mean(-1, keepdim=True) + 1e-5) * qw.to(F64)
    wk = p64[:, a:b] / torch.sqrt((p64[:, a:b] ** 2).mean(-1, keepdim=True) + 1e-5) * kw.to(F64)
    assert torch.allclose(qn, wq, rtol=tol, atol=tol)
    for r in range(T):
        pos = ctx + r
        assert torch.allclose(kc.cpu()[table[pos // page], pos % page].reshape(-1).to(F64), wk[r], rtol=tol, atol=tol)
        assert torch.equal(vc.cpu()[table[pos // page], pos % page].reshape(-1), proj[r, b:c])


# ------------------------------------------------------------------------------------- the engine
def _model(tmp_path, cfg, seed):
    weights = oracle.random_weights(cfg, seed)
    return K.write_model(tmp_path / f"m{seed}", cfg, weights), weights


def _oracle_logits(cfg, weights, prompts):
    return {i: oracle.forward(cfg, weights, t) for i, t in prompts.items()}


def case_engine_schedules(device, dtype, tmp_path, cfg=None, seed=5):
    """Whole prompts, token-by-token decoding, portions down to two tokens and mixed batches of unequal
    requests give the logits of the whole-sequence oracle at every position: the first tokens, every
    window and block edge and page border included (pages of 16 tokens, windows and pools that do not
    divide them)."""
    cfg = cfg or K.CFG_MAIN
    model_dir, weights = _model(tmp_path, cfg, seed)
    prompts = {"a": K.tokens_for(cfg, 53, 1), "b": K.tokens_for(cfg, 21, 2), "c": K.tokens_for(cfg, 38, 3)}
    want = _oracle_logits(cfg, weights, prompts)
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
            if len(logits):
                err = K.rel_err(logits, want[i][:len(logits)])
                assert err <= K.TOL[dtype], (name, i, err)


def case_engine_reuse(device, dtype, tmp_path):
    """More requests than state slots and more tokens than pages: both are given back and used again,
    in another order, and a sequence that starts on a used slot and used pages starts from nothing."""
    cfg = K.CFG_MAIN
    model_dir, weights = _model(tmp_path, cfg, 6)
    prompts = {f"r{n}": K.tokens_for(cfg, length, 10 + n) for n, length in enumerate((30, 17, 33, 9, 26, 31))}
    want = _oracle_logits(cfg, weights, prompts)
    schedule = [[("r0", 30), ("r1", 10)], [("r1", 7), ("r2", 20)], [("r3", 9), ("r2", 13)], [("r4", 13)],
                [("r5", 15), ("r4", 13)], [("r5", 16)]]
    got = K.replay(model_dir, dtype, device, prompts, schedule, max_tokens=64, page=16, slots=2)   # 4 pages, 2 slots
    for i, logits in got.items():
        K.assert_close(logits, want[i], dtype, i)


def case_engine_long_decode(device, dtype, tmp_path):
    """Decoding far past every window: hundreds of single-token steps through state, pages and pooled blocks."""
    cfg = K.CFG_MAIN
    model_dir, weights = _model(tmp_path, cfg, 7)
    prompts = {"a": K.tokens_for(cfg, 140, 21)}
    want = _oracle_logits(cfg, weights, prompts)
    got = K.replay(model_dir, dtype, device, prompts, [[("a", 3)]] + [[("a", 1)]] * 137, max_tokens=192, page=16, slots=1)
    K.assert_close(got["a"], want["a"], dtype, "long decode")


def case_generate(device, tmp_path, enforce_eager=True):
    """Greedy generation through LLM.generate: the scheduler admits, cuts prompts into portions under a small
    token budget, mixes them with decoding sequences, preempts nothing it need not, and every completion is
    the oracle's greedy continuation."""
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


def case_generate_preemption(device, tmp_path):
    """A page pool too small for the sequences that run: the scheduler preempts from the tail, frees pages and
    state slot, and recomputes the preempted sequence from its first token later; completions do not change."""
    from light_vllm_amd.llm import LLM
    from light_vllm_amd.sampling_params import SamplingParams
    cfg = K.CFG_MAIN
    model_dir, weights = _model(tmp_path, cfg, 8)
    prompts = [K.tokens_for(cfg, n, 50 + n) for n in (27, 29, 14)]
    steps = 9
    llm = LLM(model_dir, dtype="float32", device=device, kvcache_block_size=16, max_num_seqs=3, max_cache_tokens=64,
              max_num_batched_tokens=32, max_model_len=64)
    preempted = []
    original = llm.scheduler.preempt
    llm.scheduler.preempt = lambda seq: (preempted.append(seq.seq_id), original(seq))[1]
    outs = llm.generate([list(p) for p in prompts], SamplingParams(temperature=0.0, max_tokens=steps, ignore_eos=True))
    assert preempted, "the case is meant to run out of pages"
    assert llm.scheduler.block_manager.num_free_blocks == 4 and llm.scheduler.state_slots.num_free == 3
    llm.exit()
    for p, out in zip(prompts, outs):
        seq = list(p)
        for _ in range(steps):
            seq.append(int(oracle.forward(cfg, weights, seq)[-1].argmax()))
        assert out["token_ids"] == seq[len(p):]
