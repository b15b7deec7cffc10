"""Rorevik on the GPU against the plain implementation (``plain_rorevik``): each mechanism's kernels alone, with inputs
made so that a fault shows (a far key whose score is capped, a write that must be recalled after hundreds of tokens, a
state that must survive a cut shorter than the convolution's window), then whole models under every cutting, batching,
page and slot reuse, long decoding, and greedy generation through the engine's own entry point."""
import json
import math
import os
from types import SimpleNamespace

import numpy as np
import pytest
import torch

import plain_rorevik as P
import tiny_rorevik as TR
from gpu_tools import DEV, attention_ctx, cut_steps, live_token_need, run_trace
from tiny_models import random_tokens

pytestmark = pytest.mark.gpu
DTYPES = ["float32", "bfloat16"]
TORCH = {"float32": torch.float32, "bfloat16": torch.bfloat16}
F64 = torch.float64


def randn(*shape, seed=0, scale=1.0):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed), dtype=F64) * scale


def close(got, ref, what, tol=2e-5):
    tol = tol * max(1.0, float(ref.abs().max()))
    err = float((got.double().cpu() - ref).abs().max())
    assert err <= tol, f"{what}: error {err:.3e} > {tol:.3e}"


def dev32(t):
    return t.float().to(DEV).contiguous()


def state_ctx(q_lens, slots):
    """The fields of a StepContext that the kernels of mixers with a state read."""
    q_start = np.zeros(len(q_lens) + 1, np.int32)
    np.cumsum(q_lens, out=q_start[1:])
    return SimpleNamespace(T=int(sum(q_lens)), R=len(q_lens), max_q_len=max(q_lens),
                           q_start=torch.from_numpy(q_start).to(DEV), slots=torch.tensor(slots, dtype=torch.int32, device=DEV))


def in_steps(seqs, cuts):
    """Steps over several sequences at once: ``cuts[name]`` are the portion sizes of sequence ``name`` (cycled); a step
    holds the next portion of every sequence that has tokens left.  Yields [(name, begin, end)]."""
    at = {n: 0 for n in seqs}
    k = 0
    while any(at[n] < seqs[n] for n in seqs):
        step = []
        for n in seqs:
            if at[n] < seqs[n]:
                size = min(cuts[n][k % len(cuts[n])], seqs[n] - at[n])
                step.append((n, at[n], at[n] + size))
                at[n] += size
        k += 1
        yield step


# ----------------------------------------------------------------------------- mechanisms alone
@pytest.mark.parametrize("taps,bias", [(1, True), (2, False), (3, True), (4, True), (5, False), (8, True)])
def test_convolution_whole_in_portions_and_in_slots_used_again(taps, bias):
    from photon_infer_amd import ops
    C = 70
    w, b = randn(C, taps, seed=1, scale=0.6), (randn(C, seed=2, scale=0.3) if bias else None)
    seqs = {"a": randn(150, C, seed=3), "b": randn(9, C, seed=4), "c": randn(67, C, seed=5)}
    want = {n: P.silu(P.causal_conv(u, w, b)) for n, u in seqs.items()}
    wd, bd = dev32(w), (dev32(b) if bias else None)
    state = torch.full((4, (taps - 1) * C + 5), 7.0, device=DEV)      # rows wider than needed, full of rubbish
    slot = {"a": 2, "b": 0, "c": 2}                                    # c takes a's slot afterwards
    for group, cuts in (({"a": 150, "b": 9}, {"a": [150], "b": [9]}), ({"a": 150, "b": 9}, {"a": [1, 2, 1, 64, 3, 65], "b": [2, 1]}),
                        ({"c": 67}, {"c": [1]}), ({"c": 67, "b": 9}, {"c": [66, 1], "b": [1, 1, 7]})):
        for n in group:
            state[slot[n], :(taps - 1) * C].zero_()                    # admission clears the slot's row
        got = {n: [] for n in group}
        for step in in_steps(group, cuts):
            x = torch.cat([seqs[n][i:j] for n, i, j in step])
            wide = torch.full((x.shape[0], C + 3), 9.0, device=DEV)    # the input as a column view of a wider tensor
            wide[:, 2:2 + C] = dev32(x)
            out = torch.empty((x.shape[0], C), device=DEV)
            ops.causal_conv_silu(out, wide[:, 2:2 + C], wd, bd, state_ctx([j - i for _, i, j in step], [slot[n] for n, _, _ in step]),
                                 state[:, :(taps - 1) * C])
            for (n, i, j), part in zip(step, torch.split(out, [j - i for _, i, j in step])):
                got[n].append(part)
        for n in group:
            close(torch.cat(got[n]), want[n], f"taps {taps}, {n} cut {cuts[n]}")
    assert bool((state[:, (taps - 1) * C:] == 7.0).all()) and bool((state[1] == 7.0).all()) and bool((state[3] == 7.0).all())


@pytest.mark.parametrize("sizes", [(2, 24, 16, 1), (4, 32, 32, 2), (3, 20, 12, 3), (1, 5, 100, 1), (2, 64, 128, 2), (6, 16, 3, 2)])
def test_state_space_recurrence_whole_in_portions_and_token_by_token(sizes):
    from photon_infer_amd import ops
    H, Pd, N, G = sizes
    T = {"a": 83, "b": 10}
    A_log, D, dt_bias = randn(H, seed=1, scale=0.5), randn(H, seed=2), randn(H, seed=3, scale=0.5)
    data, want = {}, {}
    for i, (n, t) in enumerate(T.items()):
        x, B, C, dt = randn(t, H, Pd, seed=10 + i), randn(t, G, N, seed=20 + i, scale=0.5), randn(t, G, N, seed=30 + i, scale=0.5), randn(t, H, seed=40 + i)
        data[n] = (torch.cat([x.reshape(t, -1), B.reshape(t, -1), C.reshape(t, -1)], dim=1), dt)
        want[n] = P.state_space_recurrence(x, B, C, P.softplus(dt + dt_bias), A_log, D)
    slot = {"a": 3, "b": 1}
    for cuts in ({"a": [83], "b": [10]}, {"a": [1], "b": [1]}, {"a": [2, 17, 1, 40], "b": [3, 2]}, {"a": [9], "b": [10]}):
        floats = ops.scan_state_floats(H, N, Pd)
        state = torch.zeros((4, floats + 3), device=DEV)
        got = {n: [] for n in T}
        for step in in_steps(T, cuts):
            xbc = dev32(torch.cat([data[n][0][i:j] for n, i, j in step]))
            dt = dev32(torch.cat([data[n][1][i:j] for n, i, j in step]))
            y = torch.empty((xbc.shape[0], H * Pd), device=DEV)
            ops.state_space_scan(y, xbc, dt, dev32(dt_bias), dev32(A_log), dev32(D), state_ctx([j - i for _, i, j in step], [slot[n] for n, _, _ in step]),
                                 state[:, :floats], H, Pd, N, G)
            for (n, i, j), part in zip(step, torch.split(y, [j - i for _, i, j in step])):
                got[n].append(part)
        for n in T:
            close(torch.cat(got[n]), want[n][0].reshape(T[n], -1), f"{sizes} {n} cut {cuts[n]}", 5e-5)
            close(ops.unpack_scan_state(state[slot[n]], H, N, Pd), want[n][1], f"{sizes} {n} state after {cuts[n]}", 5e-5)
        assert bool((state[0] == 0).all()) and bool((state[2] == 0).all())


def delta_inputs(t, H, G, d, dv, seed):
    q, k, v = randn(t, G, d, seed=seed), randn(t, G, d, seed=seed + 1), randn(t, H, dv, seed=seed + 2)
    return q, k, v, randn(t, H * d, seed=seed + 3), randn(t, H, seed=seed + 4)


def delta_plain(q, k, v, a, b, dt_bias, A_log, H, d):
    t = q.shape[0]
    decay = torch.exp(-torch.exp(A_log).view(1, H, 1) * P.softplus(a + dt_bias).view(t, H, d))
    return P.delta_recurrence(P.unit(q) * d ** -0.5, P.unit(k), v, torch.sigmoid(b), decay)


@pytest.mark.parametrize("sizes", [(4, 2, 16, 24), (4, 4, 32, 32), (3, 1, 20, 28), (1, 1, 48, 80), (5, 5, 8, 8), (2, 1, 128, 64), (2, 2, 3, 200)])
def test_delta_rule_whole_in_portions_and_token_by_token(sizes):
    from photon_infer_amd import ops
    H, G, d, dv = sizes
    T = {"a": 90, "b": 11}
    A_log, dt_bias = randn(H, seed=1, scale=0.5) - 1.0, randn(H * d, seed=2)
    data = {n: delta_inputs(t, H, G, d, dv, 100 * i) for i, (n, t) in enumerate(T.items())}
    want = {n: delta_plain(*data[n], dt_bias, A_log, H, d) for n in T}
    slot = {"a": 0, "b": 2}
    for cuts in ({"a": [90], "b": [11]}, {"a": [1], "b": [1]}, {"a": [2, 30, 1, 8, 9], "b": [4, 1]}, {"a": [7], "b": [11]}):
        state = torch.zeros((3, ops.scan_state_floats(H, d, dv)), device=DEV)
        got = {n: [] for n in T}
        for step in in_steps(T, cuts):
            cat = lambda idx: torch.cat([data[n][idx][i:j].reshape(j - i, -1) for n, i, j in step])
            qkv = dev32(torch.cat([cat(0), cat(1), cat(2)], dim=1))
            o = torch.empty((qkv.shape[0], H * dv), device=DEV)
            ops.delta_scan(o, qkv, dev32(cat(3)), dev32(dt_bias), dev32(A_log), dev32(cat(4)),
                           state_ctx([j - i for _, i, j in step], [slot[n] for n, _, _ in step]), state, H, G, d, dv, d ** -0.5, 1e-6)
            for (n, i, j), part in zip(step, torch.split(o, [j - i for _, i, j in step])):
                got[n].append(part)
        for n in T:
            close(torch.cat(got[n]), want[n][0].reshape(T[n], -1), f"{sizes} {n} cut {cuts[n]}", 5e-5)
            close(ops.unpack_scan_state(state[slot[n]], H, d, dv), want[n][1], f"{sizes} {n} state after {cuts[n]}", 5e-5)
        assert bool((state[1] == 0).all())


@pytest.mark.parametrize("decode", [False, True])
def test_a_write_is_recalled_after_hundreds_of_tokens_and_forgotten_by_its_channel_alone(decode):
    """Token 0 writes v0 under key e0 with beta 1.  600 tokens follow with keys in the other channels: with channel 0's
    decay at one the last token's query e0 reads v0 back whole; with three steps of decay one half on channel 0 alone it
    reads an eighth.  A state that is lost or mixed at a cut, or a decay on the wrong axis, shows at once."""
    from photon_infer_amd import ops
    H, d, dv, T = 2, 16, 24, 601
    big = 40.0                                              # sigmoid(40) = 1 in float32; softplus(-40) = 0: no decay
    g = torch.Generator().manual_seed(5)
    k = torch.zeros(T, d, dtype=F64)
    k[0, 0] = 3.0
    k[torch.arange(1, T), torch.randint(1, d, (T - 1,), generator=g)] = 2.0
    q = torch.zeros(T, d, dtype=F64); q[:, 0] = 5.0
    v = randn(T, H * dv, seed=6)
    b = torch.full((T, H), big, dtype=F64)
    A_log = torch.zeros(H, dtype=F64)
    dt_bias = torch.zeros(H * d, dtype=F64)
    for halvings in (0, 3):
        a = torch.full((T, H, d), -big, dtype=F64)
        a[300:300 + halvings, :, 0] = math.log(math.e ** math.log(2.0) - 1.0)    # softplus = ln 2: decay one half
        a = a.view(T, H * d)
        state = torch.zeros((2, ops.scan_state_floats(H, d, dv)), device=DEV)
        sizes = [T - 40] + [1] * 40 if decode else [64, 2, 200, 1, 3]
        outs, i, kk = [], 0, 0
        while i < T:
            n = min(sizes[kk % len(sizes)], T - i); kk += 1
            qkv = dev32(torch.cat([q[i:i + n], k[i:i + n], v[i:i + n]], dim=1))
            o = torch.empty((n, H * dv), device=DEV)
            ops.delta_scan(o, qkv, dev32(a[i:i + n]), dev32(dt_bias), dev32(A_log), dev32(b[i:i + n]), state_ctx([n], [1]), state, H, 1, d, dv, d ** -0.5, 1e-6)
            outs.append(o); i += n
        o = torch.cat(outs).double().cpu()
        close(o[-1], v[0] * d ** -0.5 / 2 ** halvings, f"recall after {T} tokens, {halvings} halvings", 1e-5)
        close(o[0], v[0] * d ** -0.5, "the read-out sees its own token's write", 1e-5)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("N,parts", [(48, 2), (96, 1), (60, 3), (1024, 4)])
def test_gate_then_norm_in_equal_parts(dtype, N, parts):
    from photon_infer_amd import ops
    T, eps, mult = 6, 1e-5, 0.9
    y, z, w = randn(T, N, seed=1, scale=3.0), randn(T, N, seed=2), randn(N, seed=3)
    v = y * P.silu(z)
    want = P.rms_norm(v.view(T, parts, N // parts), None, eps).reshape(T, N) * w * mult
    wide = torch.zeros((T, 2 * N + 4), device=DEV)         # z and y as column views of one projection
    wide[:, :N], wide[:, N + 4:] = dev32(z), dev32(y)
    out = torch.empty((T, N), dtype=TORCH[dtype], device=DEV)
    ops.gated_group_norm(out, wide[:, N + 4:], wide[:, :N], dev32(w), eps, parts, mult)
    close(out, want, f"gated norm {N} / {parts}", 2e-5 if dtype == "float32" else 1e-2)


@pytest.mark.parametrize("dtype", DTYPES)
def test_clamped_unit_with_biases_and_the_stream_bias(dtype):
    from photon_infer_amd import ops
    T, I, D, limit, alpha = 7, 50, 24, 1.5, 1.702
    gu = randn(T, 2 * I, seed=1, scale=3.0)                 # many values beyond the limit on both sides
    bg, bu, bd = randn(I, seed=2), randn(I, seed=3), randn(D, seed=4)
    g = torch.clamp(gu[:, :I] + bg, max=limit)
    u = torch.clamp(gu[:, I:] + bu, min=-limit, max=limit)
    want = g * torch.sigmoid(alpha * g) * (u + 1.0)
    assert bool((gu[:, :I] + bg > limit).any()) and bool((gu[:, :I] + bg < -limit).any()) and bool((gu[:, I:] + bu < -limit).any())
    x = randn(T, D, seed=5)
    xs = dev32(x)
    out = torch.empty((T, I), dtype=TORCH[dtype], device=DEV)
    ops.clamped_glu(out, dev32(gu), dev32(bg), dev32(bu), limit, alpha, xs, dev32(bd))
    close(out, want, "clamped unit", 2e-5 if dtype == "float32" else 1e-2)
    close(xs, x + bd, "stream bias")


@pytest.mark.parametrize("M,I,K", [(200, 96, 128), (129, 512, 320), (5, 96, 128), (300, 40, 64)])
def test_product_and_clamped_unit_in_one_kernel(M, I, K):
    """The gate | up product with the clamped unit as its epilogue (bfloat16, rows interleaved by 16, more rows than
    the weight-streaming products take) against the product and the unit's own kernel, and against plain arithmetic."""
    from photon_infer_amd import ops
    limit, alpha = 1.2, 1.702
    a = randn(M, K, seed=1).to(torch.bfloat16)
    wg, wu = randn(I, K, seed=2, scale=0.3).to(torch.bfloat16), randn(I, K, seed=3, scale=0.3).to(torch.bfloat16)
    bg, bu = randn(I, seed=4), randn(I, seed=5)
    g = torch.clamp(a.double() @ wg.double().T + bg, max=limit)
    u = torch.clamp(a.double() @ wu.double().T + bu, min=-limit, max=limit)
    want = g * torch.sigmoid(alpha * g) * (u + 1.0)
    if I % 16 == 0:
        pair = lambda x, y: torch.stack([x.view(I // 16, 16, -1), y.view(I // 16, 16, -1)], dim=1)
        w, b, block = pair(wg, wu).reshape(2 * I, K).contiguous(), pair(bg, bu).reshape(2 * I).contiguous(), 16
    else:
        w, b, block = torch.cat([wg, wu]).contiguous(), torch.cat([bg, bu]).contiguous(), 0
    ws = ops.KernelWorkspace(torch.device(DEV))
    ws.prepare(True)
    out = torch.empty((M, I), dtype=torch.bfloat16, device=DEV)
    ops.gemm_clamped_glu(out, a.to(DEV), w.to(DEV), dev32(b), limit, alpha, block, ws=ws)
    assert ws.counts["gated_epilogues"] == (1 if (block and M > 128) else 0)
    close(out, want, f"clamped unit behind a product of {M} rows", 1e-2)
    prev = ops.use_fast_kernels(False)
    try:
        slow = torch.empty_like(out)
        ops.gemm_clamped_glu(slow, a.to(DEV), w.to(DEV), dev32(b), limit, alpha, block)
    finally:
        ops.use_fast_kernels(prev)
    close(slow, want, "the same on the general kernels", 1e-2)


def test_embedding_scaled_with_learned_positions():
    from photon_infer_amd import ops
    V, D, Pn = 50, 36, 20
    table, pos = randn(V, D, seed=1).to(torch.bfloat16), randn(Pn, D, seed=2).to(torch.bfloat16)
    ids = torch.tensor([3, 49, 0, 7], dtype=torch.int32)
    where = torch.tensor([0, 19, 5, 5], dtype=torch.int32)
    out = torch.empty((4, D), device=DEV)
    ops.embedding(out, table.to(DEV), ids.to(DEV), 7.5, pos.to(DEV), where.to(DEV))
    close(out, table.double()[ids.long()] * 7.5 + pos.double()[where.long()], "embedding", 1e-6)
    ops.embedding(out, table.to(DEV), ids.to(DEV), 1.0, pos.to(DEV), torch.tensor([0, 20, 5, 5], dtype=torch.int32, device=DEV))
    assert bool(torch.isnan(out[1]).all()) and not bool(torch.isnan(out[0]).any())       # a position beyond the table is loud


def paged(seq_lens, page):
    """A block table whose pages are dealt out of order, and the pool's size."""
    blocks = [-(-n // page) for n in seq_lens]
    order = torch.randperm(sum(blocks) + 2, generator=torch.Generator().manual_seed(3)).tolist()
    table = torch.full((len(seq_lens), max(blocks)), -1, dtype=torch.int32)
    it = iter(order)
    for r, nb in enumerate(blocks):
        for bidx in range(nb):
            table[r, bidx] = next(it)
    return table.to(DEV), sum(blocks) + 2


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("sizes", [(4, 2, 16, 32, 8), (4, 1, 64, 64, 64), (6, 3, 24, 12, 10), (3, 3, 40, 40, 0), (2, 2, 128, 128, 64)])
def test_attention_rotation_capped_scores_and_values_of_another_width(dtype, sizes):
    """Neighbouring pairs of the first dims rotated, keys and values into pages, scores capped, a factor on the output:
    a prompt whole, then its last tokens alone over the cache, against the plain attention.  One key far back has a
    score that dwarfs all others: uncapped it would take all the weight."""
    from photon_infer_amd import ops
    from photon_infer_amd.parts.rope import rope_frequencies
    H, G, d, dv, rot = sizes
    T, page, cap, scale, mult, base = 333, 16, 6.0, 0.17, 1.3, 1000.0
    q, k, v = randn(T, H, d, seed=1), randn(T, G, d, seed=2), randn(T, G, dv, seed=3)
    k[7] *= 6.0                                            # far back, and loud
    q[-5:] *= 3.0
    rq = torch.stack([P.rotate_interleaved(q[t], t, rot, base) for t in range(T)]) if rot else q
    rk = torch.stack([P.rotate_interleaved(k[t], t, rot, base) for t in range(T)]) if rot else k
    tdt = TORCH[dtype]
    rnd = (lambda t: t.to(tdt).double())
    want = P.attend(rnd(rq), rnd(rk), rnd(v), scale, cap) * mult
    uncapped = P.attend(rnd(rq), rnd(rk), rnd(v), scale, None) * mult
    assert float((want[-1] - uncapped[-1]).abs().max()) > 0.05          # the cap matters here
    table, pages = paged([T], page)
    kc = torch.zeros((pages, G, page, d), dtype=tdt, device=DEV)
    vc = torch.zeros((pages, G, dv, page), dtype=tdt, device=DEV)
    rotary = (rope_frequencies(rot, base).float().to(DEV), rot, True) if rot else None
    tol = 3e-5 if dtype == "float32" else 3e-2
    for q_len in (T, 1, 4):
        ctx = attention_ctx([q_len], [T], tdt)
        rows = slice(T - q_len, T)
        qd = q[rows].reshape(q_len, -1).to(tdt).to(DEV).contiguous()
        kd, vd_ = k[rows].reshape(q_len, -1).to(tdt).to(DEV).contiguous(), v[rows].reshape(q_len, -1).to(tdt).to(DEV).contiguous()
        ops.rope_kv_write(qd, kd, vd_, ctx.positions, ctx.req_of_token, rotary, H, G, d, kc, vc, table, page, value_dim=dv)
        out = torch.empty((q_len, H * dv), dtype=tdt, device=DEV)
        ops.paged_attention(out, qd, kc, vc, table, ctx, H, G, d, page, scale, 0, None, value_dim=dv, softcap=cap, out_scale=mult)
        close(out, want[rows].reshape(q_len, -1), f"{sizes} {q_len} tokens ending the sequence", tol)
    if dtype == "float32":      # what the pages hold: rotated keys by position, values transposed
        p0 = int(table[0, 1])
        close(kc[p0, :, 3], rk[19], "rotated key in its page", 1e-5)
        close(vc[p0, :, :, 3], v[19], "value in its page", 1e-6)


# ----------------------------------------------------------------------------- whole models
@pytest.fixture(scope="module")
def model_dirs(tmp_path_factory):
    base = tmp_path_factory.mktemp("rorevik")
    return {name: TR.make_model_dir(base, name, ranks_in_config=(name != "C")) for name in TR.ALL}


_plain = {}


def plain_logits(model_dir, tokens, emulate=False):
    key = (model_dir, tuple(tokens), emulate)
    if key not in _plain:
        cfg, W = P.read_model_folder(model_dir)
        _plain[key] = P.forward(cfg, W, list(tokens), act_round=P.bf16_round if emulate else None).float()
    return _plain[key]


def runner_for(model_dir, name, dtype, max_tokens):
    from photon_infer_amd.engine.replay import make_runner
    return make_runner(model_dir, dtype, max(max_tokens, 64), TR.ALL[name][1]["block_size"])


def check(got, model_dir, reqs, dtype, what):
    assert got, "no logits came back"
    for rid, toks in reqs.items():
        ref = plain_logits(model_dir, toks)
        if dtype == "float32":
            tol = 1e-4 * max(1.0, float(ref.abs().max()))
        else:       # three times what rounding activations to bfloat16 does to the plain implementation itself
            tol = 3.0 * float((plain_logits(model_dir, toks, True) - ref).abs().max())
        over = []
        for p in range(len(toks)):
            assert (rid, p) in got, f"{what}: logits of {rid} position {p} are missing"
            err = float((got[(rid, p)] - ref[p]).abs().max())
            assert err <= 5.0 * tol, f"{what}: {rid} position {p}: error {err:.3e} > {tol:.3e} (first wrong position)"
            if err > tol:
                over.append(p)
        # The state-space mixer normalises its gated output in parts: where a part of some twenty values happens to be
        # small at one token, rounding noise (which differs between a batch's kernels and a single request's) is blown
        # up to full size there (measured: 5e-5 before the norm, 1.4e-4 behind it, at one token of 120).  Such positions
        # are rare and stay within five times the bound; a fault of cache, state or batch is a hundred times larger.
        assert len(over) <= max(1, len(toks) // 50), f"{what}: {rid}: positions {over} are over {tol:.3e}"


LENGTHS = {"A": [1, 26, 90], "B": [3, 130, 210], "C": [2, 30, 75], "D": [2, 45, 100]}


def requests_for(name, seed=0):
    vocab = TR.ALL[name][0]["vocab"]
    return {f"r{i}": random_tokens(n, vocab, seed * 100 + i) for i, n in enumerate(LENGTHS[name])}


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", list(TR.ALL))
def test_whole_prompts_and_every_layer_runs_stream(name, dtype, model_dirs, tmp_path):
    reqs = requests_for(name)
    steps = []
    for rid, toks in reqs.items():
        steps += cut_steps(rid, toks, [len(toks)], first_step=len(steps))
    runner = runner_for(model_dirs[name], name, dtype, live_token_need(steps))
    check(run_trace(runner, steps, str(tmp_path)), model_dirs[name], reqs, dtype, "whole")
    if dtype == "float32":         # the stream after every layer run (a looped layer counts each time), for the longest request
        from photon_infer_amd import ops
        from photon_infer_amd.engine.step import StepEntry
        toks = reqs["r2"]
        cfg, W = P.read_model_folder(model_dirs[name])
        want, got = [], []
        P.forward(cfg, W, toks, streams=want)
        for blk in runner.model.blocks:
            def wrapped(x, ctx, cache, f=blk.forward):
                f(x, ctx, cache)
                ops.materialize(x, ctx.workspace)
                got.append(x.detach().double().cpu())
            blk.forward = wrapped
        runner.admit("s")
        runner.step([StepEntry("s", toks, [])])
        assert len(got) == len(want) == len(P.run_order(cfg))
        for i, (g, w) in enumerate(zip(got, want)):
            close(g, w, f"stream after layer run {i}", 1e-4)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", list(TR.ALL))
def test_prefill_then_token_by_token_and_all_token_by_token(name, dtype, model_dirs, tmp_path):
    reqs = requests_for(name, seed=1)
    steps = []
    for rid, toks in reqs.items():
        head = max(0, len(toks) - 40)
        sizes = ([head] if head else []) + [1] * (len(toks) - head)
        steps += cut_steps(rid, toks, sizes, first_step=len(steps))
    steps += cut_steps("all", reqs["r1"], [1], first_step=len(steps))
    runner = runner_for(model_dirs[name], name, dtype, live_token_need(steps))
    check(run_trace(runner, steps, str(tmp_path)), model_dirs[name], dict(reqs, all=reqs["r1"]), dtype, "decoding")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", list(TR.ALL))
@pytest.mark.parametrize("sizes", [[2], [7, 2, 31, 1, 3], [64, 5], [17]])
def test_portions_of_changing_size(name, dtype, sizes, model_dirs, tmp_path):
    reqs = {"r2": requests_for(name, seed=2)["r2"]}
    steps = cut_steps("r2", reqs["r2"], sizes)
    runner = runner_for(model_dirs[name], name, dtype, live_token_need(steps))
    check(run_trace(runner, steps, str(tmp_path)), model_dirs[name], reqs, dtype, f"portions {sizes}")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", list(TR.ALL))
def test_mixed_batches_with_pages_and_slots_used_again(name, dtype, model_dirs, tmp_path):
    """Seven unequal requests through four slots: portions of some beside single tokens of others; a request may sit
    out a step; a finished request's pages and slot go to the next one.  Each must come out as it does alone."""
    vocab = TR.ALL[name][0]["vocab"]
    lengths = [70, 33, 5, 120, 64, 18, 91]
    reqs = {f"m{i}": random_tokens(n, vocab, 50 + i) for i, n in enumerate(lengths)}
    rng = np.random.default_rng(7)
    waiting, live, at, steps = list(reqs), [], {}, []
    while waiting or live:
        while waiting and len(live) < 4:
            live.append(waiting.pop(0))
            at[live[-1]] = 0
        entries, end = [], []
        for rid in list(live):
            left = len(reqs[rid]) - at[rid]
            if len(live) > 1 and rng.random() < 0.2:
                continue                               # sits this step out
            n = 1 if left <= 12 else int(min(left - 12, rng.choice([2, 3, 16, 29, 40])))
            entries.append({"id": rid, "tokens": reqs[rid][at[rid]:at[rid] + n], "want": list(range(n))})
            at[rid] += n
            if at[rid] == len(reqs[rid]):
                end.append(rid)
                live.remove(rid)
        if entries:
            steps.append({"step": len(steps), "entries": entries, "end": end})
    runner = runner_for(model_dirs[name], name, dtype, live_token_need(steps))
    assert runner.cache.max_slots == 4
    check(run_trace(runner, steps, str(tmp_path)), model_dirs[name], reqs, dtype, "mixed")
    assert all(g.pool.num_allocated == 0 for g in runner.cache.groups)


@pytest.mark.parametrize("name", ["A", "D"])
def test_long_decoding_keeps_its_state(name, model_dirs, tmp_path):
    """250 tokens one by one after a portion of three: the states carry everything from step to step."""
    vocab = TR.ALL[name][0]["vocab"]
    toks = random_tokens(250, vocab, 9)
    steps = cut_steps("long", toks, [3] + [1] * 247)
    runner = runner_for(model_dirs[name], name, "float32", 256)
    check(run_trace(runner, steps, str(tmp_path)), model_dirs[name], {"long": toks}, "float32", "long decoding")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", list(TR.ALL))
def test_greedy_generation_through_the_engine(name, dtype, model_dirs):
    """The engine's own entry point, scheduler, sampling and decode steps: unequal prompts at once, more requests than
    slots, prompts longer than a portion; every request must generate what the plain implementation generates alone."""
    from photon_infer_amd.engine import ContinuousBatchEngine, EngineOptions
    cfg, W = P.read_model_folder(model_dirs[name])
    vocab = cfg["vocab"]
    prompts = [random_tokens(n, vocab, 70 + i) for i, n in enumerate([5, 41, 18, 70, 2])]
    engine = ContinuousBatchEngine(model_dirs[name], EngineOptions(dtype=dtype, block_size=TR.ALL[name][1]["block_size"], max_batch=3,
                                                                   max_cache_tokens=1024, chunk_size=32, max_model_len=200))
    got = engine.generate(prompts, max_new_tokens=10)
    for prompt, out in zip(prompts, got):
        want = P.greedy(cfg, W, prompt, 10)
        if dtype == "float32":
            assert list(out) == want
        else:       # bfloat16: a near tie may fall the other way; everything before the first difference must agree and the
            # differing token must be a close second of the plain logits
            for i, (a, b) in enumerate(zip(out, want)):
                if a != b:
                    lg = P.forward(cfg, W, prompt + want[:i])[-1]
                    assert float(lg[b] - lg[a]) < 0.05 * float(lg.std()), f"token {i}: {a} instead of {b}"
                    break


def test_command_line_and_replayed_decode_steps(model_dirs, tmp_path):
    """The framework's commands serve the design as they serve its others (from a folder, and from a bare configuration
    with random weights); and decode steps replayed as HIP graphs give the tokens of eager steps, with new requests'
    prompts in between and states in slots that are used again."""
    import subprocess
    from photon_infer_amd.engine import ContinuousBatchEngine, EngineOptions
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    cfg, W = P.read_model_folder(model_dirs["A"])
    prompt = random_tokens(9, cfg["vocab"], 81)
    want = P.greedy(cfg, W, prompt, 5)
    proc = subprocess.run([os.path.join(root, "bin", "llama_infer"), model_dirs["A"], "--dtype", "fp32", "--prompt-ids",
                           ",".join(map(str, prompt)), "--max-new-tokens", "5", "--temperature", "0", "--ignore-eos"],
                          capture_output=True, text=True, timeout=300)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert "Architecture: Rorevik" in proc.stdout and f"Generated ids: {','.join(map(str, want))}" in proc.stdout
    (tmp_path / "cfg").mkdir()
    json.dump(TR.TINY_D, open(tmp_path / "cfg" / "config.json", "w"))
    proc = subprocess.run([os.path.join(root, "bin", "llama_infer"), str(tmp_path / "cfg"), "--random-weights", "--seed", "3",
                           "--prompt-ids", "5,6,7", "--max-new-tokens", "4", "--ignore-eos"], capture_output=True, text=True, timeout=300)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert "Generated ids:" in proc.stdout
    # the trace replay as a command, from the folder
    toks = random_tokens(12, cfg["vocab"], 82)
    lines = "\n".join(json.dumps(s) for s in cut_steps("x", toks, [5, 1, 6])) + "\n"
    proc = subprocess.run([os.path.join(root, "bin", "trace_run"), "--model", model_dirs["A"], "--dtype", "float32", "--out", str(tmp_path / "out"),
                           "--max-tokens", "64"], input=lines, capture_output=True, text=True, timeout=300)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert [l for l in proc.stdout.split("\n") if l.startswith("done")] == ["done 0", "done 1", "done 2"]
    last = torch.from_numpy(np.fromfile(tmp_path / "out" / "2.f32", dtype="<f4").reshape(6, cfg["vocab"]))
    close(last, plain_logits(model_dirs["A"], toks)[6:].double(), "trace_run", 1e-4)

    prompts = [random_tokens(n, cfg["vocab"], 90 + n) for n in (3, 40, 17, 9, 26)]

    def run(use_graphs):
        eng = ContinuousBatchEngine(model_dirs["A"], EngineOptions(dtype="bfloat16", block_size=16, max_batch=3, max_cache_tokens=1024,
                                                                   chunk_size=8, max_step_tokens=24, max_model_len=200, use_graphs=use_graphs))
        assert eng.runner.graph_safe
        out = eng.generate(prompts, max_new_tokens=20, ignore_eos=True)
        return out, eng.runner.graphs_captured

    graphs, captured = run(True)
    eager, none = run(False)
    assert captured > 0 and none == 0
    assert [list(o) for o in graphs] == [list(o) for o in eager]


def wide_config():
    left = dict(heads=16, kv_heads=4, dim=64, vdim=64, scale=0.1, softcap=15.0, rot={"base": 10000.0, "dims": 32})
    right = dict(heads=8, vdim=64, state=64, groups=2, norm_groups=2, conv=4)
    delta = dict(heads=8, kv_heads=8, dim=64, vdim=128, conv=4, decay_rank=64, gate_rank=64)
    ff = {"kind": "dense", "ff": 2048, "limit": 5.0}
    return {"architecture": "Rorevik", "vocab": 1000, "width": 1024, "max_positions": 1024, "embedding": {"scale": 32.0}, "norm": {"eps": 1e-5},
            "layers": [{"type": "parallel", "mixer": {"left": left, "right": right, "left_scale": 1.1, "right_scale": 0.8}, "mlp": ff},
                       {"type": "channel_delta", "mixer": delta, "mlp": ff}]}


def test_kernels_chosen_at_real_widths_against_the_general_kernels(tmp_path):
    """A model wide enough that the bfloat16 engine takes what it takes at real sizes (tile products for the prompt,
    weight-streaming products for single tokens, the matrix-core attention) against the same engine on the general
    kernels: a 300-token prompt, a mixed step and decode steps of a batch."""
    from photon_infer_amd import ops
    from photon_infer_amd.config import RorevikConfig
    from photon_infer_amd.engine.replay import make_runner
    from photon_infer_amd.engine.step import StepEntry
    from photon_infer_amd.weights import write_random_model
    d = write_random_model(RorevikConfig.from_dict(wide_config()), str(tmp_path / "wide"), seed=2, std=0.03, norm_init="uniform", dtype="bfloat16")
    prompts = {"a": random_tokens(300, 1000, 1), "b": random_tokens(70, 1000, 2), "c": random_tokens(5, 1000, 3)}
    outs = []
    for fast in (True, False):
        prev = ops.use_fast_kernels(fast)
        try:
            r = make_runner(d, "bfloat16", 1024, 16)
            for rid in prompts:
                r.admit(rid)
            got = [r.step([StepEntry("a", prompts["a"], [0, 150, 299])]),
                   r.step([StepEntry("b", prompts["b"][:60], [59]), StepEntry("c", prompts["c"], [4]), StepEntry("a", [7], [0])])]
            for k in range(3):
                got.append(r.step([StepEntry("a", [8 + k], [0]), StepEntry("b", [prompts["b"][60 + k]], [0]), StepEntry("c", [9 + k], [0])]))
            outs.append(torch.cat(got).float().cpu())
            if fast:
                assert r.workspace.counts["gated_epilogues"] > 0, dict(r.workspace.counts)
        finally:
            ops.use_fast_kernels(prev)
    err = float((outs[0] - outs[1]).abs().max())
    assert err <= 0.04 * float(outs[1].std()) + 0.02, (err, float(outs[1].std()))
