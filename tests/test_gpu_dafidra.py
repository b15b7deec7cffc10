"""Dafidra on the GPU against the plain implementation (``plain_dafidra``): each mechanism's
kernels alone, with inputs made so that a fault shows (a far key that dominates, keys just
inside and just outside a window, a large sink, a state that must survive a cut), then whole
models under every cutting, batching, page and slot reuse, long decoding, and greedy generation
through the engine's own entry point."""
import math
import os
from types import SimpleNamespace

import numpy as np
import pytest
import torch

import plain_dafidra as P
import tiny_dafidra as TD
from gpu_tools import DEV, PagedKV, attention_ctx, cut_steps, live_token_need, run_trace
from tiny_models import random_tokens

pytestmark = pytest.mark.gpu
DTYPES = ["float32", "bfloat16"]
TORCH = {"float32": torch.float32, "bfloat16": torch.bfloat16}


def randn(*shape, seed=0, scale=1.0):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed), dtype=torch.float64) * scale


def close(got, ref, dtype, what, bf16=2e-2, f32=2e-5):
    tol = (f32 if dtype == "float32" else bf16) * max(1.0, float(ref.abs().max()))
    err = float((got.double().cpu() - ref).abs().max())
    assert err <= tol, f"{what}: error {err:.3e} > {tol:.3e}"


# ----------------------------------------------------------------------------- mechanisms alone
@pytest.mark.parametrize("two", [False, True])
@pytest.mark.parametrize("D", [48, 200, 1024])
def test_branch_norms_mean_outer_norm_and_scaled_add(two, D):
    from photon_infer_amd import ops
    T, eps, mult = 5, 1e-5, 0.7
    x, a, b = randn(T, D, seed=1), randn(T, D, seed=2, scale=3.0), randn(T, D, seed=3, scale=0.2)
    wa, wb, wo = randn(D, seed=4), randn(D, seed=5), randn(D, seed=6)
    y = 0.5 * (P.rms_norm(a, wa, eps) + P.rms_norm(b, wb, eps)) if two else a
    ref = x + mult * P.rms_norm(y, wo, eps, 1.0)
    dev = lambda t: t.float().to(DEV).contiguous()
    xs = dev(x)
    h = ops.branch_norm_add(xs, dev(a), dev(1.0 + wo), eps, mult, dev(wa) if two else None, dev(b) if two else None,
                            dev(wb) if two else None, h_dtype=torch.bfloat16)
    close(xs, ref, "float32", "stream")
    assert h.dtype == torch.bfloat16 and torch.equal(h, xs.to(torch.bfloat16))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("sizes", [(4, 2, 16, 32, 24), (2, 2, 32, 16, 9), (4, 1, 64, 64, 100), (3, 3, 20, 12, 7)])
def test_attention_mechanisms_alone(dtype, sizes):
    """Whole-projection q/k norm, temperature, pages, window, distance bias, sink, gate and values of another width,
    for portions and single tokens at once, against the plain attention over the same inputs."""
    from photon_infer_amd import ops
    H, G, d, dv, window = sizes
    Dm, eps, page = 40, 1e-5, (16 if d == dv == 64 else 8)    # pages of 16 and 64-wide heads: the matrix-core kernels in bfloat16
    c = dict(heads=H, kv_heads=G, dim=d, vdim=dv, scale=0.21, mask={"size": window}, q_temp={"coef": 0.6, "every": 5})
    W = {"q": randn(H * d, Dm, seed=1, scale=0.3), "k": randn(G * d, Dm, seed=2, scale=0.3), "v": randn(G * dv, Dm, seed=3, scale=0.3),
         "g": randn(H, Dm, seed=4, scale=0.3), "q.norm": randn(H * d, seed=5) + 2.0, "k.norm": randn(G * d, seed=6) + 2.0,
         "sink": randn(H, seed=7) * 2.0, "o": torch.eye(H * dv, dtype=torch.float64)}
    lens, new = [70, 33, 1], [30, 1, 1]                  # a portion late in a request, a single token, a first token
    hs = [randn(n, Dm, seed=10 + i) for i, n in enumerate(lens)]
    if dtype == "bfloat16":
        hs = [P.bf16_round(t.float()).double() for t in hs]
        W = {n: P.bf16_round(t.float()).double() for n, t in W.items()}
    refs = [P.sink_window_attention(h, W, c, eps, P.bf16_round if dtype == "bfloat16" else None) for h in hs]
    td = TORCH[dtype]
    # the earlier tokens' keys and values come from the same kernel: first a step with the old tokens, then the new ones
    pool_k = torch.zeros((40, G, page, d), dtype=td, device=DEV)
    pool_v = torch.zeros((40, G, dv, page), dtype=td, device=DEV)
    table = torch.full((3, 12), -1, dtype=torch.int32)
    order = torch.randperm(40, generator=torch.Generator().manual_seed(3)).tolist()
    for r, n in enumerate(lens):
        for blk in range(-(-n // page)):
            table[r, blk] = order.pop()
    table = table.to(DEV)
    w_in = torch.cat([W["q"], W["k"], W["v"], W["g"]]).float().to(DEV)
    slopes = torch.tensor([P.distance_slope(n, H) for n in range(H)], dtype=torch.float32, device=DEV)
    out = None
    for q_lens, kv_lens in (([n - m for n, m in zip(lens, new) if n - m], [n - m for n, m in zip(lens, new) if n - m]), (new, lens)):
        rows = [r for r, (n, m) in enumerate(zip(lens, new)) if (n - m if kv_lens is not lens else True)]
        ctx = attention_ctx(q_lens, kv_lens, td)
        h = torch.cat([hs[r][kv - ql:kv] for r, ql, kv in zip(rows, q_lens, kv_lens)]).float().to(DEV)
        proj = (h @ w_in.T).contiguous()
        T = h.shape[0]
        q = torch.empty((T, H * d), dtype=td, device=DEV)
        gate = torch.empty((T, H), dtype=torch.float32, device=DEV)
        tab = table[rows].contiguous()
        ops.qk_norm_kv_write(q, gate, proj, W["q.norm"].float().to(DEV), W["k.norm"].float().to(DEV), ctx, eps, 0.6, 5, H, G, d, dv, H,
                             pool_k, pool_v, tab, page)
        out = torch.empty((T, H * dv), dtype=td, device=DEV)
        ops.paged_attention(out, q, pool_k, pool_v, tab, ctx, H, G, d, page, c["scale"], window, None, value_dim=dv,
                            slopes=slopes, sinks=W["sink"].float().to(DEV), gate=gate)
    ref = torch.cat([refs[r][n - m:] for r, (n, m) in enumerate(zip(lens, new))])
    close(out, ref, dtype, "attention output", bf16=3e-2)


@pytest.mark.parametrize("dtype", DTYPES)
def test_qk_norm_adds_the_pieces_of_a_split_projection(dtype):
    """The projection as the float32 pieces of a product split over k gives what their sum gives as a tensor:
    queries, gates and the pages' keys and values, bit for bit."""
    from photon_infer_amd import ops
    from photon_infer_amd.ops import Partials
    H, G, d, dv, page, T, splits = 4, 2, 24, 40, 8, 11, 5
    N = H * d + G * d + G * dv + H
    td = TORCH[dtype]
    part = randn(splits, T, N, seed=1).float().to(DEV).contiguous()
    whole = torch.zeros((T, N), dtype=torch.float32, device=DEV)
    for s_ in range(splits):         # in split order, as the kernel adds them
        whole += part[s_]
    ctx = attention_ctx([T], [T + 20], td)
    table = torch.arange(8, dtype=torch.int32, device=DEV).flip(0).view(1, 8).contiguous()
    wq, wk = (randn(H * d, seed=2) + 2.0).float().to(DEV), (randn(G * d, seed=3) + 2.0).float().to(DEV)
    got = []
    for proj in (whole, Partials(part.view(-1), splits, T, N)):
        q = torch.zeros((T, H * d), dtype=td, device=DEV)
        gate = torch.zeros((T, H), dtype=torch.float32, device=DEV)
        kc = torch.zeros((8, G, page, d), dtype=td, device=DEV)
        vc = torch.zeros((8, G, dv, page), dtype=td, device=DEV)
        ops.qk_norm_kv_write(q, gate, proj, wq, wk, ctx, 1e-5, 0.3, 4, H, G, d, dv, H, kc, vc, table, page)
        got.append((q, gate, kc, vc))
    for a, b in zip(*got):
        assert torch.equal(a, b) and float(a.float().abs().max()) > 0


@pytest.mark.parametrize("window", [0, 100, 700])
@pytest.mark.parametrize("hd,H,G", [(64, 8, 2), (128, 4, 4), (32, 2, 1)])
def test_matrix_core_attention_with_options_against_the_general_kernel(hd, H, G, window):
    """bfloat16: the matrix-core kernels (tiles for portions, key ranges for single tokens, cut tiles and merged
    ranges late in long contexts) with distance bias, sink and gate against the general kernel on the same pages."""
    from photon_infer_amd import ops
    page = 16
    cases = {"single tokens over long contexts": ([1, 1, 1], [1500, 37, 2600]),
             "a portion late in a long context": ([96], [3000]),
             "a whole prompt beside a single token and a portion": ([300, 1, 40], [300, 900, 170])}
    slopes = torch.tensor([P.distance_slope(n, H) for n in range(H)], dtype=torch.float32, device=DEV)
    sinks = (randn(H, seed=2) * 2.0).float().to(DEV)
    for what, (q_lens, kv_lens) in cases.items():
        seqs = [(randn(n, G, hd, seed=10 + i).float(), randn(n, G, hd, seed=20 + i).float()) for i, n in enumerate(kv_lens)]
        kv = PagedKV(seqs, page, torch.bfloat16, seed=4)
        T = sum(q_lens)
        q = (randn(T, H * hd, seed=3) * 0.7).to(torch.bfloat16).to(DEV)
        gate = torch.sigmoid(randn(T, H, seed=5)).float().to(DEV).contiguous()
        outs = []
        for fast in (True, False):
            prev = ops.use_fast_kernels(fast)
            try:
                ctx = attention_ctx(q_lens, kv_lens, torch.bfloat16)
                out = torch.zeros((T, H * hd), dtype=torch.bfloat16, device=DEV)
                ops.paged_attention(out, q, kv.k, kv.v, kv.table, ctx, H, G, hd, page, 0.17, window, None, value_dim=hd,
                                    slopes=slopes, sinks=sinks, gate=gate)
                outs.append(out.float().cpu())
            finally:
                ops.use_fast_kernels(prev)
        err = float((outs[0] - outs[1]).abs().max())
        assert err <= 2e-2 * max(1.0, float(outs[1].abs().max())), f"{what}: {err}"


@pytest.mark.parametrize("distance,seen", [(23, True), (24, False), (0, True)])
@pytest.mark.parametrize("decode", [False, True])
def test_a_key_at_the_windows_edge_is_seen_or_not(distance, seen, decode):
    """One key carries a huge score and a value of its own: it shows in the output exactly when it lies inside the
    window (distance < window), in a prompt's portion and for a single token; the sink alone answers with nothing."""
    from photon_infer_amd import ops
    H, d, dv, window, page, S = 2, 16, 8, 24, 8, 61
    k = torch.zeros(S, 1, d)
    v = torch.zeros(S, 1, dv)
    target = S - 1 - distance
    k[target, 0, 0] = 50.0
    v[target, 0, :] = 7.0
    kv = PagedKV([(k, v)], page, torch.float32, seed=5)
    q_len = 1 if decode else 9
    ctx = attention_ctx([q_len], [S], torch.float32)
    q = torch.zeros(q_len, H * d)
    q[-1, 0::d] = 1.0                                  # the last token asks for the marked key, with every head
    out = torch.empty((q_len, H * dv), dtype=torch.float32, device=DEV)
    sinks = torch.full((H,), 5.0, device=DEV)
    ops.paged_attention(out, q.to(DEV), kv.k, kv.v, kv.table, ctx, H, 1, d, page, 1.0, window, None, value_dim=dv,
                        slopes=torch.zeros(H, device=DEV), sinks=sinks)
    last = out[-1].cpu()
    if seen:
        assert torch.allclose(last, torch.full_like(last, 7.0), atol=1e-3)
    else:       # only zero values and the sink are in reach: the sink takes weight and leaves nothing
        assert float(last.abs().max()) < 1e-6


def test_the_sink_counts_once_and_the_bias_grows_with_distance():
    from photon_infer_amd import ops
    H, d, dv, page, S = 2, 16, 4, 8, 20
    k = torch.zeros(S, 1, d)                           # all scores zero: weights follow the bias alone
    v = torch.arange(S, dtype=torch.float32).view(S, 1, 1).repeat(1, 1, dv)
    kv = PagedKV([(k, v)], page, torch.float32, seed=1)
    ctx = attention_ctx([1], [S], torch.float32)
    out = torch.empty((1, H * dv), dtype=torch.float32, device=DEV)
    slopes = torch.tensor([0.5, 0.0], device=DEV)
    sinks = torch.tensor([math.log(3.0), math.log(S)], device=DEV)
    ops.paged_attention(out, torch.zeros(1, H * d, device=DEV), kv.k, kv.v, kv.table, ctx, H, 1, d, page, 1.0, 0, None, value_dim=dv,
                        slopes=slopes, sinks=sinks)
    w = [math.exp(-0.5 * (S - 1 - j)) for j in range(S)]
    want0 = sum(wj * j for j, wj in enumerate(w)) / (sum(w) + 3.0)
    want1 = sum(range(S)) / (2.0 * S)                  # no bias, a sink as heavy as all keys together
    assert abs(float(out[0, 0]) - want0) < 1e-4 and abs(float(out[0, dv]) - want1) < 1e-4


@pytest.mark.parametrize("sizes", [(2, 16, 24, 37), (1, 40, 48, 37), (4, 32, 32, 300), (3, 5, 7, 150), (1, 100, 130, 37), (2, 64, 16, 420)])
def test_matrix_memory_whole_in_portions_and_token_by_token(sizes):
    """The recurrence through the state slots: whole, in portions of every size down to one token, two requests in
    one step, and a slot used again after it was cleared, against the plain recurrence."""
    from photon_infer_amd import ops
    H, d, dv, T = sizes              # more than 64 tokens of a request in a step: the walk runs in segments side by side
    cap = 6.0
    QK, V = H * d, H * dv
    N = 2 * QK + 2 * V + 2 * H
    offsets = (0, QK, 2 * QK, 2 * QK + 2 * V, 2 * QK + 2 * V + H)
    ib, fb = randn(H, seed=1), randn(H, seed=2) + 2.0

    def plain(proj):
        """the cell before its head norm, from the plain module's recurrence (identity projections)"""
        W = {"q": torch.eye(N, dtype=torch.float64)[0:QK], "k": torch.eye(N, dtype=torch.float64)[QK:2 * QK],
             "v": torch.eye(N, dtype=torch.float64)[2 * QK:2 * QK + V], "g": torch.zeros(V, N, dtype=torch.float64),
             "i": torch.eye(N, dtype=torch.float64)[offsets[3]:offsets[3] + H], "f": torch.eye(N, dtype=torch.float64)[offsets[4]:offsets[4] + H],
             "i.b": ib, "f.b": fb, "norm": torch.full((V,), 2.0, dtype=torch.float64), "o": torch.eye(V, dtype=torch.float64)}
        return P.matrix_memory(proj, W, dict(heads=H, dim=d, vdim=dv, gate_cap=cap), 1e-6)   # = head-normed cell (gate 1/2, weight 2)

    projs = [randn(T, N, seed=5, scale=1.5), randn(T - 9, N, seed=6, scale=1.5)]
    for p in projs:
        p[:, offsets[3]:] *= 4.0                        # gates that move: the running maximum matters
    refs = [plain(p) for p in projs]
    floats = ops.matrix_memory_state_floats(H, d, dv)
    state = torch.zeros((3, floats), dtype=torch.float32, device=DEV)
    w_norm = torch.full((V,), 2.0, device=DEV)

    def run(steps, slots):
        """steps: list of {request: (lo, hi)}; returns per request the head-normed output rows"""
        got = {r: [] for r in slots}
        for step in steps:
            reqs = sorted(step)
            q_lens = [step[r][1] - step[r][0] for r in reqs]
            ctx = SimpleNamespace(R=len(reqs), max_q_len=max(q_lens), q_start=torch.tensor(np.concatenate([[0], np.cumsum(q_lens)]), dtype=torch.int32, device=DEV),
                                  slots=torch.tensor([slots[r] for r in reqs], dtype=torch.int32, device=DEV))
            proj = torch.cat([projs[r][step[r][0]:step[r][1]] for r in reqs]).float().to(DEV).contiguous()
            cell = torch.empty((proj.shape[0], V), dtype=torch.float32, device=DEV)
            ops.matrix_memory_scan(cell, proj, offsets, ib.float().to(DEV), fb.float().to(DEV), cap, d ** -0.5, ctx, state, H, d, dv)
            y = torch.empty((proj.shape[0], V), dtype=torch.float32, device=DEV)
            ops.head_norm_gate(y, cell, torch.zeros_like(cell), w_norm, 1e-6, H, dv)
            for r, rows in zip(reqs, torch.split(y, q_lens)):
                got[r].append(rows)
        return {r: torch.cat(v) for r, v in got.items()}

    whole = run([{0: (0, T), 1: (0, T - 9)}], {0: 2, 1: 0})
    for r in (0, 1):
        close(whole[r], refs[r], "float32", f"whole, request {r}", f32=1e-4)
    state.zero_()                                      # the slots are used again
    cuts, lo = [], 0
    for n in [5, 1, 2, 13, 1, 1, 7, 3, 100, 129, 1, 500]:
        hi = min(T, lo + n)
        step = {0: (lo, hi)}
        if hi <= T - 9:
            step[1] = (lo, hi)                         # the second request rides along while it lasts
        elif lo < T - 9:
            step[1] = (lo, T - 9)
        cuts.append(step)
        lo = hi
        if lo >= T:
            break
    cut = run(cuts, {0: 1, 1: 2})
    for r in (0, 1):
        close(cut[r], refs[r], "float32", f"in portions, request {r}", f32=1e-4)
        close(cut[r], whole[r].double().cpu(), "float32", f"portions against whole, request {r}", f32=2e-6)


@pytest.mark.parametrize("E,top,groups,keep", [(6, 2, 3, 2), (4, 1, 1, 1), (8, 4, 4, 4), (8, 3, 2, 1), (64, 6, 8, 3), (5, 5, 1, 1)])
def test_routing_groups_and_choices(E, top, groups, keep):
    from photon_infer_amd import ops
    z = randn(50, E, seed=E + top, scale=2.0).float()
    ids, w = ops.route(z.to(DEV), top, groups, keep)
    ids, w = ids.cpu(), w.cpu()
    for t in range(z.shape[0]):
        want = P.route(z[t].double(), top, groups, keep)
        assert [e for e, _ in want] == ids[t].tolist(), f"token {t}"
        assert max(abs(a - float(b)) for (_, a), b in zip(want, w[t])) < 1e-6


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("T", [1, 3, 70, 300])
def test_routed_experts_against_the_plain_sum(dtype, T):
    from photon_infer_amd.parts import FEED_FORWARDS
    D, Fe, E = 64, 40, 6
    c = {"router": {"experts": E, "top": 2, "groups": {"count": 3, "keep": 2}}}
    W = {"router": randn(E, D, seed=1, scale=0.5)}
    for e in range(E):
        W.update({f"e{e}.gate": randn(Fe, D, seed=10 + e, scale=0.2), f"e{e}.up": randn(Fe, D, seed=20 + e, scale=0.2),
                  f"e{e}.down": randn(D, Fe, seed=30 + e, scale=0.2)})
    h = randn(T, D, seed=3)
    if dtype == "bfloat16":
        W = {n: P.bf16_round(t.float()).double() for n, t in W.items()}
        h = P.bf16_round(h.float()).double()
    ref = P.routed_experts(h, W, c, P.bf16_round if dtype == "bfloat16" else None)
    part = FEED_FORWARDS.make("routed_experts", hidden_size=D, expert_size=Fe, num_experts=E, top=2, groups=3, keep=2, accumulate=False)
    td = TORCH[dtype]
    part.load({n: t.to(td).to(DEV) for n, t in W.items()}, td, torch.device(DEV))
    out = torch.full((T, D), 9.0, dtype=torch.float32, device=DEV)
    part.forward(h.to(td).to(DEV), out, SimpleNamespace(workspace=None))
    close(out, ref, dtype, "routed experts")


# ----------------------------------------------------------------------------- whole models
@pytest.fixture(scope="module")
def model_dirs(tmp_path_factory):
    root = tmp_path_factory.mktemp("dafidra")
    return {name: TD.make_model_dir(root, name, seed=5) for name in TD.ALL}


_plain = {}
CLOSE_CALL = 0.25            # router logits (their spread is about 1): a bfloat16 choice that differs from the plain one must be
                             # this close to a tie; float32 runs are held to the plain choices themselves


class RouteRecorder:
    """Records the experts the engine chooses (every call of ``ops.route``, in order), so that the plain implementation
    can be asked for the logits of the same choices: among hundreds of routing decisions some are near ties, which
    bfloat16 rounding decides either way, and one flipped expert changes everything after it."""

    def __enter__(self):
        from photon_infer_amd import ops
        self.ops, self.real, self.calls = ops, ops.route, []

        def route(*a, **k):
            ids, w = self.real(*a, **k)
            self.calls.append(ids.cpu())
            return ids, w
        ops.route = route
        return self

    def __exit__(self, *exc):
        self.ops.route = self.real

    def by_request(self, steps, config):
        """{request: {routed layer: [tokens, top] expert ids}} from the calls, given the trace's steps."""
        layers = [i for i, l in enumerate(config["layers"]) if l["mlp"] and l["mlp"]["kind"] == "moe"]
        out, k = {}, 0
        for s in steps:
            sizes = [len(e["tokens"]) for e in s["entries"]]
            for i in layers:
                for e, part in zip(s["entries"], torch.split(self.calls[k], sizes)):
                    out.setdefault(e["id"], {}).setdefault(i, []).append(part)
                k += 1
        assert k == len(self.calls)
        return {rid: {i: torch.cat(p) for i, p in per.items()} for rid, per in out.items()}


def plain_logits(model_dir, tokens, emulate=False, forced=None):
    key = (model_dir, tuple(tokens), emulate)
    if forced is not None or key not in _plain:
        cfg, W = P.read_model_folder(model_dir)
        out = P.forward(cfg, W, list(tokens), P.bf16_round if emulate else None, forced=forced).float()
        if forced is not None:
            return out
        _plain[key] = out
    return _plain[key]


def runner_for(model_dir, name, dtype, max_tokens):
    from photon_infer_amd.engine.replay import make_runner
    return make_runner(model_dir, dtype, max_tokens, TD.ALL[name][1]["block_size"])


def check_choices(model_dir, toks, forced, what):
    """The engine's experts are the plain implementation's, or differ only where the plain router was within a
    whisker of choosing otherwise."""
    cfg, W = P.read_model_folder(model_dir)
    margins, chosen = {}, {}
    P.forward(cfg, W, list(toks), forced=forced, margins=margins, chosen=chosen)
    for i, ids in forced.items():
        for t in range(len(toks)):
            if sorted(int(e) for e in ids[t]) != sorted(chosen[i][t]):
                assert margins[i][t] < CLOSE_CALL, f"{what}: layer {i} token {t}: experts {ids[t].tolist()} instead of {chosen[i][t]} (margin {margins[i][t]:.3f})"


def check(got, model_dir, reqs, dtype, what, choices=None):
    """``choices`` (bfloat16 runs): the experts the engine chose per request; the plain logits are then those of the
    same choices, which must be the plain ones up to close calls."""
    assert got, "no logits came back"
    for rid, toks in reqs.items():
        forced = choices.get(rid) if choices else None
        if forced:
            check_choices(model_dir, toks, forced, what)
        ref = plain_logits(model_dir, toks, forced=forced)
        if dtype == "float32":
            tol = 1e-4 * max(1.0, float(ref.abs().max()))
        else:       # three times what rounding activations to bfloat16 does to the plain implementation itself
            tol = 3.0 * float((plain_logits(model_dir, toks, True, forced=forced) - ref).abs().max())
        over = []
        for p in range(len(toks)):
            assert (rid, p) in got, f"{what}: logits of {rid} position {p} are missing"
            err = float((got[(rid, p)] - ref[p]).abs().max())
            if dtype == "float32" or err > 3.0 * tol:
                assert err <= tol, f"{what}: {rid} position {p}: error {err:.3e} > {tol:.3e} (first wrong position)"
            elif err > tol:
                over.append(p)
        # bfloat16: a sublayer's result is normalised before it is added, so where a result happens to be small (an
        # expert whose terms cancel) rounding noise is blown up to full size at that one position; such positions are
        # rare, stay within three times the bound, and leave their neighbours alone - a fault of cache, state or window
        # does none of the three
        assert len(over) <= max(1, len(toks) // 50), f"{what}: {rid}: positions {over} are over {tol:.3e}"


def run_checked(runner, steps, out_dir, model_dir, reqs, dtype, what):
    """Replay ``steps`` and compare; in bfloat16 the plain implementation follows the engine's routing choices."""
    if dtype == "float32":
        return check(run_trace(runner, steps, out_dir), model_dir, reqs, dtype, what)
    with RouteRecorder() as rec:
        got = run_trace(runner, steps, out_dir)
    check(got, model_dir, reqs, dtype, what, rec.by_request(steps, P.read_model_folder(model_dir)[0]))


LENGTHS = {"P": [1, 26, 90], "Q": [2, 45, 100], "R": [3, 130, 210], "S": [2, 30, 75]}


def requests_for(name, seed=0, model_dir=None):
    vocab = TD.ALL[name][0]["vocab"]
    return {f"r{i}": random_tokens(n, vocab, seed * 100 + i) for i, n in enumerate(LENGTHS[name])}


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", list(TD.ALL))
def test_whole_prompts_and_every_layers_stream(name, dtype, model_dirs, tmp_path):
    reqs = requests_for(name, model_dir=model_dirs[name])
    steps = []
    for rid, toks in reqs.items():
        steps += cut_steps(rid, toks, [len(toks)], first_step=len(steps))
    runner = runner_for(model_dirs[name], name, dtype, live_token_need(steps))
    run_checked(runner, steps, str(tmp_path), model_dirs[name], reqs, dtype, "whole")
    if dtype == "float32":         # the stream after every layer, for the longest request
        from photon_infer_amd.engine.step import StepEntry
        toks = reqs["r2"]
        cfg, W = P.read_model_folder(model_dirs[name])
        want = []
        P.forward(cfg, W, toks, streams=want)
        got = []
        for b in runner.model.blocks:
            def wrapped(x, ctx, cache, f=b.forward):
                f(x, ctx, cache)
                got.append(x.detach().double().cpu())
            b.forward = wrapped
        runner.admit("s")
        runner.step([StepEntry("s", toks, [])])
        for i, (g, w) in enumerate(zip(got, want)):
            close(g, w, "float32", f"stream after layer {i}", f32=1e-4)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", list(TD.ALL))
def test_prefill_then_token_by_token_and_all_token_by_token(name, dtype, model_dirs, tmp_path):
    reqs = requests_for(name, seed=1, model_dir=model_dirs[name])
    steps = []
    for rid, toks in reqs.items():
        head = max(0, len(toks) - 50)                  # the window passes over decoded tokens
        sizes = ([head] if head else []) + [1] * (len(toks) - head)
        steps += cut_steps(rid, toks, sizes, first_step=len(steps))
    steps += cut_steps("all", reqs["r1"], [1], first_step=len(steps))
    runner = runner_for(model_dirs[name], name, dtype, live_token_need(steps))
    run_checked(runner, steps, str(tmp_path), model_dirs[name], dict(reqs, all=reqs["r1"]), dtype, "decoding")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", list(TD.ALL))
@pytest.mark.parametrize("sizes", [[2], [7, 2, 31, 1, 3], [64, 5], [17]])
def test_portions_of_changing_size(name, dtype, sizes, model_dirs, tmp_path):
    reqs = {"r2": requests_for(name, seed=2, model_dir=model_dirs[name])["r2"]}
    steps = cut_steps("r2", reqs["r2"], sizes)
    runner = runner_for(model_dirs[name], name, dtype, live_token_need(steps))
    run_checked(runner, steps, str(tmp_path), model_dirs[name], reqs, dtype, f"portions {sizes}")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", list(TD.ALL))
def test_mixed_batches_with_pages_and_slots_used_again(name, dtype, model_dirs, tmp_path):
    """Seven unequal requests through four slots: portions of some beside single tokens of others; a request may sit
    out a step; a finished request's pages and slot go to the next one.  Each must come out as it does alone."""
    vocab = TD.ALL[name][0]["vocab"]
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
    run_checked(runner, steps, str(tmp_path), model_dirs[name], reqs, dtype, "mixed")
    assert all(g.pool.num_allocated == 0 for g in runner.cache.groups)


@pytest.mark.parametrize("name", ["P", "Q"])
def test_long_decoding_gives_pages_back_and_keeps_its_state(name, model_dirs, tmp_path):
    """400 tokens one by one: many windows pass, the windowed cache group hands pages back while the request runs, and
    the memory's state is all that remembers the early tokens."""
    vocab = TD.ALL[name][0]["vocab"]
    toks = random_tokens(400, vocab, 9)
    steps = cut_steps("long", toks, [3] + [1] * 397)
    runner = runner_for(model_dirs[name], name, "float32", 128)      # far fewer pages than 400 tokens: only a window's worth is live
    check(run_trace(runner, steps, str(tmp_path)), model_dirs[name], {"long": toks}, "float32", "long decoding")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", list(TD.ALL))
def test_greedy_generation_through_the_engine(name, dtype, model_dirs):
    """The engine's own entry point, scheduler, sampling and decode steps: unequal prompts at once, more requests than
    slots, prompts longer than a portion; every request must generate what the plain implementation generates alone."""
    from photon_infer_amd.engine import ContinuousBatchEngine, EngineOptions
    cfg, W = P.read_model_folder(model_dirs[name])
    vocab = cfg["vocab"]
    prompts = [random_tokens(n, vocab, 70 + i) for i, n in enumerate([5, 41, 18, 70, 2])]
    engine = ContinuousBatchEngine(model_dirs[name], EngineOptions(dtype=dtype, block_size=TD.ALL[name][1]["block_size"], max_batch=3,
                                                                   max_cache_tokens=1024, chunk_size=32, max_model_len=256))
    got = engine.generate(prompts, max_new_tokens=12)
    for prompt, out in zip(prompts, got):
        want = P.greedy_generate(cfg, W, prompt, 12)
        if dtype == "float32":
            assert list(out) == want
        else:       # bfloat16: a near tie may fall the other way; everything before the first difference must agree and the
            # differing token must be a close second of the plain logits (sequences with a routing tie are left out)
            margins = {}
            P.forward(cfg, W, prompt + want, margins=margins)
            if any(m < CLOSE_CALL for per in margins.values() for m in per):
                continue
            for i, (a, b) in enumerate(zip(out, want)):
                if a != b:
                    lg = P.forward(cfg, W, prompt + want[:i])[-1]
                    assert float(lg[b] - lg[a]) < 0.05 * float(lg.std()), f"token {i}: {a} instead of {b}"
                    break


def test_command_line_and_replayed_decode_steps(model_dirs, tmp_path):
    """The framework's command serves the design as it serves its others (from a folder, and from a bare configuration
    with random weights); and decode steps replayed as HIP graphs give the tokens of eager steps, with new requests'
    prompts in between and states in slots that are used again."""
    import json
    import subprocess
    from photon_infer_amd.engine import ContinuousBatchEngine, EngineOptions
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    cfg, W = P.read_model_folder(model_dirs["P"])
    prompt = random_tokens(9, cfg["vocab"], 81)
    want = P.greedy_generate(cfg, W, prompt, 5)
    proc = subprocess.run([os.path.join(root, "bin", "llama_infer"), model_dirs["P"], "--dtype", "fp32", "--prompt-ids",
                           ",".join(map(str, prompt)), "--max-new-tokens", "5", "--temperature", "0", "--ignore-eos"],
                          capture_output=True, text=True, timeout=300)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert "Architecture: Dafidra" in proc.stdout and f"Generated ids: {','.join(map(str, want))}" in proc.stdout
    (tmp_path / "cfg").mkdir()
    json.dump(TD.TINY_Q, open(tmp_path / "cfg" / "config.json", "w"))
    proc = subprocess.run([os.path.join(root, "bin", "llama_infer"), str(tmp_path / "cfg"), "--random-weights", "--seed", "3",
                           "--prompt-ids", "5,6,7", "--max-new-tokens", "4", "--ignore-eos"], capture_output=True, text=True, timeout=300)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert "Layers: 3" in proc.stdout and "Generated ids:" in proc.stdout

    prompts = [random_tokens(n, cfg["vocab"], 90 + n) for n in (3, 40, 17, 9, 26)]

    def run(use_graphs):
        eng = ContinuousBatchEngine(model_dirs["P"], EngineOptions(dtype="bfloat16", block_size=16, max_batch=3, max_cache_tokens=1024,
                                                                   chunk_size=8, max_step_tokens=24, max_model_len=256, use_graphs=use_graphs))
        assert eng.runner.graph_safe
        out = eng.generate(prompts, max_new_tokens=20, ignore_eos=True)
        return out, eng.runner.graphs_captured

    graphs, captured = run(True)
    eager, none = run(False)
    assert captured > 0 and none == 0
    assert [list(o) for o in graphs] == [list(o) for o in eager]


def test_kernels_chosen_at_real_widths_against_the_general_kernels(tmp_path):
    """A model wide enough that the bfloat16 engine takes what it takes at real sizes - products split over k whose pieces
    the q/k norm kernel adds, tile products for the prompt, the memory walked in segments, the matrix-core attention -
    against the same engine on the general kernels: a 300-token prompt, a mixed step and decode steps of a batch."""
    from photon_infer_amd import ops
    from photon_infer_amd.config import DafidraConfig
    from photon_infer_amd.engine.replay import make_runner
    from photon_infer_amd.engine.step import StepEntry
    from photon_infer_amd.weights import write_random_model
    left = dict(heads=16, kv_heads=4, dim=64, vdim=64, scale=0.1, mask={"size": 200}, q_temp={"coef": 0.3, "every": 64})
    right = dict(heads=4, dim=64, vdim=128, gate_cap=9.0)
    layer = {"type": "parallel", "mixer": {"left": left, "right": right}, "mlp": {"kind": "dense", "ff": 2048}}
    raw = {"architecture": "Dafidra", "vocab": 1000, "width": 1024, "norm": {"eps": 1e-5}, "residual_mult": 0.6, "layers": [layer, layer]}
    d = write_random_model(DafidraConfig.from_dict(raw), str(tmp_path / "wide"), seed=2, std=0.03, norm_init="uniform", dtype="bfloat16")
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
                assert r.workspace.counts["qkv_pieces"] > 0, dict(r.workspace.counts)
        finally:
            ops.use_fast_kernels(prev)
    err = float((outs[0] - outs[1]).abs().max())
    assert err <= 0.04 * float(outs[1].std()) + 0.02, (err, float(outs[1].std()))
