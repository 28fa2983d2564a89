"""Kesovik on the GPU against the plain implementation (tests/plain/kesovik_plain.py), in 32-bit and in bfloat16.

Small configurations of their own and seeded random weights: one whose layers all differ (keys wider than values and
the other way round, grouped and ungrouped heads, a rotation on part of a head, windows of 7 and 24 tokens, a layer
without a feed-forward, routers with and without identity experts and shared expert, a decay of exactly one), one
whose constants are one and whose sizes coincide, and one at widths where the serving kernels run.  Each mechanism
alone at its kernel, with inputs made so that a fault shows (a key that takes all the weight just inside and just
outside the window, states and pages filled with NaN before use); then whole prompts, token-by-token decoding,
portions down to two tokens, mixed batches with pages and slots used again, long decoding through recorded steps,
greedy generation through the scheduler, the command line and the trace replay program.
"""
import json
import os
import subprocess
import sys

import pytest
import torch

from conftest import ROOT, token_ids
from plain import kesovik_plain as P
from test_gpu_model import SPLIT_TOL, TOL, close, mixed_trace, pages_were_used_again, run_alone, run_mixed

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
F64 = torch.float64


def left(heads, kv_heads, dim, vdim, window, rot_dims, base, scale):
    out = {"dim": dim, "heads": heads, "kv_heads": kv_heads, "scale": scale, "vdim": vdim}
    if window is not None:
        out["mask"] = {"size": window}
    if rot_dims:
        out["rot"] = {"base": base, "dims": rot_dims}
    return out


def lightning(heads, dim, vdim, decay):
    assert len(decay) == heads
    return {"decay": decay, "dim": dim, "heads": heads, "vdim": vdim}


def parallel(l, r, left_scale, right_scale):
    return "parallel", {"left": l, "left_scale": left_scale, "right": r, "right_scale": right_scale}


def moe(experts, identity, top, ff, shared):
    out = {"expert": {"ff": ff}, "kind": "moe", "router": {"experts": experts, "identity": identity, "top": top}}
    if shared is not None:
        out["shared"] = {"ff": shared}
    return out


def dense(ff):
    return {"ff": ff, "kind": "dense"}


def layer(mixer, mlp):
    kind, sizes = mixer if isinstance(mixer, tuple) else ("lightning", mixer)
    return {"mixer": sizes, "mlp": mlp, "type": kind}


def config(vocab, width, eps, alpha, embed_scale, softcap, layers):
    return {"architecture": "Kesovik", "embedding": {"scale": embed_scale}, "layers": layers, "logit_softcap": softcap,
            "norm": {"eps": eps}, "postln_alpha": alpha, "vocab": vocab, "width": width}


# every layer another shape
MIXED = config(307, 96, 1e-5, 1.7, 2.0, 9.0, [
    layer(parallel(left(6, 2, 32, 16, 24, 16, 1e4, 0.2), lightning(3, 16, 32, [0.5, 0.9, 0.99]), 0.7, 1.3),
          moe(5, 2, 3, 48, 80)),
    layer(lightning(2, 48, 16, [0.8, 1.0]), dense(160)),
    layer(parallel(left(4, 4, 16, 48, 7, 16, 500.0, 0.4), lightning(1, 32, 64, [0.95]), 1.2, 0.6), None),
    layer(lightning(4, 16, 16, [0.3, 0.7, 0.97, 0.999]), moe(3, 0, 1, 64, None)),
])
# constants that are one, sizes that coincide, a window no prompt of the tests reaches
EQUAL = config(515, 128, 1e-6, 1.0, 1.0, 30.0, [
    layer(parallel(left(2, 2, 64, 64, 1000, 64, 1e4, 0.125), lightning(2, 64, 64, [0.9, 0.9]), 1.0, 1.0), dense(128)),
    layer(parallel(left(2, 2, 64, 64, 1000, 64, 1e4, 0.125), lightning(2, 64, 64, [0.9, 0.9]), 1.0, 1.0),
          moe(2, 1, 1, 128, 128)),
])
# widths of a real model's layers (inner sizes that are multiples of 1,024, heads of 128 in groups of four)
WIDE = config(300, 1024, 1e-6, 2.0, 1.5, 20.0, [
    layer(parallel(left(8, 2, 128, 128, 64, 64, 1e6, 0.09), lightning(4, 128, 128, [0.7, 0.9, 0.99, 0.999]), 0.9, 1.1),
          moe(4, 1, 2, 256, 512)),
    layer(lightning(8, 128, 128, [0.5, 0.8, 0.9, 0.95, 0.98, 0.99, 0.995, 0.999]), dense(2048)),
])
CONFIGS = {"mixed": MIXED, "equal": EQUAL, "wide": WIDE}


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    if not torch.cuda.is_available():
        pytest.skip("no GPU visible")
    from pulse_infer_amd.config import KesovikConfig
    from pulse_infer_amd.weights import write_model_folder

    out = {}
    for seed, (name, cfg) in enumerate(CONFIGS.items()):
        out[name] = write_model_folder(KesovikConfig.from_dict(cfg), str(tmp_path_factory.mktemp(name)), seed=170 + seed)
    return out


@pytest.fixture(scope="module")
def plain(folders):
    models = {name: P.PlainKesovik.from_folder(folder) for name, folder in folders.items()}
    memo = {}

    def logits(name, ids):
        key = (name, tuple(ids))
        if key not in memo:
            memo[key] = models[name].logits(list(ids))
        return memo[key]

    def close_calls(name, ids):
        """Positions at which a router's choice hangs on less than CLOSE_CALL: bfloat16 may choose otherwise there."""
        key = ("calls", name, tuple(ids))
        if key not in memo:
            memo[key] = set((models[name].router_margins(list(ids)) < CLOSE_CALL).nonzero().flatten().tolist())
        return memo[key]

    logits.models = models
    logits.close_calls = close_calls
    return logits


CLOSE_CALL = 0.006


def agree(got, want, dtype, what, calls=(), first=0, tol=TOL, carried=False):
    """``close``; in bfloat16 without the positions at which a router's choice is a close call (``calls``, positions
    in the sequence; row 0 of ``got`` is position ``first``), which must stay few.  ``carried``: another choice at one
    position may reach all later ones (through a state that forgets nothing, say) and close calls may be many: then
    the positions before the first close call are compared one by one, and of the rest the median error."""
    if dtype == "bfloat16" and calls and carried:
        cut = max(0, min(calls) - first)
        if cut:
            close(got[:cut], want[:cut], dtype, what + " (before the first close call)", tol)
        if cut < want.shape[0]:
            rest = (got[cut:].double().cpu() - want[cut:].double().cpu()).abs().max(dim=1).values
            assert torch.isfinite(rest).all(), what
            assert float(rest.median()) <= tol[dtype] * max(1.0, float(want.abs().max())), f"{what}: median error {float(rest.median()):.3e}"
        return
    if dtype == "bfloat16" and calls:
        keep = [i for i in range(want.shape[0]) if i + first not in calls]
        assert len(keep) >= 0.7 * want.shape[0] or want.shape[0] < 10, f"{what}: too many close calls to say anything"
        if not keep:
            return
        got, want = got[keep], want[keep]
    close(got, want, dtype, what, tol)


@pytest.fixture(scope="module")
def runners(folders):
    from pulse_infer_amd.engine.runner import ModelRunner
    from pulse_infer_amd.models.factory import load_model

    made = {}

    def get(name, dtype, page=16, tokens=512):
        key = (name, dtype, page, tokens)
        if key not in made:
            _, model = load_model(folders[name], mode=dtype)
            made[key] = ModelRunner(model, page_size=page, num_pages=tokens // page, max_requests=4)
        return made[key]

    return get


# ------------------------------------------------------------------------------------------- mechanisms alone
def rnd(*shape, seed=0, scale=1.0):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed), dtype=torch.float32) * scale


def stored(x, dtype):
    dev = x.to(dtype).to(DEV)
    return dev, dev.cpu().to(F64)


def tol(dtype):
    return dict(atol=2e-5, rtol=2e-5) if dtype == torch.float32 else dict(atol=2e-2, rtol=2e-2)


def ints(values):
    return torch.tensor(values, dtype=torch.int32, device=DEV)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads,d,dv,groups", [(3, 16, 32, 1), (2, 48, 16, 4), (1, 32, 100, 4), (4, 128, 128, 16),
                                               (2, 64, 64, 16), (1, 130, 24, 1)])
def test_the_state_walk(dtype, heads, d, dv, groups):
    """Three requests in one step (a portion of 37 tokens that continues a state, a fresh prompt of 20 in a slot whose
    state holds NaN, a single decoded token), then the same requests one token further: outputs and states are the
    plain walk's, whatever number of lanes shares a column's rows."""
    from pulse_infer_amd.ops import kernels

    decay = [0.5, 1.0, 0.97, 0.999][:heads]
    slots = 5
    counts, starts, slot_of = [37, 20, 1], [12, 0, 300], [3, 0, 4]
    state = torch.full((slots, heads, d, dv), float("nan"), device=DEV)
    before = {}
    for i, s in enumerate(slot_of):
        if starts[i]:
            before[i] = rnd(heads, d, dv, seed=40 + i)
            state[s] = before[i].to(DEV)
    cols = 2 * heads * d + heads * dv + 8
    lam = torch.tensor(decay, dtype=torch.float32, device=DEV)
    first = [0, 37, 57, 58]
    for round_ in range(2):
        total = first[-1]
        x, xref = stored(rnd(total, cols, seed=7 + round_), dtype)
        out = torch.full((total, heads * dv), float("nan"), device=DEV)
        kernels.lightning_scan(x, 4, 4 + heads * d, 8 + 2 * heads * d, out, state, lam, ints(first), ints(starts),
                               ints(slot_of), heads, d, dv, "silu", groups)
        for i in range(3):
            rows = xref[first[i]:first[i + 1]]
            q = P.silu(rows[:, 4:4 + heads * d]).view(-1, heads, d)
            k = P.silu(rows[:, 4 + heads * d:4 + 2 * heads * d]).view(-1, heads, d)
            v = P.silu(rows[:, 8 + 2 * heads * d:8 + 2 * heads * d + heads * dv]).view(-1, heads, dv)
            want, last = P.decayed_state_walk(q, k, v, decay, before[i].to(F64) if starts[i] else None)
            got = out[first[i]:first[i + 1]].cpu().to(F64).view(-1, heads, dv)
            scale = max(1.0, float(want.abs().max()))
            assert float((got - want).abs().max()) <= 3e-5 * scale, (round_, i)
            assert float((state[slot_of[i]].cpu().to(F64) - last).abs().max()) <= 3e-5 * max(1.0, float(last.abs().max()))
            before[i] = last.to(torch.float32)
        starts = [s + c for s, c in zip(starts, counts)]
        counts, first = [1, 1, 1], [0, 1, 2, 3]
    assert torch.isnan(state[1]).all() and torch.isnan(state[2]).all()      # slots of no request are left alone


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads,d,dv,groups,piece", [(3, 16, 32, 1, 16), (2, 64, 64, 16, 32), (4, 128, 128, 4, 64),
                                                     (1, 48, 100, 4, 16)])
def test_the_state_walk_in_pieces(dtype, heads, d, dv, groups, piece):
    """A long portion that continues a state, a fresh one, a short one and a single token in one step, the long ones
    cut into pieces that are walked at the same time: outputs and final states are those of the walk token by token,
    and of the plain walk."""
    from pulse_infer_amd.ops import kernels

    class E:
        def __init__(self, first_row, count):
            self.first_row, self.count = first_row, count

    decay = [0.5, 1.0, 0.97, 0.999][:heads]
    counts, starts, slot_of = [5 * piece + 3, 2 * piece, piece + 1, 1], [7, 0, 40, 300], [3, 0, 4, 1]
    first = [0]
    for n in counts:
        first.append(first[-1] + n)
    flat = kernels.lightning_pieces([E(f, n) for f, n in zip(first, counts)], piece)
    assert flat is not None and len(flat) // 4 == 6 + 2 + 1 + 1
    state = torch.full((5, heads, d, dv), float("nan"), device=DEV)
    before = {}
    for i, slot in enumerate(slot_of):
        if starts[i]:
            before[i] = rnd(heads, d, dv, seed=40 + i)
            state[slot] = before[i].to(DEV)
    whole = state.clone()
    cols = 2 * heads * d + heads * dv
    lam = torch.tensor(decay, dtype=torch.float32, device=DEV)
    x, xref = stored(rnd(first[-1], cols, seed=9), dtype)
    out = torch.full((first[-1], heads * dv), float("nan"), device=DEV)
    scratch = torch.full((len(flat) // 4, heads, d, dv), float("nan"), device=DEV)
    kernels.lightning_scan(x, 0, heads * d, 2 * heads * d, out, state, lam, ints(first), ints(starts), ints(slot_of),
                           heads, d, dv, "silu", groups, ints(flat), scratch)
    direct = torch.full_like(out, float("nan"))
    kernels.lightning_scan(x, 0, heads * d, 2 * heads * d, direct, whole, lam, ints(first), ints(starts), ints(slot_of),
                           heads, d, dv, "silu", groups)
    for i in range(len(counts)):
        rows = xref[first[i]:first[i + 1]]
        q = P.silu(rows[:, :heads * d]).view(-1, heads, d)
        k = P.silu(rows[:, heads * d:2 * heads * d]).view(-1, heads, d)
        v = P.silu(rows[:, 2 * heads * d:]).view(-1, heads, dv)
        want, last = P.decayed_state_walk(q, k, v, decay, before[i].to(F64) if starts[i] else None)
        got = out[first[i]:first[i + 1]].cpu().to(F64).view(-1, heads, dv)
        scale = max(1.0, float(want.abs().max()))
        assert float((got - want).abs().max()) <= 5e-5 * scale, i
        assert float((got - direct[first[i]:first[i + 1]].cpu().to(F64).view(-1, heads, dv)).abs().max()) <= 5e-5 * scale
        assert float((state[slot_of[i]].cpu().to(F64) - last).abs().max()) <= 5e-5 * max(1.0, float(last.abs().max()))
    assert torch.isnan(state[2]).all()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_heads_normed_together_and_gated(dtype):
    from pulse_infer_amd.ops import kernels

    tokens, n, eps, scale = 7, 96, 1e-5, 1.3
    o = rnd(tokens, n, seed=1, scale=3.0).to(DEV)
    w, wref = stored(1.0 + rnd(n, seed=2, scale=0.1), dtype)
    wide, gref = stored(rnd(tokens, n + 40, seed=3), dtype)
    out = torch.zeros(tokens, 2 * n, dtype=dtype, device=DEV)
    kernels.gated_rmsnorm(o, w, wide[:, 40:], out[:, n:], eps, scale)
    want = scale * P.unit_rms(o.cpu().to(F64), eps) * wref * torch.sigmoid(gref[:, 40:])
    assert torch.allclose(out[:, n:].cpu().to(F64), want, **tol(dtype))
    assert float(out[:, :n].abs().max()) == 0.0


def paged(lens, nkv, d, bs, dtype, seed):
    """Pages filled with NaN (nothing stale may reach an output) and a shuffled block table."""
    pages_per = [(n + bs - 1) // bs for n in lens]
    total = sum(pages_per) + 2
    perm = torch.randperm(total, generator=torch.Generator().manual_seed(seed)).tolist()
    kc = torch.full((total, nkv, bs, d), float("nan"), dtype=dtype, device=DEV)
    vc = torch.full((total, nkv, d, bs), float("nan"), dtype=dtype, device=DEV)
    table = torch.full((len(lens), max(pages_per)), -1, dtype=torch.int32)
    at = 0
    for r, n in enumerate(pages_per):
        table[r, :n] = torch.tensor(perm[at:at + n], dtype=torch.int32)
        at += n
    return kc, vc, table


WINDOW_CASES = [
    dict(nq=6, nkv=2, d=32, dv=16, bs=16, window=24, rot=16, lens=[150, 1, 64, 65, 71, 72, 73], portion=70),   # (the
    # window's far edge of the last three lies at a page's last and first slot)
    dict(nq=4, nkv=4, d=16, dv=48, bs=16, window=7, rot=16, lens=[90, 33, 17], portion=40),
    dict(nq=8, nkv=2, d=128, dv=128, bs=32, window=64, rot=64, lens=[257, 100], portion=129),
    dict(nq=3, nkv=1, d=48, dv=96, bs=16, window=40, rot=48, lens=[200, 41, 40, 5], portion=2),
    dict(nq=2, nkv=1, d=20, dv=10, bs=4, window=5, rot=10, lens=[45, 9], portion=11),
]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("case", WINDOW_CASES)
@pytest.mark.parametrize("needle", [None, "inside", "outside"])
def test_prepared_rows_and_the_window(case, dtype, needle):
    """Biases, the norm over a token's whole q and whole k, the rotation on part of a head, keys and values of
    different widths in pages of one width, and the window: a portion of request 0 beside single tokens of the
    others.  With a needle, the stored key at the window's far edge (or the one just beyond it) is replaced by 40 times
    the last query of every request, so that it takes all the weight if it is seen."""
    from pulse_infer_amd.parts.attention_rows import stored_width
    from pulse_infer_amd.ops import attention_mfma as M
    from pulse_infer_amd.ops import kernels

    nq, nkv, d, dv, bs, window, rot, lens, portion = (case[x] for x in ("nq", "nkv", "d", "dv", "bs", "window", "rot",
                                                                         "lens", "portion"))
    eps, scale, share, base, vscale = 1e-5, 0.3, nq // nkv, 1e4, 0.8
    D = stored_width(d, dv)
    kc, vc, table = paged(lens, nkv, D, bs, dtype, seed=3)
    cols = nq * d + nkv * (d + dv)
    bias = [stored(rnd(n, seed=30 + i, scale=0.3), dtype) for i, n in enumerate((nq * d, nkv * d, nkv * dv))]
    wq, wqref = stored(1.0 + rnd(nq * d, seed=33, scale=0.1), dtype)
    wk, wkref = stored(1.0 + rnd(nkv * d, seed=34, scale=0.1), dtype)
    inv = base ** (-2.0 * torch.arange(rot // 2, dtype=F64) / rot)
    rows_of, keys, values, queries = [], [], [], []
    for r, n in enumerate(lens):
        raw = rnd(n, cols, seed=10 + r)
        rows, ref = stored(raw, dtype)
        rows_of.append(rows)
        q = P.unit_rms(ref[:, :nq * d] + bias[0][1], eps) * wqref
        k = P.unit_rms(ref[:, nq * d:nq * d + nkv * d] + bias[1][1], eps) * wkref
        positions = list(range(n))
        queries.append(P.rotate_pairs(q.view(n, nq, d), positions, base, rot))
        keys.append(P.rotate_pairs(k.view(n, nkv, d), positions, base, rot))
        values.append(((ref[:, nq * d + nkv * d:] + bias[2][1]) * vscale).view(n, nkv, dv))
    def tables_for(positions):
        angle = torch.tensor(positions, dtype=F64).view(-1, 1) * inv.view(1, -1)
        return torch.cos(angle).float().to(DEV).contiguous(), torch.sin(angle).float().to(DEV).contiguous()

    def prepare(rows, positions, entry):
        cos, sin = tables_for(positions)
        q = torch.full((rows.shape[0], nq * D), float("nan"), dtype=dtype, device=DEV)
        kernels.qkv_rows(rows, q, nq, nkv, d, dv, D, tuple(b[0] for b in bias), (wq, wk), eps, cos, sin, rot, 0, kc, vc,
                         ints(positions), ints(entry), table.to(DEV), value_scale=vscale)
        return q

    fed = [lens[0] - portion] + [n - 1 for n in lens[1:]]
    for r, n in enumerate(fed):
        if n:
            prepare(rows_of[r][:n].contiguous(), list(range(n)), [r] * n)
    positions = list(range(fed[0], lens[0])) + [n - 1 for n in lens[1:]]
    entry = [0] * portion + list(range(1, len(lens)))
    step = torch.cat([rows_of[0][fed[0]:]] + [rows_of[r][n - 1:] for r, n in enumerate(lens) if r]).contiguous()
    q = prepare(step, positions, entry)
    # what the kernel left: q in heads of D channels (zeros beyond d), k and v in their pages (zeros beyond d and dv)
    got_q = q.cpu().to(F64).view(-1, nq, D)
    want_q = torch.cat([queries[0][fed[0]:]] + [queries[r][n - 1:] for r, n in enumerate(lens) if r])
    if needle is None:
        assert torch.allclose(got_q[..., :d], want_q, **tol(dtype))
        assert float(got_q[..., d:].abs().sum()) == 0.0
        for r, n in enumerate(lens):
            for j in (0, n // 2, n - 1):
                page, slot = int(table[r, j // bs]), j % bs
                assert torch.allclose(kc[page, :, slot, :d].cpu().to(F64), keys[r][j], **tol(dtype))
                assert torch.allclose(vc[page, :, :dv, slot].cpu().to(F64), values[r][j], **tol(dtype))
                assert float(kc[page, :, slot, d:].float().abs().sum()) == 0.0
                assert float(vc[page, :, dv:, slot].float().abs().sum()) == 0.0
        stored_keys, stored_values = keys, values
    else:
        # plant the needle in the pages themselves: 40 times the last query of the group's first head
        stored_keys, stored_values = [k.clone() for k in keys], values
        for r, n in enumerate(lens):
            if n <= window:
                continue
            j = n - 1 - (window - 1 if needle == "inside" else window)
            page, slot = int(table[r, j // bs]), j % bs
            for g in range(nkv):
                planted = (40.0 * queries[r][n - 1, g * share]).to(dtype)
                kc[page, g, slot, :d] = planted.to(DEV)
                stored_keys[r][j, g] = planted.to(F64)
    out = torch.zeros(len(positions), nq * D, dtype=dtype, device=DEV)
    pos_t, ent_t = ints(positions), ints(entry)
    paths = ["generic"]
    if M.supported(D, bs, dtype, dtype):
        paths.append("matrix")
    used_q = q.cpu().to(F64).view(-1, nq, D)[..., :d]
    want = torch.zeros(len(positions), nq, dv, dtype=F64)
    for t, (p, e) in enumerate(zip(positions, entry)):
        lo = max(0, p - window + 1)
        for h in range(nq):
            g = h // share
            w = torch.softmax((stored_keys[e][lo:p + 1, g].to(dtype).to(F64) @ used_q[t, h]) * scale, dim=0)
            want[t, h] = (w.view(-1, 1) * stored_values[e][lo:p + 1, g].to(dtype).to(F64)).sum(0)
    if needle == "inside":
        # the needle is seen by the last token of every long request, and decides its output
        for r, n in enumerate(lens):
            if n > window:
                t = portion - 1 if r == 0 else portion + r - 1
                j = n - window
                assert torch.allclose(want[t, 0], stored_values[r][j, 0].to(dtype).to(F64), atol=1e-2, rtol=1e-2)
    for path in paths:
        out.zero_()
        if path == "generic":
            kernels.attn_generic(q, out, nq, nkv, D, kc, vc, pos_t, ent_t, table.to(DEV), scale, window)
        else:
            class E:
                def __init__(self, first_row, count):
                    self.first_row, self.count = first_row, count
            numbered = list(enumerate([E(0, portion)] + [E(portion + i, 1) for i in range(len(lens) - 1)]))
            small = numbered
            if portion >= M.PORTION_MIN_TOKENS:
                small = numbered[1:]
                big = ints(M.build_items(numbered[:1], M.portion_tokens(share, D)))
                M.attn_prefill(q, out, nq, nkv, D, kc, vc, pos_t, table.to(DEV), big, scale, window)
            items = ints(M.build_items(small, M.tokens_per_item(share)))
            split = (max(lens) + 31) // 32 * 32
            M.attn_mfma(q, out, nq, nkv, D, kc, vc, pos_t, table.to(DEV), items, scale, window, split, 1, max(lens),
                        None, None)
        got = out.cpu().to(F64).view(-1, nq, D)
        assert torch.allclose(got[..., :dv], want, **tol(dtype)), (path, float((got[..., :dv] - want).abs().max()))
        assert float(got[..., dv:].abs().sum()) == 0.0, path


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("experts,identity,top,ff,hidden", [(5, 2, 3, 48, 96), (3, 0, 1, 64, 80), (10, 3, 4, 72, 192),
                                                            (2, 1, 3, 40, 64)])
def test_router_and_experts(dtype, experts, identity, top, ff, hidden):
    """Choice by score plus correction (a correction large enough to change the choice), weights from the scores
    alone, identity experts that give the input back, the weighted sum in float32."""
    from pulse_infer_amd.ops import kernels

    tokens, outputs = 33, experts + identity
    x, xref = stored(rnd(tokens, hidden, seed=1), dtype)
    router, rref = stored(rnd(outputs, hidden, seed=2, scale=hidden ** -0.5 * 2), dtype)
    corr, cref = stored(rnd(outputs, seed=3, scale=0.6), dtype)
    z = torch.zeros(tokens, outputs, device=DEV)
    kernels.gemm_f32(x, router, z)
    idx = torch.full((tokens, top), -7, dtype=torch.int32, device=DEV)
    weight = torch.full((tokens, top), float("nan"), device=DEV)
    kernels.moe_route(z, corr, top, idx, weight)
    want_idx, want_w = P.route(z.cpu().to(F64), cref, top)
    plain_idx, _ = P.route(z.cpu().to(F64), torch.zeros_like(cref), top)
    assert not torch.equal(want_idx, plain_idx), "the correction changes no choice: the test shows nothing"
    assert torch.equal(idx.cpu().long(), want_idx)
    assert torch.allclose(weight.cpu().to(F64), want_w, atol=1e-5)
    if identity:
        assert int((want_idx >= experts).sum()) > 0
    idx2, weight2 = torch.full_like(idx, -7), torch.full_like(weight, float("nan"))
    kernels.moe_router(x, router, corr, top, idx2, weight2)          # product and routing in one kernel
    assert torch.equal(idx2, idx) and torch.allclose(weight2, weight, atol=1e-5)
    wg, gref = stored(rnd(experts, ff, hidden, seed=4, scale=hidden ** -0.5), dtype)
    wu, uref = stored(rnd(experts, ff, hidden, seed=5, scale=hidden ** -0.5), dtype)
    wd, dref = stored(rnd(experts, hidden, ff, seed=6, scale=ff ** -0.5), dtype)
    act = torch.full((tokens * top, ff), float("nan"), dtype=dtype, device=DEV)
    out = torch.full((tokens, hidden), float("nan"), device=DEV)
    kernels.moe_gate_up(x, wg, wu, idx, act)
    kernels.moe_down(x, act, wd, idx, weight, out)
    want = torch.zeros(tokens, hidden, dtype=F64)
    for t in range(tokens):
        for e, a in zip(want_idx[t].tolist(), want_w[t]):
            want[t] += a * (xref[t] if e >= experts else P.gated_expert(xref[t], gref[e], uref[e], dref[e]))
    assert torch.allclose(out.cpu().to(F64), want, **tol(dtype))
    if dtype == torch.bfloat16:
        # the same through the products grouped by expert on the matrix cores, in tiles of both heights
        assert kernels.moe_grouped_takes(x, wg, wd)
        for rows in kernels.MOE_TILE_ROWS:
            act.fill_(float("nan"))
            out.fill_(float("nan"))
            y = torch.full((tokens * top, hidden), float("nan"), device=DEV)
            ints = torch.full((2 * tokens * top + 3 * kernels.moe_max_tiles(tokens * top, experts, rows) + 1,), -5,
                              dtype=torch.int32, device=DEV)
            kernels.moe_grouped(x, wg, wu, wd, idx, weight, act, y, out, ints, rows)
            assert torch.allclose(out.cpu().to(F64), want, **tol(dtype)), rows


@pytest.mark.parametrize("rows_of", [[700, 0, 3, 130, 1, 0, 33, 129]])
def test_experts_with_many_and_with_no_rows(rows_of):
    """Tiles of the grouped products: an expert with several full tiles and a rest, experts that nobody chose, experts
    with one row; every pair's result is its own row's whatever tile it lands in."""
    from pulse_infer_amd.ops import kernels

    experts, hidden, ff, top = len(rows_of), 128, 96, 2
    pairs = sum(rows_of)
    chosen = torch.tensor([e for e, n in enumerate(rows_of) for _ in range(n)])
    chosen = chosen[torch.randperm(pairs, generator=torch.Generator().manual_seed(1))]
    tokens = pairs // top
    idx = chosen[:tokens * top].view(tokens, top).to(torch.int32).to(DEV)
    idx[5, 1] = experts          # one identity expert among them
    weight = torch.rand(tokens, top, generator=torch.Generator().manual_seed(2)).to(DEV)
    x, xref = stored(rnd(tokens, hidden, seed=3), torch.bfloat16)
    wg, gref = stored(rnd(experts, ff, hidden, seed=4, scale=hidden ** -0.5), torch.bfloat16)
    wu, uref = stored(rnd(experts, ff, hidden, seed=5, scale=hidden ** -0.5), torch.bfloat16)
    wd, dref = stored(rnd(experts, hidden, ff, seed=6, scale=ff ** -0.5), torch.bfloat16)
    want = torch.zeros(tokens, hidden, dtype=F64)
    for e in range(experts):
        rows = (idx.cpu() == e)
        for k in range(top):
            t = rows[:, k].nonzero().flatten()
            if len(t):
                want[t] += weight.cpu().to(F64)[t, k].view(-1, 1) * P.gated_expert(xref[t], gref[e], uref[e], dref[e])
    want[5] += float(weight[5, 1]) * xref[5]
    for rows in kernels.MOE_TILE_ROWS:
        act = torch.full((tokens * top, ff), float("nan"), dtype=torch.bfloat16, device=DEV)
        y = torch.full((tokens * top, hidden), float("nan"), device=DEV)
        out = torch.full((tokens, hidden), float("nan"), device=DEV)
        ints = torch.full((2 * tokens * top + 3 * kernels.moe_max_tiles(tokens * top, experts, rows) + 1,), -5,
                          dtype=torch.int32, device=DEV)
        kernels.moe_grouped(x, wg, wu, wd, idx, weight, act, y, out, ints, rows)
        assert torch.allclose(out.cpu().to(F64), want, atol=2e-2, rtol=2e-2), rows


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("hidden", [96, 1000, 4096])
def test_the_norm_after_the_sum(dtype, hidden):
    from pulse_infer_amd.ops import kernels

    rows, eps, alpha = 5, 3e-6, 2.5
    h0 = rnd(rows, hidden, seed=1, scale=3.0)
    w, wref = stored(1.0 + rnd(hidden, seed=3, scale=0.1), dtype)
    ls, lref = stored(rnd(hidden, seed=4, scale=0.5), dtype)
    d1, d1ref = stored(rnd(rows, hidden, seed=5), dtype)
    d2 = rnd(rows, hidden, seed=6).to(DEV)
    for first, second, factors in ((d1, d2, ls), (d1, None, ls), (d2, d1, None), (None, None, None)):
        h = h0.clone().to(DEV)
        copy = torch.zeros(rows, hidden, dtype=dtype, device=DEV)
        kernels.scale_add_rmsnorm(h, w, eps, alpha, first, second, factors, copy)
        update = torch.zeros(rows, hidden, dtype=F64)
        for part in (first, second):
            if part is not None:
                update = update + part.cpu().to(F64)
        if factors is not None:
            update = update * lref
        want = P.unit_rms(alpha * h0.to(F64) + update, eps) * wref
        assert torch.allclose(h.cpu().to(F64), want, atol=2e-5, rtol=2e-5)
        assert torch.allclose(copy.cpu().to(F64), want, **tol(dtype))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_activations_cap_and_scaled_embedding(dtype):
    from pulse_infer_amd.ops import kernels

    x, xref = stored(rnd(9, 70, seed=1, scale=2.0), dtype)
    for kind, fn in (("relu2", lambda z: torch.relu(z) ** 2), ("gelu_tanh", P.gelu_tanh), ("silu", P.silu)):
        out = torch.zeros_like(x)
        kernels.activation(x, out, kind)
        assert torch.allclose(out.cpu().to(F64), fn(xref), **tol(dtype)), kind
    z = rnd(4, 50, seed=2, scale=20.0).to(DEV)
    want = 7.5 * torch.tanh(z.cpu().to(F64) / 7.5)
    kernels.softcap(z, 7.5)
    assert torch.allclose(z.cpu().to(F64), want, atol=1e-5)
    table, tref = stored(rnd(11, 24, seed=3), dtype)
    out = torch.zeros(3, 24, device=DEV)
    kernels.embed_gather(ints([10, 0, 4]), table, out, torch.zeros(1, dtype=torch.int32, device=DEV), 3.0)
    assert torch.allclose(out.cpu().to(F64), tref[[10, 0, 4]] * 3.0, atol=1e-6)


# ------------------------------------------------------------------------------------------------ whole models
LENGTH = {"mixed": 150, "equal": 130, "wide": 90}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name,page", [("mixed", 16), ("mixed", 4), ("equal", 16), ("equal", 64), ("wide", 16)])
def test_whole_tail_and_portions(runners, plain, name, page, dtype):
    ids = token_ids(CONFIGS[name]["vocab"], LENGTH[name], seed=3)
    want, calls = plain(name, ids), plain.close_calls(name, ids)
    runner = runners(name, dtype, page)
    n = len(ids)
    whole = run_alone(runner, ids, [n])
    agree(whole, want, dtype, f"{name} whole", calls)
    tail = run_alone(runner, ids, [n - 40] + [1] * 40)               # prefill against token-by-token decoding
    agree(tail, want, dtype, f"{name} tail", calls)
    agree(tail, whole, dtype, f"{name} tail against whole", calls, tol=SPLIT_TOL)
    for cuts in ([2, 3, 31, 2, 17, n - 57, 2], [1, 1, 1, 31, n - 34], [n - 2, 2], [7] * (n // 7) + [n % 7 or 7][:n % 7 > 0]):
        cuts = [c for c in cuts if c]
        portions = run_alone(runner, ids, cuts)
        agree(portions, want, dtype, f"{name} portions {cuts}", calls)
        agree(portions, whole, dtype, f"{name} portions against whole", calls, tol=SPLIT_TOL)
    first = run_alone(runner, ids[:3], [1, 1, 1])                     # the first tokens of a sequence
    agree(first, want[:3], dtype, f"{name} first tokens", calls)


@pytest.mark.parametrize("name", ["mixed", "equal"])
def test_the_stream_after_every_layer(runners, plain, name):
    from pulse_infer_amd.engine.runner import StepEntry

    ids = token_ids(CONFIGS[name]["vocab"], 37, seed=8)
    runner = runners(name, "float32")
    model, seen = runner.model, []
    originals = [b.forward for b in model.blocks]

    def watched(forward):
        def run(stream, ctx, cache):
            forward(stream, ctx, cache)
            seen.append(stream.h.clone())
        return run

    try:
        for block, forward in zip(model.blocks, originals):
            block.forward = watched(forward)
        runner.add_request("layers")
        runner.reserve("layers", len(ids))
        runner.step([StepEntry("layers", ids, [])])
    finally:
        for block, forward in zip(model.blocks, originals):
            block.forward = forward
        runner.free_request("layers")
    want = plain.models[name].residuals(ids)
    assert len(seen) == len(want)
    for i, (got, ref) in enumerate(zip(seen, want)):
        close(got, ref, "float32", f"{name} after layer {i}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name,page", [("mixed", 16), ("equal", 16), ("equal", 32), ("wide", 16)])
def test_mixed_batches_with_pages_and_slots_used_again(runners, plain, name, page, dtype):
    """Up to four live requests over a pool of 256 tokens and four slots, portions of some beside single tokens of
    others: every request's logits are what it gets alone, whoever held its pages and its state's slot before."""
    ids, steps = mixed_trace(CONFIGS[name]["vocab"], seed=6, sizes=(2, 3, 5, 8, 13, 21, 34))
    runner = runners(name, dtype, page, tokens=256)
    got, pages_seen, most_live = run_mixed(runner, steps)
    assert most_live == 4 and pages_were_used_again(pages_seen)
    for k, mine in got.items():
        agree(mine, plain(name, ids[k]), dtype, f"{name} mixed request {k}", plain.close_calls(name, ids[k]))


def test_slots_and_pages_are_used_again_by_requests_of_other_lengths(runners, plain):
    from pulse_infer_amd.engine.runner import StepEntry

    name = "mixed"
    runner = runners(name, "float32", 16, tokens=160)
    for storage in runner.cache.state.values():       # whatever a slot held before must not show
        storage.fill_(float("nan"))
    lengths = [70, 3, 64, 17, 1, 80, 33, 16, 65, 48]
    for i in range(0, len(lengths), 2):
        pair = {f"q{i + j}": token_ids(CONFIGS[name]["vocab"], n, seed=40 + i + j) for j, n in enumerate(lengths[i:i + 2])}
        for rid, ids in pair.items():
            runner.add_request(rid)
            runner.reserve(rid, len(ids))
        logits = runner.step([StepEntry(rid, ids, [len(ids) - 1]) for rid, ids in pair.items()])
        for row, (rid, ids) in enumerate(pair.items()):
            close(logits[row:row + 1], plain(name, ids)[-1:], "float32", f"request {rid} of {len(ids)} tokens")
            runner.free_request(rid)
        runner.cache.check()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_long_prompt_far_beyond_the_windows(runners, plain, dtype):
    """400 tokens through windows of 7 and 24 (pages below the windows go back to the pool while the request runs)
    and through states that keep everything (a decay of one): whole, and with the last 60 tokens decoded."""
    name = "mixed"
    ids = token_ids(CONFIGS[name]["vocab"], 400, seed=21)
    want, calls = plain(name, ids), plain.close_calls(name, ids)
    runner = runners(name, dtype, 16, tokens=512)
    agree(run_alone(runner, ids, [400]), want, dtype, "whole", calls)
    agree(run_alone(runner, ids, [150, 190] + [1] * 60), want, dtype, "decoded tail", calls)


# ------------------------------------------------------------------------------------ seeded random configurations
def random_config(rng):
    """Layers drawn one by one: head sizes that are no multiples of 16, keys wider or narrower than values, any
    grouping of heads, windows from one token on, rotations on a part of a head, inner widths that are no multiples of
    8 (the experts' products then take the kernel without matrix cores), routers that choose all their outputs."""
    width = rng.choice([64, 96, 160, 256])
    layers = []
    for _ in range(rng.choice([1, 2, 3])):
        heads = rng.choice([1, 2, 3, 5])
        light = lightning(heads, rng.choice([16, 24, 32, 64]), rng.choice([16, 20, 32, 72]),
                          [rng.choice([0.0, 0.5, 0.9, 0.99, 1.0]) for _ in range(heads)])
        if rng.random() < 0.6:
            groups, share = rng.choice([1, 2, 3]), rng.choice([1, 2, 3, 4])
            dim = rng.choice([16, 24, 32, 48, 64])
            rot = rng.choice([d for d in (0, 2, 8, 16, 24, dim) if d <= dim])      # (0: the configuration names no rotation)
            mixer = parallel(left(groups * share, groups, dim, rng.choice([8, 16, 40, 48, 64]),
                                  rng.choice([1, 5, 16, 33, 100, None]),
                                  rot, rng.choice([100.0, 1e4, 5e5]), rng.choice([0.1, dim ** -0.5, 0.5])),
                             light, rng.choice([0.5, 1.0, 1.5]), rng.choice([0.7, 1.0]))
        else:
            mixer = light
        kind = rng.choice(["none", "dense", "moe", "moe"])
        if kind == "none":
            mlp = None
        elif kind == "dense":
            mlp = dense(rng.choice([32, 100, 256]))
        else:
            experts, identity = rng.choice([1, 2, 4, 9]), rng.choice([0, 1, 3])
            mlp = moe(experts, identity, rng.randint(1, min(4, experts + identity)), rng.choice([32, 40, 64, 100]),
                      rng.choice([None, 48, 128]))
        layers.append(layer(mixer, mlp))
    return config(rng.choice([257, 300, 1000]), width, rng.choice([1e-6, 1e-5]), rng.choice([1.0, 2.5, 4.0]),
                  rng.choice([1.0, 3.0]), rng.choice([5.0, 15.0, 50.0]), layers)


@pytest.mark.parametrize("seed", range(12))
def test_random_configurations(tmp_path, seed):
    """Whole, with the last 20 tokens one by one, and in portions of 2 to 70 tokens, in 32-bit and in bfloat16."""
    if not torch.cuda.is_available():
        pytest.skip("no GPU visible")
    import random

    from pulse_infer_amd.config import KesovikConfig
    from pulse_infer_amd.engine.runner import ModelRunner
    from pulse_infer_amd.models.factory import load_model
    from pulse_infer_amd.weights import write_model_folder

    rng = random.Random(7000 + seed)
    cfg = random_config(rng)
    length = rng.choice([90, 150])
    folder = write_model_folder(KesovikConfig.from_dict(cfg), str(tmp_path / "m"), seed=seed)
    oracle = P.PlainKesovik.from_folder(folder)
    ids = token_ids(cfg["vocab"], length, seed=seed)
    want = oracle.logits(ids)
    calls = set((oracle.router_margins(ids) < CLOSE_CALL).nonzero().flatten().tolist())
    what = f"{cfg} length {length}"
    for dtype in ("float32", "bfloat16"):
        _, model = load_model(folder, mode=dtype)
        runner = ModelRunner(model, page_size=16, num_pages=16, max_requests=4)
        whole = run_alone(runner, ids, [length])
        agree(whole, want, dtype, f"whole: {what}", calls, carried=True)
        agree(run_alone(runner, ids, [length - 20] + [1] * 20), want, dtype, f"tail: {what}", calls, carried=True)
        cuts, left_over, sizes = [], length, [40, 2, 17, 3, 70, 5, 19]
        while left_over:
            n = min(sizes[len(cuts) % len(sizes)], left_over)
            cuts.append(n)
            left_over -= n
        agree(run_alone(runner, ids, cuts), want, dtype, f"portions {cuts}: {what}", calls, carried=True)
        del runner, model
    torch.cuda.empty_cache()


# ------------------------------------------------------------------------------------------------ long decoding
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["mixed", "wide"])
def test_long_decoding_of_three_requests(runners, plain, name, dtype):
    """Three requests of unequal prompts decode 100 tokens together, over page borders and out of every window; in
    bfloat16 the steps are recorded and replayed."""
    from pulse_infer_amd.engine.runner import StepEntry

    vocab, new = CONFIGS[name]["vocab"], 100
    runner = runners(name, dtype, 16, tokens=704)
    prompt = {"d0": 1, "d1": 30, "d2": 47}
    ids = {k: token_ids(vocab, n + new, seed=60 + i) for i, (k, n) in enumerate(prompt.items())}
    replays = runner.graph_replays
    got = {k: [] for k in ids}
    for k in ids:
        runner.add_request(k)
        runner.reserve(k, prompt[k])
    first = runner.step([StepEntry(k, ids[k][:prompt[k]], [prompt[k] - 1]) for k in ids])
    for row, k in enumerate(ids):
        got[k].append(first[row:row + 1])
    for step in range(new):
        for k in ids:
            runner.reserve(k, prompt[k] + step + 1)
        logits = runner.step([StepEntry(k, [ids[k][prompt[k] + step]], [0]) for k in ids])
        for row, k in enumerate(ids):
            got[k].append(logits[row:row + 1])
    for k in ids:
        runner.free_request(k)
        agree(torch.cat(got[k]), plain(name, ids[k])[prompt[k] - 1:], dtype, f"{name} decoding request {k}",
              plain.close_calls(name, ids[k]), first=prompt[k] - 1)
    if dtype == "bfloat16" and runner.model.recordable(list(range(3))):
        assert runner.graph_replays > replays, "no decoding step was replayed from a recording"


# --------------------------------------------------------------------------- generation through the scheduler
@pytest.mark.parametrize("name", ["mixed", "equal"])
def test_greedy_generation_through_the_engine(folders, plain, name):
    """In 32-bit the greedy choice does not depend on the batch: requests generated together, in small portions and
    with a pool so tight that some are preempted and recomputed (their states start again from zero), give what
    each gives alone and what the plain implementation chooses."""
    from pulse_infer_amd import LLM

    vocab, new, page = CONFIGS[name]["vocab"], 12, 16
    prompts = [token_ids(vocab, n, seed=80 + i) for i, n in enumerate((1, 5, 18, 40, 77))]
    make = lambda **kw: LLM.from_pretrained(folders[name], dtype="float32", page_size=page, **kw)
    alone = [make(max_batch_size=1, chunk_size=256, num_pages=32).generate([p], max_new_tokens=new, ignore_eos=True)[0]
             for p in prompts]
    assert alone == [plain.models[name].greedy(p, new) for p in prompts]
    roomy = make(max_batch_size=4, chunk_size=16, num_pages=64, max_num_batched_tokens=24)
    assert roomy.generate(prompts, max_new_tokens=new, ignore_eos=True) == alone
    need = max((len(p) + new + page - 1) // page for p in prompts)
    tight = make(max_batch_size=4, chunk_size=16, num_pages=need + 2)
    assert tight.generate(prompts, max_new_tokens=new, ignore_eos=True) == alone
    tight.engine.runner.cache.check()


def test_bfloat16_generation_stays_within_rounding_of_the_plain_choice(folders, plain):
    from pulse_infer_amd import LLM

    name, new = "wide", 10
    prompts = [token_ids(CONFIGS[name]["vocab"], n, seed=90 + i) for i, n in enumerate((3, 21))]
    llm = LLM.from_pretrained(folders[name], dtype="bfloat16", max_batch_size=2, chunk_size=8, page_size=16, num_pages=32)
    for prompt, out in zip(prompts, llm.generate(prompts, max_new_tokens=new, ignore_eos=True)):
        assert len(out) == new
        for t, token in enumerate(out):
            row = plain(name, prompt + out[:t])[-1]
            assert float(row[token]) >= float(row.max()) - 3e-2 * float(row.abs().max())


def test_the_command_line_generates(folders, plain):
    name = "equal"
    prompt = token_ids(CONFIGS[name]["vocab"], 9, seed=99)
    run = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "pulse_infer"), folders[name], "--dtype", "float32",
                          "--prompt-ids", ",".join(map(str, prompt)), "--max-new-tokens", "6", "--greedy",
                          "--ignore-eos", "--max-positions", "64"], capture_output=True, text=True, timeout=300)
    assert run.returncode == 0, run.stderr[-2000:]
    out = json.loads(run.stdout.strip().splitlines()[0])
    assert out["output_ids"] == plain.models[name].greedy(prompt, 6)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_replay_program(folders, plain, tmp_path, dtype):
    import numpy as np

    name = "mixed"
    vocab = CONFIGS[name]["vocab"]
    a, b = token_ids(vocab, 70, seed=1), token_ids(vocab, 21, seed=2)
    steps = [
        {"step": 0, "entries": [{"id": "a", "tokens": a[:50], "want": [0, 49]}], "end": []},
        {"step": 1, "entries": [{"id": "a", "tokens": a[50:69], "want": []}, {"id": "b", "tokens": b[:20], "want": [19]}],
         "end": []},
        {"step": 2, "entries": [{"id": "b", "tokens": b[20:], "want": [0]}, {"id": "a", "tokens": a[69:], "want": [0]}],
         "end": ["a", "b"]},
    ]
    out = tmp_path / f"out_{dtype}"
    run = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", folders[name], "--dtype", dtype,
                          "--out", str(out), "--max-tokens", "192"], input="\n".join(json.dumps(s) for s in steps) + "\n",
                         capture_output=True, text=True, timeout=300)
    assert run.returncode == 0, run.stderr[-2000:]
    assert [line for line in run.stdout.splitlines() if line.startswith("done")] == ["done 0", "done 1", "done 2"]
    la, lb = plain(name, a), plain(name, b)
    read = lambda i: torch.from_numpy(np.fromfile(out / f"{i}.f32", dtype="<f4").reshape(-1, vocab).copy())
    close(read(0), la[[0, 49]], dtype, "step 0")
    close(read(1), lb[[19]], dtype, "step 1")
    close(read(2), torch.stack([lb[20], la[69]]), dtype, "step 2")
