"""The Titozen decoder in the engine against its plain statement (plain_titozen.py), on the GPU: each mechanism alone,
then whole models under every way of cutting and batching, in 32-bit and in bfloat16, at sizes of the tests' own."""
import json
import os

import numpy as np
import pytest
import torch

import helpers as H
import plain_titozen as pt

pytestmark = pytest.mark.gpu

HG = lambda heads, dim, vdim: dict(heads=heads, dim=dim, vdim=vdim)
LA = lambda heads, dim, vdim, q_rank, kv_rank, scale, window: dict(
    heads=heads, dim=dim, vdim=vdim, q_rank=q_rank, kv_rank=kv_rank, scale=scale, mask=dict(size=window))
FF = lambda ff, limit: dict(kind="dense", ff=ff, limit=limit)


def config(width, vocab, taps, layers, eps=1e-5):
    return dict(architecture="Titozen", vocab=vocab, width=width, norm=dict(eps=eps), canon=dict(taps=taps),
                layers=[dict(type=t, mixer=m, mlp=f) for t, m, f in layers])


# Sizes that differ from one another wherever the design allows it: key, value and latent widths all unequal, ranks that
# are no multiple of 8, more heads than a workgroup takes, windows that are no multiple of a page, layers without a
# feed-forward, one tap (no convolution state), a window of one key.
MIXED = config(96, 211, 3, [
    ("hgrn2", HG(3, 20, 24), FF(136, 1.25)),
    ("latent_attention", LA(5, 24, 40, 56, 48, 0.3, 19), None),
    ("hgrn2", HG(2, 33, 17), FF(72, 0.75)),
    ("latent_attention", LA(2, 16, 8, 12, 20, 0.21, 37), FF(64, 2.0)),
])
ATTENTION_ONLY = config(64, 150, 2, [
    ("latent_attention", LA(9, 8, 16, 24, 136, 0.5, 23), None),
    ("latent_attention", LA(3, 32, 24, 40, 264, 0.11, 1), FF(80, 1.5)),
    ("latent_attention", LA(1, 40, 48, 16, 64, 0.2, 300), None),
], eps=3e-6)
RECURRENT_ONLY = config(72, 97, 1, [
    ("hgrn2", HG(1, 130, 20), None),
    ("hgrn2", HG(4, 7, 70), FF(40, 1.0)),
    ("hgrn2", HG(2, 64, 64), None),
], eps=1e-6)
FIVE_TAPS = config(40, 64, 5, [("hgrn2", HG(2, 16, 16), None), ("latent_attention", LA(2, 16, 16, 16, 16, 0.25, 8), FF(48, 1.5))])
CONFIGS = {"mixed": (MIXED, 8), "attention": (ATTENTION_ONLY, 16), "recurrent": (RECURRENT_ONLY, 16), "taps": (FIVE_TAPS, 8)}


def make_folder(path, cfg, seed, std_scale=5.0, edit=None):
    """A model folder with random weights, stored in bfloat16 as this design's checkpoints are (so the 32-bit engine, the
    bfloat16 engine and the plain statement all start from the same numbers); `edit(tensors)` may change them before
    they are written."""
    folder = H.make_model_folder(path, cfg, seed, "bfloat16", std_scale=std_scale)
    if edit is not None:
        from safetensors.torch import load_file, save_file
        file = os.path.join(folder, "model.safetensors")
        tensors = {k: v.clone() for k, v in load_file(file).items()}
        edit(tensors)
        save_file(tensors, file)
    return folder


def sharpen(tensors):
    """Peaked attention and long memory: the queries four times as large (one key takes most of a softmax, so a key
    that is wrongly seen or missed moves the result), sinks that hold a visible share, and a third of the recurrence's
    channels with a forget gate near one (what was written hundreds of tokens ago still counts)."""
    for name, t in tensors.items():
        if name.endswith(".mix.uq"):
            t *= 4.0
        if name.endswith(".mix.sink"):
            t += 1.0
        if name.endswith(".mix.lower"):
            t[::3] = 63.0 / 64.0


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    return {name: make_folder(tmp_path_factory.mktemp(name), cfg, seed=i, edit=sharpen)
            for i, (name, (cfg, _)) in enumerate(CONFIGS.items())}


def runner_for(folder, name, dtype, tokens=1024, max_requests=4, **kw):
    from ginfer_amd import ModelRunner
    ps = CONFIGS[name][1]
    return ModelRunner(folder, dtype=dtype, page_size=ps, num_pages=-(-tokens // ps), max_requests=max_requests, **kw)


def requests_for(name, lengths, seed=20):
    return {"q%d" % i: H.random_tokens(n, CONFIGS[name][0]["vocab"], seed + i) for i, n in enumerate(lengths)}


_plain = {}


def plain(folder, ids):
    key = (folder, tuple(ids))
    if key not in _plain:
        _plain[key] = pt.logits(folder, ids)
    return _plain[key]


def compare(got, requests, folder, tol, what):
    worst = 0.0
    for (rid, p), row in sorted(got.items()):
        ref = plain(folder, requests[rid])
        assert np.isfinite(row).all(), "%s: request %s position %d: non-finite logits" % (what, rid, p)
        err = float(np.abs(row.astype(np.float64) - ref[p]).max() / np.abs(ref).max())
        assert err <= tol, ("%s: first wrong place is request %s position %d of %d: error %.3g > %.3g"
                            % (what, rid, p, len(requests[rid]), err, tol))
        worst = max(worst, err)
    for rid, ids in requests.items():
        missing = [p for p in range(len(ids)) if (rid, p) not in got]
        assert not missing, "%s: request %s lacks logits at %s" % (what, rid, missing[:8])
    return worst


# 32-bit differs from the 64-bit plain statement by the rounding of a few hundred terms per sum; bfloat16 rounds every
# stored activation to 8 bits, and peaked softmaxes pass that on
TOL = {"float32": 2e-5, "bfloat16": 5e-2}


# ----------------------------------------------------------------------------------------------- mechanisms alone

class _Step:
    """The few arrays of a step that the kernels under test read."""

    def __init__(self, q_len, q_start):
        dev = torch.device("cuda")
        cu = np.concatenate([[0], np.cumsum(q_len)]).astype(np.int32)
        self.cu_tokens = torch.tensor(cu, device=dev)
        self.q_start = torch.tensor(q_start, dtype=torch.int32, device=dev)
        self.token_entry = torch.tensor(np.repeat(np.arange(len(q_len)), q_len), dtype=torch.int32, device=dev)
        self.positions = torch.tensor(np.concatenate([np.arange(s, s + n) for s, n in zip(q_start, q_len)]), dtype=torch.int32,
                                      device=dev)


def test_norm_with_one_gain():
    from ginfer_amd.kernels import ops
    g = torch.Generator().manual_seed(0)
    for H_ in (7, 96, 328, 1000):
        x = torch.randn((5, H_), generator=g) * 3
        y = torch.randn((5, H_), generator=g)
        gain = torch.tensor([0.7])
        rows = torch.tensor([4, 0, 4], dtype=torch.int32)
        got = ops.scalar_rmsnorm_rows(x.cuda(), gain.cuda(), 1e-5, torch.float32, rows=rows.cuda()).cpu()
        ref = pt.scalar_norm(x.double(), 0.7, 1e-5)[rows.long()]
        assert H.rel_err(got, ref) < 1e-6
        res = x.cuda().clone()
        copy = ops.add_scalar_rmsnorm(res, y.cuda().to(torch.bfloat16), gain.cuda().to(torch.bfloat16), 1e-5, copy=True)
        ref = x.double() + pt.scalar_norm(y.to(torch.bfloat16).double(), float(gain.to(torch.bfloat16)), 1e-5)
        assert H.rel_err(res.cpu(), ref) < 1e-6 and copy.dtype == torch.bfloat16
        assert H.rel_err(copy.float().cpu(), ref) < 5e-3


def test_embedding_with_position_vectors_far_into_a_sequence():
    from ginfer_amd.kernels import ops
    g = torch.Generator().manual_seed(1)
    for width in (6, 96, 321):
        table = torch.randn((50, width), generator=g)
        ids = torch.randint(0, 50, (9,), generator=g)
        pos = torch.tensor([0, 1, 2, 63, 64, 1000, 4097, 70001, 1000000], dtype=torch.int32)
        i = torch.arange((width + 1) // 2, dtype=torch.float64)
        freq = torch.pow(torch.tensor(10000.0, dtype=torch.float64), -2.0 * i / width).float()
        got = ops.embedding_sinusoid_norm(table.cuda(), ids.int().cuda(), pos.cuda(), freq.cuda(), torch.tensor([1.3]).cuda(), 1e-5)
        p_all = pt.position_vectors(1000001, width, torch.float64) if width == 6 else None
        for r in range(9):
            pv = p_all[int(pos[r])] if p_all is not None else pt.position_vectors(int(pos[r]) + 1, width, torch.float64)[-1] \
                if int(pos[r]) < 100000 else None
            if pv is None:
                continue
            ref = pt.scalar_norm(table[ids[r]].double() + pv, 1.3, 1e-5)
            assert H.rel_err(got[r].cpu(), ref) < 2e-6, (width, r)


@pytest.mark.parametrize("taps", [1, 2, 4, 7])
def test_short_convolution_across_cuts_and_slots(taps):
    """Two requests whose tokens come in portions (down to one token, shorter than the taps) in state slots that are not
    their entries' numbers; a third request then starts in a slot that was used before."""
    from ginfer_amd.kernels import ops
    W = 37
    g = torch.Generator().manual_seed(taps)
    w = torch.randn((W, taps), generator=g)
    xs = {"a": torch.randn((23, W), generator=g), "b": torch.randn((9, W), generator=g), "c": torch.randn((6, W), generator=g)}
    refs = {k: pt.input_convolution(x.double(), w.double()) for k, x in xs.items()}
    state = torch.full((4, max(taps - 1, 1), W), 7.0).cuda()[:, :taps - 1].contiguous() if taps > 1 else None
    slot = {"a": 2, "b": 0, "c": 2}
    plan = [[("a", 5), ("b", 1)], [("b", 1), ("a", 1)], [("a", 2), ("b", 7)], [("a", 15)], [("c", 2)], [("c", 4)]]
    at = {k: 0 for k in xs}
    for entries in plan:
        step = _Step([n for _, n in entries], [at[k] for k, _ in entries])
        x = torch.cat([xs[k][at[k]:at[k] + n] for k, n in entries]).cuda()
        slots = torch.tensor([slot[k] for k, _ in entries], dtype=torch.int64).cuda()
        got = ops.short_conv(x, w.cuda(), state, slots if taps > 1 else None, step, torch.float32).cpu()
        o = 0
        for k, n in entries:
            assert H.rel_err(got[o:o + n], refs[k][at[k]:at[k] + n]) < 1e-6, (taps, k, at[k], n)
            o += n
            at[k] += n


@pytest.mark.parametrize("heads,dim,vdim", [(1, 5, 3), (3, 40, 72), (2, 130, 20), (2, 16, 100), (1, 256, 16)])
def test_gated_recurrence_across_cuts(heads, dim, vdim):
    """The recurrence of one request in portions of 1 to 40 tokens beside another request, against the plain loop; the
    forget gates reach from 0.02 to 0.98, so both what fades at once and what stays for the whole sequence count."""
    from ginfer_amd.kernels import ops
    g = torch.Generator().manual_seed(dim)
    T = 90
    cols = 2 * heads * dim + heads * vdim
    proj = {k: torch.randn((T, cols), generator=g) * 2 for k in "ab"}
    bias = torch.randn((heads * dim,), generator=g)
    lower = torch.rand((heads * dim,), generator=g) * 0.96 + 0.02
    refs = {}
    for k in "ab":
        p = proj[k].double()
        q = torch.nn.functional.silu(p[:, :heads * dim]).view(T, heads, dim)
        f = (lower.double() + (1 - lower.double()) * torch.sigmoid(p[:, heads * dim:2 * heads * dim] + bias.double())).view(T, heads, dim)
        v = p[:, 2 * heads * dim:].view(T, heads, vdim)
        S = torch.zeros((heads, dim, vdim), dtype=torch.float64)
        out = torch.zeros((T, heads, vdim), dtype=torch.float64)
        for t in range(T):
            S = f[t][:, :, None] * S + (1 - f[t])[:, :, None] * v[t][:, None, :]
            out[t] = torch.einsum("hdv,hd->hv", S, q[t])
        refs[k] = out
    state = torch.full((3, heads, dim, vdim), 5.0).cuda()          # what an earlier request left in the slots
    slot = {"a": 2, "b": 1}
    at = {"a": 0, "b": 0}
    for cut_a, cut_b in [(1, 40), (2, 17), (17, 1), (40, 16), (30, 16)]:
        entries = [("a", cut_a), ("b", cut_b)]
        step = _Step([n for _, n in entries], [at[k] for k, _ in entries])
        x = torch.cat([proj[k][at[k]:at[k] + n] for k, n in entries]).cuda()
        slots = torch.tensor([slot[k] for k, _ in entries], dtype=torch.int64).cuda()
        got = ops.hgrn2_scan(x, bias.cuda(), lower.cuda(), state, slots, step, heads, dim, vdim).cpu()
        o = 0
        for k, n in entries:
            assert H.rel_err(got[o:o + n], refs[k][at[k]:at[k] + n]) < 2e-6, (k, at[k], n)
            o += n
            at[k] += n
    assert at == {"a": 90, "b": 90}
    w = torch.randn((vdim,), generator=g)
    got = ops.headwise_rmsnorm(refs["a"].float().cuda(), w.cuda(), 1e-5, torch.float32).cpu()
    assert H.rel_err(got, pt.rms(refs["a"], 1e-5) * w.double()) < 1e-6


@pytest.mark.parametrize("rank,heads,window,page", [(64, 5, 70, 16), (20, 2, 5, 8), (136, 9, 33, 16), (264, 3, 64, 32), (48, 1, None, 8)])
def test_latent_attention_sees_exactly_its_window(rank, heads, window, page):
    """One request of 150 cached rows.  The rows just inside and just outside the window of the last tokens, the first
    rows of the sequence, a row a hundred back and the rows at the borders of pages are made to match the query twenty
    times as well as any other, one at a time: where such a row is seen it takes the whole softmax, where it is not it
    must leave no trace.  A sink that is larger than every score holds most of the mass in another run."""
    from ginfer_amd.kernels import ops
    g = torch.Generator().manual_seed(rank)
    n, T = 150, 3                                   # the last T rows are the step's tokens
    pages = -(-n // page)
    order = torch.randperm(pages + 3, generator=g)[:pages]            # the request's pages lie anywhere in the pool
    table = order.int()[None, :].contiguous()
    qa = torch.randn((heads, T, rank), generator=g)
    base = torch.randn((n, rank), generator=g) * 0.3
    gate = torch.rand((T, heads), generator=g)
    w = window or n + 1
    p_last = n - 1
    marked = [p_last - w, p_last - w + 1, p_last - w + 2, 0, 1, p_last - 100, page - 1, page, p_last - 1, p_last]
    for sink_value in (None, -2.0, 60.0):
        sink = None if sink_value is None else torch.full((heads,), sink_value) + torch.arange(heads) * 0.1
        for mark in [None] + [m for m in marked if 0 <= m < n]:
            c = base.clone()
            if mark is not None:
                c[mark] = qa[0, T - 1] / qa[0, T - 1].norm() * 20.0
            pool = torch.full((pages + 3, page * rank), float("nan"))          # what lies in pages nobody wrote
            for b in range(pages):
                rows = c[b * page:(b + 1) * page]
                pool[order[b], :rows.numel()] = rows.reshape(-1)
                pool[order[b], rows.numel():] = 0.0
            step = _Step([T], [n - T])
            got = ops.latent_attention(qa.cuda(), pool.cuda(), table.cuda(), step, None if sink is None else sink.cuda(),
                                       gate.cuda(), heads, rank, page, 0.37, window, torch.float32).cpu()
            for t in range(T):
                i = n - T + t
                lo = max(0, i - w + 1)
                s = torch.einsum("hr,jr->hj", qa[:, t].double(), c[lo:i + 1].double()) * 0.37
                top = s.max(dim=1).values if sink is None else torch.maximum(s.max(dim=1).values, sink.double())
                e = torch.exp(s - top[:, None])
                den = e.sum(dim=1) + (0 if sink is None else torch.exp(sink.double() - top))
                ref = torch.einsum("hj,jr->hr", e / den[:, None], c[lo:i + 1].double()) * gate[t].double()[:, None]
                err = float((got[:, t].double() - ref).abs().max() / max(float(ref.abs().max()), 1e-3))
                assert err < 2e-5, "mark %s, sink %s, token %d: %.3g" % (mark, sink_value, i, err)


@pytest.mark.parametrize("rank,heads,window,page", [(64, 7, 75, 16), (48, 3, 19, 8), (128, 20, 33, 16), (256, 5, 100, 32),
                                                    (512, 17, None, 16), (136, 2, 40, 64)])
def test_latent_attention_on_the_matrix_cores(rank, heads, window, page):
    """bfloat16, both copies of the latent in the pages.  Three requests in one step: a portion of 21 tokens behind 140
    cached ones, a single token behind 90, and a request's first 5 tokens (so a group of 16 neighbouring tokens holds two
    requests); then a step of single tokens only, with the keys of each dealt to several workgroups.  In each, one row
    just inside or just outside a window, or a far one, matches a query twenty times as well as the others."""
    from ginfer_amd.kernels import ops
    from ginfer_amd.kernels.tuning import TUNING
    g = torch.Generator().manual_seed(rank + heads)
    lens = [161, 91, 5]                              # cached + new tokens of the three requests
    new = [21, 1, 5]
    w = window or 10 ** 6
    per_req = [-(-n // page) for n in lens]
    order = torch.randperm(sum(per_req) + 2, generator=g)
    width = max(per_req)
    table = torch.full((3, width), -1, dtype=torch.int32)
    rows, o = [], 0
    for i, n in enumerate(lens):
        table[i, :per_req[i]] = order[o:o + per_req[i]].int()
        o += per_req[i]
        rows.append((torch.randn((n, rank), generator=g) * 0.3).to(torch.bfloat16))
    T = sum(new)
    qa = torch.randn((heads, T, rank), generator=g)
    # request 0: the last token's query finds the row just outside its window, the one before it the row just inside its own
    last0 = new[0] - 1
    for tok, key in ((last0, lens[0] - 1 - w), (last0 - 1, lens[0] - 2 - w + 1), (last0 - 2, 3), (new[0], lens[1] - 1 - w + 1)):
        if 0 <= key:
            req = 0 if tok <= last0 else 1
            rows[req][key] = (qa[0, tok] / qa[0, tok].norm() * 20.0).to(torch.bfloat16)
    pool = torch.zeros((sum(per_req) + 2, page * rank), dtype=torch.bfloat16)
    pool_t = torch.zeros_like(pool)
    for i, n in enumerate(lens):
        for b in range(per_req[i]):
            blk = rows[i][b * page:(b + 1) * page]
            full = torch.zeros((page, rank), dtype=torch.bfloat16)
            full[:blk.shape[0]] = blk
            pool[table[i, b]] = full.reshape(-1)
            pool_t[table[i, b]] = full.t().contiguous().reshape(-1)
    gate = torch.rand((T, heads), generator=g)
    sink = torch.randn((heads,), generator=g)

    def reference(step_new, which):
        out = torch.zeros((heads, sum(step_new), rank), dtype=torch.float64)
        t = 0
        for i, n in zip(which, step_new):
            for k in range(n):
                p = lens[i] - n + k
                lo = max(0, p - w + 1)
                c = rows[i][lo:p + 1].double()
                q = qa_step[:, t].to(torch.bfloat16).double()
                s = torch.einsum("hr,jr->hj", q, c) * 0.37
                top = torch.maximum(s.max(dim=1).values, sink.double())
                e = torch.exp(s - top[:, None])
                den = e.sum(dim=1) + torch.exp(sink.double() - top)
                out[:, t] = torch.einsum("hj,jr->hr", e / den[:, None], c) * gate_step[t].double()[:, None]
                t += 1
        return out

    for step_new, which in ((new, [0, 1, 2]), ([1, 1], [0, 1])):
        Ts = sum(step_new)
        qa_step, gate_step = qa[:, :Ts].contiguous(), gate[:Ts].contiguous()
        step = _Step(step_new, [lens[i] - n for i, n in zip(which, step_new)])
        singles = [(int(step.cu_tokens[j]), lens[i] - 1, j, 0) for j, (i, n) in enumerate(zip(which, step_new)) if n == 1]
        step.extra = {"decode_info": torch.tensor(singles, dtype=torch.int32).reshape(-1, 4).cuda(), "decode_span": 256}
        step.max_kv_len = max(lens)
        tbl = table[which].contiguous().cuda()
        for splits in (1, 32):
            old = TUNING.latent_decode_max_splits
            TUNING.latent_decode_max_splits = splits
            try:
                got = ops.latent_attention(qa_step.cuda(), pool.cuda(), tbl, step, sink.cuda(), gate_step.cuda(), heads, rank, page,
                                           0.37, window, torch.bfloat16, ct_pages=pool_t.cuda()).float().cpu()
            finally:
                TUNING.latent_decode_max_splits = old
            ref = reference(step_new, which)
            for t in range(Ts):
                err = float((got[:, t].double() - ref[:, t]).abs().max() / max(float(ref[:, t].abs().max()), 1e-2))
                assert err < 3e-2, "step %s, splits %d, token %d: %.3g" % (step_new, splits, t, err)


def test_bounded_gated_activation():
    from ginfer_amd.kernels import ops
    g = torch.Generator().manual_seed(3)
    for inter in (5, 64, 136):
        gu = torch.randn((7, 2 * inter), generator=g) * 3
        got = ops.clamped_glu(gu.cuda(), 1.25, 1.702, 1.0).cpu()
        a = torch.clamp(gu[:, :inter].double(), max=1.25)
        u = torch.clamp(gu[:, inter:].double(), -1.25, 1.25)
        assert H.rel_err(got, a * torch.sigmoid(1.702 * a) * (u + 1)) < 1e-6
        assert float(gu[:, :inter].max()) > 1.25 and float(gu[:, inter:].min()) < -1.25      # the bounds were reached


@pytest.mark.parametrize("rows,inter", [(1, 136), (8, 2048), (16, 8960), (40, 256)])
def test_gated_product_with_the_bounded_gate_in_its_epilogue(rows, inter):
    """The decode step's gate-up product with the bounded activation folded in, against the plain formula on the same
    bfloat16 operands; the sizes take the kernel's ordinary tiles and the evenly dealt ones."""
    from ginfer_amd.kernels import ops
    g = torch.Generator().manual_seed(rows + inter)
    x = (torch.randn((rows, 192), generator=g) * 0.5).to(torch.bfloat16)
    w = (torch.randn((2 * inter, 192), generator=g) * 0.25).to(torch.bfloat16)
    got = ops.gemm_skinny(x.cuda(), w.cuda(), gated=True, gate_bounds=(1.25, 1.702, 1.0)).float().cpu()
    a = torch.clamp(x.double() @ w[:inter].double().T, max=1.25)
    u = torch.clamp(x.double() @ w[inter:].double().T, -1.25, 1.25)
    ref = a * torch.sigmoid(1.702 * a) * (u + 1)
    assert float((x.double() @ w[:inter].double().T).max()) > 1.25                 # the bound was reached
    assert H.rel_err(got, ref) < 1e-2
    # and without bounds the same entry computes the plain SiLU gate
    plain = ops.gemm_skinny(x.cuda(), w.cuda(), gated=True).float().cpu()
    gate, up = x.double() @ w[:inter].double().T, x.double() @ w[inter:].double().T
    assert H.rel_err(plain, torch.nn.functional.silu(gate) * up) < 1e-2


# ----------------------------------------------------------------------------------------------- whole models

@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(CONFIGS))
def test_whole_decoded_and_in_portions(folders, name, dtype):
    """Every request whole; then most of it in one step and the rest token by token (past every window of the tests'
    models); then in portions of 1 to 64 tokens.  In 32-bit the three agree to the bit."""
    reqs = requests_for(name, [1, 2, 5, 44, 131])
    runner = runner_for(folders[name], name, dtype)
    got = {}
    for what, steps in (("whole", H.steps_whole(reqs)), ("decoded", H.steps_last_decoded(reqs, last=48)),
                        ("portions", H.steps_portions(reqs)), ("pairs", H.steps_portions(reqs, sizes=(2,)))):
        got[what] = H.run_steps(runner, steps)
        runner.cache.check()
        compare(got[what], reqs, folders[name], TOL[dtype], "%s %s %s" % (name, dtype, what))
    if dtype == "float32":
        for what in ("decoded", "portions", "pairs"):
            for key, row in got["whole"].items():
                assert np.array_equal(row, got[what][key]), "%s: %s differs from whole at %s" % (name, what, key)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["mixed", "attention", "recurrent"])
def test_unequal_requests_together_with_pages_and_slots_used_again(folders, name, dtype):
    """Seven requests through three state slots and a pool that holds three of them: portions of some beside single
    tokens of others, requests that sit a step out, and every page and slot used several times."""
    reqs = requests_for(name, [70, 3, 120, 33, 64, 17, 90], seed=50)
    steps = H.steps_mixed(reqs, max_live=3, seed=4)
    ps = CONFIGS[name][1]
    tokens = H.max_live_tokens(steps, round_to=ps)
    runner = runner_for(folders[name], name, dtype, tokens=tokens, max_requests=3)
    for rounds in range(2):                      # the second time the steps' shapes are known and recorded
        got = H.run_steps(runner, steps)
        runner.cache.check()
        compare(got, reqs, folders[name], TOL[dtype], "%s %s mixed, round %d" % (name, dtype, rounds))
    assert not runner.cache.requests


def drawn_config(seed):
    """A configuration drawn at random: any order of the two kinds of layers, widths and ranks that are multiples of 8 or
    not, one to nine heads, windows from one key to longer than the sequences, with and without a feed-forward."""
    rng = np.random.RandomState(seed)
    pick = lambda *xs: xs[rng.randint(len(xs))]
    width = int(pick(24, 40, 52, 64, 96, 136, 200))
    layers = []
    for _ in range(rng.randint(1, 5)):
        mlp = None if rng.rand() < 0.3 else FF(int(pick(16, 36, 64, 100, 192)), float(pick(0.5, 1.0, 1.5, 3.0)))
        if rng.rand() < 0.5:
            layers.append(("hgrn2", HG(int(rng.randint(1, 6)), int(pick(4, 8, 13, 16, 32, 48, 72)), int(pick(4, 9, 16, 24, 40, 64))), mlp))
        else:
            layers.append(("latent_attention", LA(int(rng.randint(1, 10)), int(pick(4, 8, 12, 16, 32, 56)), int(pick(4, 8, 20, 32, 48)),
                                                  int(pick(8, 12, 24, 40, 80)), int(pick(8, 12, 16, 24, 40, 64, 72, 128, 160)),
                                                  float(pick(0.1, 0.25, 0.5)), int(pick(1, 2, 7, 16, 17, 31, 64, 100))), mlp))
    return config(width, int(pick(50, 128, 301)), int(rng.randint(1, 7)), layers, eps=float(pick(1e-6, 1e-5, 1e-4)))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("seed", range(8))
def test_configurations_drawn_at_random(tmp_path, seed, dtype):
    cfg = drawn_config(seed)
    folder = make_folder(tmp_path / "m", cfg, seed=seed, edit=sharpen)
    reqs = {"q%d" % i: H.random_tokens(n, cfg["vocab"], 200 + seed + i) for i, n in enumerate([1, 23, 70])}
    from ginfer_amd import ModelRunner
    page = [8, 16, 32][seed % 3]
    runner = ModelRunner(folder, dtype=dtype, page_size=page, num_pages=-(-256 // page), max_requests=3)
    for what, steps in (("whole", H.steps_whole(reqs)), ("decoded", H.steps_last_decoded(reqs, last=20)),
                        ("mixed", H.steps_mixed(reqs, max_live=3, seed=seed))):
        got = H.run_steps(runner, steps)
        runner.cache.check()
        compare(got, reqs, folder, TOL[dtype], "drawn configuration %d (%s) %s %s" % (seed, json.dumps(cfg), dtype, what))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding(folders, dtype):
    """A short prompt and 400 decoded tokens: many times through every window, the recurrence four hundred steps deep,
    recorded steps replayed throughout."""
    reqs = requests_for("mixed", [420], seed=70)
    runner = runner_for(folders["mixed"], "mixed", dtype)
    got = H.run_steps(runner, H.steps_last_decoded(reqs, last=400))
    compare(got, reqs, folders["mixed"], TOL[dtype], "long decoding " + dtype)
    if runner.use_graphs:
        assert runner.counts["replayed_decode"] > 300


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_recorded_steps_equal_launched_ones(folders, dtype):
    reqs = requests_for("mixed", [60, 25, 41], seed=80)
    steps = H.steps_mixed(reqs, max_live=3, seed=9)
    outs = []
    for graphs in (True, False):
        runner = runner_for(folders["mixed"], "mixed", dtype, use_graphs=graphs)
        for rounds in range(3):
            got = H.run_steps(runner, steps)
        outs.append(got)
        if graphs:
            assert runner.use_graphs and runner.counts["replayed_decode"] + runner.counts["replayed_padded"] > 0
    for key, row in outs[0].items():
        if dtype == "float32":
            assert np.array_equal(row, outs[1][key]), key
        else:
            assert H.rel_err(row, outs[1][key]) < 2e-2, key


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_replay_program(folders, tmp_path, dtype):
    reqs = requests_for("mixed", [40, 9, 77], seed=90)
    steps = H.steps_mixed(reqs, max_live=2, seed=2)
    cfg_vocab = CONFIGS["mixed"][0]["vocab"]
    import plain_model
    orig = plain_model.read_config
    plain_model.read_config = lambda folder: {"vocab_size": cfg_vocab}          # the helper only asks for the vocabulary
    try:
        got = H.run_trace(folders["mixed"], dtype, steps, tmp_path / "out", H.max_live_tokens(steps), page_size=16)
    finally:
        plain_model.read_config = orig
    compare(got, reqs, folders["mixed"], TOL[dtype], "trace replay " + dtype)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_greedy_generation_through_the_entry_point(folders, dtype):
    """Engine.generate with its scheduler: five prompts through three slots under a budget of 48 tokens a step.  Every
    token is the plain statement's greedy choice after the engine's own tokens so far (in bfloat16: or within rounding
    of it)."""
    from ginfer_amd import Engine, EngineConfig, SamplingParams
    name = "mixed"
    folder = folders[name]
    prompts = list(requests_for(name, [3, 30, 11, 64, 1], seed=100).values())
    eng = Engine(EngineConfig(model_path=folder, dtype=dtype, max_num_batched_tokens=48, max_num_seqs=3, max_seq_len=256,
                              kvcache_block_size=8, num_kvcache_blocks=96))
    outs = eng.generate(prompts, SamplingParams(max_tokens=24, ignore_eos=True))
    cfg, w = pt.read_config(folder), pt.read_weights(folder)
    for p, o in zip(prompts, outs):
        assert len(o.token_ids) == 24
        logits = pt.forward(cfg, w, (p + o.token_ids)[:-1])
        for k, tok in enumerate(o.token_ids):
            row = logits[len(p) - 1 + k]
            best = int(torch.argmax(row))
            gap = float(row[best] - row[tok]) / float(row.abs().max())
            assert tok == best or gap <= (1e-5 if dtype == "float32" else 4e-2), \
                "%s: token %d after a prompt of %d: engine %d, plain %d (gap %.3g)" % (dtype, k, len(p), tok, best, gap)
    eng.runner.cache.check()


def test_command_line_generates(folders):
    import subprocess
    import sys
    folder = folders["taps"]
    cmd = [sys.executable, os.path.join(H.ROOT, "bin", "ginfer"), "generate", "--model-path", folder, "--dtype", "float32",
           "--prompt-ids", "1,2,3,4,5", "--max-tokens", "6", "--ignore-eos", "--max-num-seqs", "2", "--max-seq-len", "64",
           "--num-kvcache-blocks", "16"]
    out = subprocess.run(cmd, capture_output=True, text=True, timeout=300)
    assert out.returncode == 0, out.stderr[-2000:]
    cfg, w = pt.read_config(folder), pt.read_weights(folder)
    ids = [1, 2, 3, 4, 5]
    for _ in range(6):
        ids.append(int(torch.argmax(pt.forward(cfg, w, ids)[-1])))
    assert json.loads(out.stdout.strip().splitlines()[0])["token_ids"] == ids[5:]
