"""Vupuzen on the GPU against the plain implementation: every mechanism's kernel alone, then
whole models cut every way (whole prompts, token by token, portions down to two tokens, mixed
batches over pages and slots that are used again), long decoding, and greedy generation
through the engine."""
import math

import numpy as np
import pytest
import torch

from tests.helpers import rows_within
from tests.plain import vupuzen as plain
from tests.vupuzen_helpers import CONFIGS, make_folder, read_folder, tokens

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
F32_BOUND = 2e-4   # of a row's largest |logit|
BF16_BOUND = 1e-1


@pytest.fixture(scope="module")
def ops():
    if not torch.cuda.is_available():
        pytest.skip("needs a GPU")
    from pylon_amd.kernels import ops as module

    return module


@pytest.fixture(scope="module")
def tmp(tmp_path_factory):
    if not torch.cuda.is_available():
        pytest.skip("needs a GPU")
    return tmp_path_factory.mktemp("vupuzen")


def i32(values):
    return torch.tensor(list(values), dtype=torch.int32, device=DEV)


# ---- mechanisms alone ---------------------------------------------------------------------------
@pytest.mark.parametrize("taps, width", [(3, 40), (4, 300), (2, 7), (8, 64), (1, 16)])
def test_short_conv_in_portions_of_two_requests_over_reused_slots(ops, taps, width):
    rng = np.random.default_rng(taps * 100 + width)
    weight = rng.normal(size=(width, taps))
    seqs = {0: rng.normal(size=(150, width)), 1: rng.normal(size=(31, width))}
    want = {s: h + plain.causal_conv(h, weight) for s, h in seqs.items()}
    state = torch.full((3, max(taps - 1, 1), width), 5.0, device=DEV)  # as a slot that was used before
    state[[0, 2]] = 0.0  # what handing out a slot does
    slot = {0: 2, 1: 0}
    w = torch.tensor(weight, dtype=torch.float32, device=DEV)
    pos = {0: 0, 1: 0}
    got = {0: [], 1: []}
    plan = [{0: 1}, {0: 2, 1: 1}, {1: 2, 0: 1}, {0: 70, 1: 1}, {1: 3}, {0: 1, 1: 24}, {0: 65}, {0: 10}]
    for step in plan:
        rows = list(step)
        h = torch.tensor(np.concatenate([seqs[s][pos[s]: pos[s] + step[s]] for s in rows]), dtype=torch.float32, device=DEV)
        starts = np.concatenate([[0], np.cumsum([step[s] for s in rows])])
        out = ops.short_conv(h, w, state if taps > 1 else None, i32(starts), i32(slot[s] for s in rows), rows=len(rows),
                             max_count=max(step.values()), out_dtype=torch.float32).cpu().numpy()
        for r, s in enumerate(rows):
            got[s].append(out[starts[r]: starts[r + 1]])
            pos[s] += step[s]
    for s in seqs:
        g = np.concatenate(got[s])
        assert np.abs(g - want[s][: len(g)]).max() < 1e-5, (s, taps)
    assert float((state[1] - 5.0).abs().max()) == 0.0  # nobody's slot is left alone
    if taps > 1:
        assert np.allclose(state[2].cpu().numpy(), seqs[0][pos[0] - (taps - 1): pos[0]], atol=1e-6)


@pytest.mark.parametrize("dim, parts, post", [(64, 1, True), (200, 4, True), (2560, 2, True), (96, 1, False), (5000, 1, True)])
def test_sum_of_a_normed_sublayer_and_the_next_norm_in_one_kernel(ops, dim, parts, post):
    rng = np.random.default_rng(dim)
    resid = rng.normal(size=(5, dim)) * 3
    delta = rng.normal(size=(parts, 5, dim))
    d = delta.sum(0)
    x = resid + (plain.scalar_rms_norm(d, 0.6, 1e-3) if post else d)
    want = plain.scalar_rms_norm(x, 1.7, 1e-5)
    r = torch.tensor(resid, dtype=torch.float32, device=DEV)
    dl = torch.tensor(delta if parts > 1 else delta[0], dtype=torch.float32, device=DEV)
    gain, post_gain = torch.tensor(1.7, device=DEV), torch.tensor(0.6, device=DEV)
    out = ops.add_normed_rmsnorm(r, dl, gain, 1e-5, torch.float32, post_gain=post_gain if post else None, post_eps=1e-3)
    assert np.abs(out.cpu().numpy() - want).max() < 2e-5
    assert np.abs(r.cpu().numpy() - x).max() < 2e-5  # the stream holds the sum
    # picked rows: normed from the sum, the stream untouched; a gain per element
    r2 = torch.tensor(resid, dtype=torch.float32, device=DEV)
    vector = torch.tensor(rng.normal(size=dim), dtype=torch.float32, device=DEV)
    out = ops.add_normed_rmsnorm(r2, dl, vector, 1e-5, torch.float32, post_gain=post_gain if post else None,
                                 post_eps=1e-3, row_idx=i32([3, 0]))
    assert np.abs(out.cpu().numpy() - (want[[3, 0]] / 1.7 * vector.cpu().numpy())).max() < 3e-5
    assert np.array_equal(r2.cpu().numpy(), resid.astype(np.float32))


def test_capped_gated_activation(ops):
    rng = np.random.default_rng(1)
    gu = rng.normal(size=(9, 2 * 37)) * 3
    g, u = np.minimum(gu[:, :37], 1.5), np.clip(gu[:, 37:], -1.5, 1.5)
    want = g / (1 + np.exp(-1.702 * g)) * (u + 1.0)
    got = ops.gated_act(torch.tensor(gu, dtype=torch.float32, device=DEV), alpha=1.702, offset=1.0, limit=1.5)
    assert np.abs(got.cpu().numpy() - want).max() < 1e-6
    plain_silu = ops.gated_act(torch.tensor(gu, dtype=torch.float32, device=DEV), alpha=1.0, offset=0.0, limit=0.0)
    assert np.abs(plain_silu.cpu().numpy() - plain.silu(gu[:, :37]) * gu[:, 37:]).max() < 1e-5


@pytest.mark.parametrize("heads, dim, vdim, rot", [(2, 16, 8, 8), (3, 24, 48, 24), (1, 64, 64, 0), (2, 128, 128, 64),
                                                     (1, 8, 200, 2)])
def test_retention_in_portions_carries_its_state(ops, heads, dim, vdim, rot):
    rng = np.random.default_rng(heads * 1000 + dim)
    total = 90
    decay = tuple(rng.uniform(0.8, 1.0, size=heads))
    proj = rng.normal(size=(total, 2 * heads * dim + 2 * heads * vdim))
    qk, vg = heads * dim, heads * vdim
    split = lambda a, n: a.reshape(total, heads, n).transpose(1, 0, 2)
    q, k = split(proj[:, :qk], dim), split(proj[:, qk: 2 * qk], dim)
    v, g = split(proj[:, 2 * qk: 2 * qk + vg], vdim), proj[:, 2 * qk + vg:]
    first = 1000  # the request's tokens before these were run elsewhere: positions go on from here
    positions = np.arange(first, first + total)
    if rot:
        q, k = plain.rotate_half_layout(q, positions, rot, 500.0), plain.rotate_half_layout(k, positions, rot, 500.0)
    start = rng.normal(size=(heads, dim, vdim))
    o, end = plain.retention(q, k * dim ** -0.5, v, decay, 1e-4, state=start)
    want = o.transpose(1, 0, 2).reshape(total, vg) * plain.silu(g)
    state = torch.zeros((4, heads, dim, vdim), device=DEV)
    state[3] = torch.tensor(start, dtype=torch.float32)
    state[1] = 9.0
    inv_freq = None
    if rot:
        inv_freq = (1.0 / (torch.tensor(500.0) ** (torch.arange(0, rot, 2, dtype=torch.float32) / rot))).to(DEV)
    x = torch.tensor(proj, dtype=torch.float32, device=DEV)
    got, at = [], 0
    for count in (1, 2, 40, 1, 3, 43):
        out = ops.retention_recurrent(
            x[at: at + count], state, torch.tensor(decay, dtype=torch.float32, device=DEV), inv_freq,
            i32(positions[at: at + count]), i32([0, count]), i32([3]), rows=1, heads=heads, dim=dim, vdim=vdim,
            rot_dims=rot, eps=1e-4, k_scale=dim ** -0.5)
        got.append(out.cpu().numpy())
        at += count
    got = np.concatenate(got)
    assert np.abs(got - want).max() < 2e-4 * np.abs(want).max()
    assert np.abs(state[3].cpu().numpy() - end).max() < 2e-4 * np.abs(end).max()
    assert float((state[1] - 9.0).abs().max()) == 0.0


@pytest.mark.parametrize("parallel", [False, True])
@pytest.mark.parametrize("heads, dim, vdim, rot", [(2, 32, 32, 32), (3, 64, 48, 16), (1, 128, 128, 128), (2, 96, 8, 0),
                                                     (1, 256, 200, 64)])
def test_retention_in_chunks_on_the_matrix_cores(ops, heads, dim, vdim, rot, parallel):
    """bfloat16 portions of two requests side by side, of sizes that fill chunks, leave ragged
    ones and mix with single tokens, from a state that is not zero, against the plain rule."""
    rng = np.random.default_rng(heads * 31 + dim)
    rnd = lambda a: torch.tensor(a).to(torch.bfloat16).to(torch.float64).numpy()
    total = 150
    decay = tuple(rng.uniform(0.9, 1.0, size=heads))
    qk, vg = heads * dim, heads * vdim
    first = {0: 700, 1: 0}
    want, proj, start = {}, {}, {}
    for r in (0, 1):
        proj[r] = rnd(rng.normal(size=(total, 2 * qk + 2 * vg)))
        split = lambda a, n: a.reshape(total, heads, n).transpose(1, 0, 2)
        q, k = split(proj[r][:, :qk], dim), split(proj[r][:, qk: 2 * qk], dim)
        v, g = split(proj[r][:, 2 * qk: 2 * qk + vg], vdim), proj[r][:, 2 * qk + vg:]
        positions = np.arange(first[r], first[r] + total)
        if rot:
            q, k = plain.rotate_half_layout(q, positions, rot, 500.0), plain.rotate_half_layout(k, positions, rot, 500.0)
        start[r] = rng.normal(size=(heads, dim, vdim)) * (1.0 if r == 0 else 0.0)
        o, _end = plain.retention(q, k * dim ** -0.5, v, decay, 1e-4, state=start[r])
        want[r] = o.transpose(1, 0, 2).reshape(total, vg) * plain.silu(g)
    state = torch.zeros((3, heads, dim, vdim), device=DEV)
    state[2] = torch.tensor(start[0], dtype=torch.float32)
    inv_freq = None
    if rot:
        inv_freq = (1.0 / (torch.tensor(500.0) ** (torch.arange(0, rot, 2, dtype=torch.float32) / rot))).to(DEV)
    slot, at, got = {0: 2, 1: 0}, {0: 0, 1: 0}, {0: [], 1: []}
    dec = torch.tensor(decay, dtype=torch.float32, device=DEV)
    assert ops.retention_chunk_parallel(1, 10, 128, 128, 2048, units=256) and not ops.retention_chunk_parallel(
        1, 10, 128, 128, 64, units=256) and not ops.retention_chunk_parallel(16, 10, 128, 128, 2048, units=256)
    plan = ({0: 64, 1: 5}, {0: 1, 1: 33}, {1: 32}, {0: 40, 1: 1}, {0: 45, 1: 79})
    if parallel:  # rows of four chunks and more, beside a short one
        plan = ({0: 130, 1: 5}, {0: 20, 1: 145})
    for step in plan:
        rows = list(step)
        x = torch.tensor(np.concatenate([proj[r][at[r]: at[r] + step[r]] for r in rows]), dtype=torch.bfloat16, device=DEV)
        pos = np.concatenate([np.arange(first[r] + at[r], first[r] + at[r] + step[r]) for r in rows])
        starts = np.concatenate([[0], np.cumsum([step[r] for r in rows])])
        out = ops.retention_recurrent(x, state, dec, inv_freq, i32(pos), i32(starts), i32(slot[r] for r in rows),
                                      rows=len(rows), heads=heads, dim=dim, vdim=vdim, rot_dims=rot, eps=1e-4,
                                      k_scale=dim ** -0.5, chunked=True,
                                      max_count=max(step.values()) if parallel else None).float().cpu().numpy()
        for i, r in enumerate(rows):
            got[r].append(out[starts[i]: starts[i + 1]])
            at[r] += step[r]
    for r in (0, 1):
        g = np.concatenate(got[r])
        assert len(g) == total
        assert np.abs(g - want[r]).max() < 1.5e-2 * np.abs(want[r]).max(), r  # the output's own bfloat16 rounding


def paged(x, page, order, pages):
    """[T, G, d] -> cache [pages, page, G, d] with the sequence's blocks on the pages ``order``."""
    total, groups, d = x.shape
    cache = np.full((pages, page, groups, d), np.nan)
    for b, p in enumerate(order):
        part = x[b * page: (b + 1) * page]
        cache[p, : len(part)] = part
    return cache


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("dim, vdim, heads, groups, rows, far", [(16, 24, 4, 2, 12, 20), (20, 7, 3, 3, 6, 9.5),
                                                                   (64, 64, 4, 1, 16, 300), (96, 48, 2, 2, 32, 130)])
def test_sink_attention_kernel_sees_far_keys_bucket_edges_and_the_sink(ops, dtype, dim, vdim, heads, groups, rows, far):
    from pylon_amd.parts.attention import distance_buckets

    rng = np.random.default_rng(dim + vdim)
    total, page = 333, 16
    bf = dtype == torch.bfloat16
    rnd = (lambda a: torch.tensor(a).to(torch.bfloat16).to(torch.float64).numpy()) if bf else (lambda a: a)
    q, k, v = rnd(rng.normal(size=(total, heads, dim))), rnd(rng.normal(size=(total, groups, dim))), rnd(rng.normal(size=(total, groups, vdim)))
    # one key far back stands out for the last queries of head 0; another sits on a page's first slot
    k[3] *= 6.0
    q[-5:, 0] = rnd(k[3, 0] * 0.9)
    k[page * 4] *= 4.0
    q[200:210, heads - 1] = rnd(k[page * 4, groups - 1] * 1.3)
    q[100:120] *= 0.0  # scores are the biases alone there: every bucket edge decides
    rel = rnd(rng.normal(size=(rows, heads)) * 3.0 - 5.0)  # low enough that the sink's one counts
    rel[-1] -= 4.0  # beyond the last edge
    q[150:160] *= 0.01
    rel_low = rel.copy()
    scale = 0.17
    want = plain.sink_softmax_attention(q.transpose(1, 0, 2), k.transpose(1, 0, 2), v.transpose(1, 0, 2), rel, scale, far)
    want = want.transpose(1, 0, 2)
    n_pages = 40
    order = rng.permutation(n_pages)[: math.ceil(total / page)]
    kc = torch.tensor(np.nan_to_num(paged(k, page, order, n_pages), nan=1e4), dtype=dtype, device=DEV)
    vc = torch.tensor(np.nan_to_num(paged(v, page, order, n_pages), nan=1e4), dtype=dtype, device=DEV)
    table = i32(order).view(1, -1)
    bucket = i32(distance_buckets(rows, far))
    rel_t = torch.tensor(rel_low, dtype=torch.float32, device=DEV)
    # the queries arrive as a slice of wider rows, and only the last 150 of them in this step
    wide = torch.zeros((150, heads * dim + 11 * 8), dtype=dtype, device=DEV)
    wide[:, : heads * dim] = torch.tensor(q[-150:].reshape(150, -1), dtype=dtype)
    qv = wide[:, : heads * dim].view(150, heads, dim)
    got = ops.paged_attention(qv, kc, vc, table, i32([0] * 150), i32(range(total - 150, total)), page_size=page,
                              window=None, scale=scale, rel=rel_t, bucket=bucket, sink=True).float().cpu().numpy()
    bound = 3e-2 if bf else 2e-5
    assert np.abs(got - want[-150:]).max() < bound * max(1.0, np.abs(want).max())
    assert np.abs(want[-1, 0] - v[3, 0]).max() < 0.2  # the far key does carry the output there
    # without its sink the same scores give another result where no key stands out
    no_sink = ops.paged_attention(qv, kc, vc, table, i32([0] * 150), i32(range(total - 150, total)), page_size=page,
                                  window=None, scale=scale, rel=rel_t, bucket=bucket, sink=False).float().cpu().numpy()
    assert np.abs(no_sink - got).max() > 0.01


@pytest.mark.parametrize("dim, vdim, heads, groups, rows, far, page", [
    (64, 64, 4, 1, 16, 300, 32), (96, 48, 6, 3, 32, 130, 64), (16, 24, 4, 2, 12, 20, 32), (40, 12, 3, 3, 6, 9.5, 96),
    (128, 128, 8, 1, 32, 70, 64), (8, 4, 2, 1, 4, 3, 32)])
def test_sink_attention_on_the_matrix_cores(ops, dim, vdim, heads, groups, rows, far, page):
    """The bfloat16 kernel against the plain rule: a prompt portion behind cached tokens, cut into
    tiles in the order the step function gives them, and single tokens of requests of unequal
    lengths.  Free slots of the last page hold NaN."""
    from pylon_amd.parts.attention import distance_buckets

    rng = np.random.default_rng(dim * 7 + vdim)
    rnd = lambda a: torch.tensor(a).to(torch.bfloat16).to(torch.float64).numpy()
    total = 333
    q, k, v = rnd(rng.normal(size=(total, heads, dim))), rnd(rng.normal(size=(total, groups, dim))), rnd(rng.normal(size=(total, groups, vdim)))
    k[3] *= 5.0
    q[-5:, 0] = rnd(k[3, 0] * 0.9)  # a far key carries the last queries of head 0
    k[page] *= 4.0
    q[200:210, heads - 1] = rnd(k[page, groups - 1] * 1.3)  # a key on a page's first slot
    q[250:270] *= 0.0  # the biases alone decide there
    rel = rnd(rng.normal(size=(rows, heads)) * 3.0 - 4.0)
    scale = 0.17
    want = plain.sink_softmax_attention(q.transpose(1, 0, 2), k.transpose(1, 0, 2), v.transpose(1, 0, 2), rel, scale, far)
    want = want.transpose(1, 0, 2)
    n_pages = 30
    order = rng.permutation(n_pages)[: math.ceil(total / page)]
    kc = torch.tensor(paged(k, page, order, n_pages), dtype=torch.bfloat16, device=DEV)  # NaN where no token lies
    vc = torch.tensor(paged(v, page, order, n_pages), dtype=torch.bfloat16, device=DEV)
    vt = vc.permute(0, 2, 3, 1).contiguous()  # [pages, kv heads, vdim, slot in page]
    table = torch.zeros((3, 16), dtype=torch.int32, device=DEV)
    table[1, : len(order)] = i32(order)
    bucket, rel_t = i32(distance_buckets(rows, far)), torch.tensor(rel, dtype=torch.float32, device=DEV)
    first = 140
    count = total - first
    wide = torch.zeros((count, heads * dim + 24), dtype=torch.bfloat16, device=DEV)
    wide[:, : heads * dim] = torch.tensor(q[first:].reshape(count, -1), dtype=torch.bfloat16)
    qv = wide.as_strided((count, heads, dim), (wide.stride(0), dim, 1))
    tiles = [(a, min(32, count - a), 1, first + a) for a in range(0, count, 32)]
    tiles = i32(np.array(tiles[::-1]).reshape(-1)).view(-1, 4)  # heaviest first, as the step function orders them
    common = dict(page_size=page, scale=scale, rel=rel_t, bucket=bucket, sink=True)
    fast = dict(page_size=page, scale=scale, bias=ops.bias_by_distance(rel_t, bucket), sink=True)
    got = ops.attention_sink(qv, kc, vt, table, tiles, None, **fast).float().cpu().numpy()
    assert not np.isnan(got).any()
    assert np.abs(got - want[first:]).max() < 2e-2 * max(1.0, np.abs(want).max())
    assert np.abs(got[-1, 0] - v[3, 0]).max() < 0.2
    general = ops.paged_attention(qv, kc.nan_to_num(0.0), vt.nan_to_num(0.0), table, i32([1] * count), i32(range(first, total)),
                                  window=None, v_transposed=True, **common).float().cpu().numpy()
    assert np.abs(got - general).max() < 2e-2 * max(1.0, np.abs(want).max())
    # single tokens: three "requests" that are this sequence at three lengths, one row of the table each
    lengths = [total, 33, 1]
    table[0], table[2] = table[1], table[1]
    singles = torch.tensor(np.stack([q[n - 1] for n in lengths]), dtype=torch.bfloat16, device=DEV)
    for cuts in (1, 2, 8):  # the keys of a request shared between workgroups, merged by a second kernel
        got = ops.attention_sink(singles, kc, vt, table, None, i32([n - 1 for n in lengths]), cuts=cuts,
                                 **fast).float().cpu().numpy()
        for r, n in enumerate(lengths):
            assert np.abs(got[r] - want[n - 1]).max() < 2e-2 * max(1.0, np.abs(want).max()), (n, cuts)
    assert ops.sink_cuts(8, 32, 8, 128, units=256) == 1 and ops.sink_cuts(8, 32, 8, 2048, units=256) == 8
    assert ops.sink_cuts(1, 32, 8, 100000, units=256) == 64 and ops.sink_cuts(64, 32, 8, 100000, units=256) == 1


def test_a_sink_takes_all_the_weight_when_every_score_is_far_below_zero(ops):
    rel = torch.full((4, 1), -30.0, device=DEV)
    kc = torch.zeros((1, 16, 1, 8), device=DEV)
    vc = torch.ones((1, 16, 1, 5), device=DEV)
    out = ops.paged_attention(torch.zeros((3, 1, 8), device=DEV), kc, vc, i32([0]).view(1, 1), i32([0, 0, 0]),
                              i32([0, 7, 15]), page_size=16, window=None, scale=1.0, rel=rel, bucket=i32([0, 1, 2, 3]),
                              sink=True)
    assert float(out.abs().max()) < 1e-10 and float(out.abs().min()) > 0.0


# ---- whole models ---------------------------------------------------------------------------------
class Case:
    def __init__(self, tmp, name, dtype, lengths, store=None, seed=3):
        from pylon_amd.engine import Runner

        self.folder = make_folder(tmp, name, dtype=store or dtype, seed=seed)
        self.cfg, self.weights = read_folder(self.folder)
        self.requests = {f"r{i}": tokens(self.cfg["vocab"], n, 50 + i) for i, n in enumerate(lengths)}
        self.want = {rid: plain.forward(self.weights, self.cfg, toks) for rid, toks in self.requests.items()}
        self.dtype = dtype
        self.bound = F32_BOUND if dtype == "float32" else BF16_BOUND

    def runner(self, page_size=16, num_pages=40, max_requests=3):
        from pylon_amd.engine import Runner

        return Runner.from_folder(self.folder, dtype=self.dtype, page_size=page_size, num_pages=num_pages,
                                  max_requests=max_requests)

    def check(self, rid, got, label):
        ok, worst, frac = rows_within(got, self.want[rid][: len(got)], self.bound)
        assert ok, f"{label}: request {rid}, position {worst} is off by {frac:.2e} of its largest logit"


def run_plan(runner, case, plan):
    """``plan``: steps ``{request: tokens to feed}``; 0 closes a request.  Returns logits per request."""
    from pylon_amd.engine import StepEntry

    live, pos = {}, {rid: 0 for rid in case.requests}
    got = {rid: [] for rid in case.requests}
    for step in plan:
        entries = []
        for rid, size in step.items():
            if size == 0:
                runner.close(live.pop(rid))
                continue
            if rid not in live:
                live[rid] = runner.open(rid)
            chunk = case.requests[rid][pos[rid]: pos[rid] + size]
            entries.append((rid, StepEntry(live[rid], chunk, list(range(len(chunk))))))
            pos[rid] += len(chunk)
        if entries:
            logits = runner.step([e for _, e in entries]).cpu().numpy()
            cursor = 0
            for rid, e in entries:
                got[rid].append(logits[cursor: cursor + len(e.tokens)])
                cursor += len(e.tokens)
        runner.manager.check()
    for seq in live.values():
        runner.close(seq)
    return {rid: np.concatenate(parts) for rid, parts in got.items() if parts}, pos


@pytest.mark.parametrize("name, dtype, page", [("P", "float32", 16), ("Q", "float32", 16), ("R", "float32", 16),
                                                ("R", "bfloat16", 16), ("P", "bfloat16", 16), ("R", "bfloat16", 32),
                                                ("P", "bfloat16", 64), ("Q", "bfloat16", 32)])
def test_whole_token_by_token_and_in_portions(tmp, name, dtype, page):
    """Pages of 16 tokens run the general attention kernel, pages of 32 and 64 the matrix-core one."""
    case = Case(tmp, name, dtype, (71, 38))
    runner = case.runner(page_size=page, num_pages=640 // page)
    whole, _ = run_plan(runner, case, [{"r0": 71}, {"r0": 0, "r1": 38}])
    for rid, got in whole.items():
        case.check(rid, got, "whole")
    single, _ = run_plan(runner, case, [{"r1": 1} for _ in range(38)])
    case.check("r1", single["r1"], "token by token")
    cut, _ = run_plan(runner, case, [{"r0": n} for n in (2, 3, 2, 17, 1, 1, 30, 2, 13)])
    case.check("r0", cut["r0"], "portions")
    if dtype == "float32":  # how a request is cut moves nothing but the order of a product's sums
        assert np.abs(cut["r0"] - whole["r0"]).max() <= 2e-5 * np.abs(whole["r0"]).max()
        assert np.abs(single["r1"] - whole["r1"]).max() <= 2e-5 * np.abs(whole["r1"]).max()


@pytest.mark.parametrize("name, dtype, page", [("P", "float32", 16), ("Q", "float32", 16), ("R", "bfloat16", 16),
                                                ("R", "bfloat16", 32), ("P", "bfloat16", 32)])
def test_mixed_batches_over_pages_and_slots_that_are_used_again(tmp, name, dtype, page):
    case = Case(tmp, name, dtype, (60, 45, 33, 20))
    pages = 9 if page == 16 else 6  # room for 144 (or 192) tokens: never all four requests at once
    runner = case.runner(page_size=page, num_pages=pages, max_requests=3)
    plan = [{"r0": 20}, {"r0": 1, "r1": 30}, {"r0": 2, "r1": 1, "r2": 5}, {"r0": 1, "r1": 1, "r2": 1},
            {"r0": 20, "r1": 13, "r2": 2}, {"r1": 0, "r0": 1, "r2": 1}, {"r3": 17, "r0": 15, "r2": 24},
            {"r2": 0, "r0": 0, "r3": 1}, {"r3": 2}]
    got, pos = run_plan(runner, case, plan)
    assert pos == {"r0": 60, "r1": 45, "r2": 33, "r3": 20}
    for rid, logits in got.items():
        case.check(rid, logits, "mixed")
    alone, _ = run_plan(runner, case, [{"r3": 20}])
    limit = 2e-5 if dtype == "float32" else 3e-2
    assert np.abs(alone["r3"] - got["r3"]).max() <= limit * np.abs(alone["r3"]).max()
    assert runner.manager.free_pages == pages and runner.manager.slots.free_slots == 3


def test_long_decoding_after_a_prompt(tmp):
    case = Case(tmp, "R", "float32", (420,))
    runner = case.runner(page_size=64, num_pages=8, max_requests=2)
    got, _ = run_plan(runner, case, [{"r0": 100}] + [{"r0": 1}] * 320)
    case.check("r0", got["r0"], "long decoding")


def test_requests_do_not_see_what_a_freed_slot_or_page_held(tmp):
    """The same request, alone in a fresh runner and after others have used every page and slot."""
    case = Case(tmp, "P", "float32", (50, 64, 64))
    fresh, _ = run_plan(case.runner(num_pages=8, max_requests=2), case, [{"r0": 50}])
    runner = case.runner(num_pages=8, max_requests=2)
    for tensor in runner.manager.slots.tensors.values():
        tensor.fill_(float("nan"))
    for group in runner.manager.groups:
        for cache in list(group.k.values()) + list(group.v.values()):
            cache.fill_(float("nan"))
    used, _ = run_plan(runner, case, [{"r1": 64, "r2": 64}, {"r1": 0, "r2": 0}, {"r0": 25}, {"r0": 25}])
    assert np.abs(used["r0"] - fresh["r0"]).max() <= 2e-5 * np.abs(fresh["r0"]).max()


@pytest.mark.parametrize("name, dtype, graphs, page", [("P", "float32", False, 16), ("Q", "float32", True, 16),
                                                         ("R", "bfloat16", True, 16), ("R", "bfloat16", True, 32)])
def test_greedy_generation_through_the_engine(tmp, name, dtype, graphs, page):
    from pylon_amd.engine.engine import Engine
    from pylon_amd.sampling import Sampling

    folder = make_folder(tmp, name, dtype=dtype, seed=8)
    cfg, weights = read_folder(folder)
    prompts = [tokens(cfg["vocab"], n, 70 + n) for n in (3, 19, 41)]
    engine = Engine.from_folder(folder, dtype=dtype, page_size=page, num_pages=384 // page, max_batch_size=3,
                                prefill_chunk_size=16, cuda_graphs=graphs)
    try:
        results = engine.generate(prompts, Sampling(max_new_tokens=12, temperature=0.0))
    finally:
        engine.close()
    slack = 1e-4 if dtype == "float32" else 5e-2
    for prompt, result in zip(prompts, results):
        assert len(result.output_ids) == 12
        sequence = list(prompt)
        for produced in result.output_ids:
            row = plain.forward(weights, cfg, sequence)[-1]
            assert produced == int(row.argmax()) or row.max() - row[produced] <= slack * np.abs(row).max(), \
                (prompt[:3], result.output_ids)
            sequence.append(produced)
