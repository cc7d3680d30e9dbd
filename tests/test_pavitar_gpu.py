"""Pavitar on the GPU against the plain implementation: every mechanism's kernel alone (masks at
their edges with a key planted so that it decides, far keys, page borders), then whole models cut
every way (whole prompts, token by token, portions down to two tokens, mixed batches over pages
and slots that are used again), long decoding over pages that windows and chunks give back, and
greedy generation through the engine."""
import numpy as np
import pytest
import torch

from tests.helpers import rows_within
from tests.pavitar_helpers import CONFIGS, make_folder, read_folder, tokens
from tests.plain import pavitar as plain

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
F32_BOUND = 2e-4   # of a row's largest |logit|
BF16_BOUND = 1e-1
ROUTER_MARGIN = 0.8  # of a router logit (the test folders' routers are scaled up: logits of several units)


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
    return tmp_path_factory.mktemp("pavitar")


def i32(values):
    return torch.tensor(list(values), dtype=torch.int32, device=DEV)


def dev(array, dtype=torch.float32):
    return torch.tensor(np.asarray(array), dtype=dtype, device=DEV)


def close(got, want, bound, what=""):
    got, want = np.asarray(got, dtype=np.float64), np.asarray(want)
    err = np.abs(got - want).max() / max(np.abs(want).max(), 1e-30)
    assert err <= bound, f"{what}: off by {err:.2e} of the largest value"


# ---- mechanisms alone ---------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads, groups, dim, vdim, rot, pairs", [
    (4, 2, 16, 24, 8, True), (3, 3, 12, 12, 12, True), (2, 1, 10, 6, 0, True), (6, 2, 64, 64, 32, True),
    (5, 1, 7, 3, 6, True), (2, 2, 32, 16, 16, False)])
def test_wide_preparation_norms_whole_projections_and_turns_pairs(ops, dtype, heads, groups, dim, vdim, rot, pairs):
    rng = np.random.default_rng(heads * 100 + dim)
    n, eps, base = 9, 1e-5, 777.0
    q_size, k_size, v_size = heads * dim, groups * dim, groups * vdim
    proj = torch.tensor(rng.normal(size=(n, q_size + k_size + v_size)), dtype=dtype)
    qw, kw = rng.normal(size=q_size) + 1, rng.normal(size=k_size) + 1
    positions = [0, 1, 2, 3, 50, 51, 1000, 4097, 7]
    slots = [5, 0, 17, 3, 9, 30, 2, 8, 1]
    x = proj.double().numpy()
    q = plain.norm_plain(x[:, :q_size], qw, eps).reshape(n, heads, dim)
    k = plain.norm_plain(x[:, q_size: q_size + k_size], kw, eps).reshape(n, groups, dim)

    def turn(t):  # rotate_pairs counts positions from 0: one call per token, at its own position
        out = np.empty_like(t)
        for row, p in enumerate(positions):
            padded = np.zeros((p + 1,) + t.shape[1:])
            padded[p] = t[row]
            if pairs:
                out[row] = plain.rotate_pairs(padded, rot, base)[p]
            else:  # halves together: the same turn on the elements put side by side
                order = [j for i in range(rot // 2) for j in (i, i + rot // 2)] + list(range(rot, t.shape[-1]))
                back = np.argsort(order)
                out[row] = plain.rotate_pairs(padded[..., order], rot, base)[p][..., back]
        return out

    q, k = turn(q), turn(k)
    inv_freq = dev(base ** (-np.arange(0, rot, 2) / rot)) if rot else None
    q_out = torch.empty((n, heads, dim), dtype=dtype, device=DEV)
    k_cache = torch.zeros((4, 8, groups, dim), dtype=dtype, device=DEV)
    v_cache = torch.zeros((4, 8, groups, vdim), dtype=dtype, device=DEV)
    ops.qkv_prepare_wide(proj.to(DEV), q_out, k_cache, v_cache, n_heads=heads, n_kv_heads=groups, head_dim=dim, v_dim=vdim,
                         q_weight=dev(qw), k_weight=dev(kw), eps=eps, inv_freq=inv_freq, rot_dim=rot, interleaved=pairs,
                         positions=i32(positions), slot_map=i32(slots), store_kv=True)
    bound = 2e-4 if dtype == torch.float32 else 1e-2  # an angle of 4,097 radians in float32 is 2e-4 off
    close(q_out.float().cpu().numpy(), q, bound, "q")
    close(k_cache.view(32, groups, dim)[slots].float().cpu().numpy(), k, bound, "k")
    assert torch.equal(v_cache.view(32, groups * vdim)[slots].cpu(), proj[:, q_size + k_size:])
    untouched = sorted(set(range(32)) - set(slots))
    assert not k_cache.view(32, -1)[untouched].any() and not v_cache.view(32, -1)[untouched].any()


def planted_case(rng, n, heads, groups, dim, vdim, planted, shared_kv):
    """Queries, keys and values of one request of ``n`` tokens in which the keys ``planted`` lie
    along one direction that every query has a large share of: whoever sees one of them gives it
    nearly all of its weight, so a mask that is one key off shows in the output."""
    u = rng.normal(size=dim)
    u /= np.linalg.norm(u)
    q = 0.3 * rng.normal(size=(n, heads, dim)) + 3.0 * u
    k = 0.3 * rng.normal(size=(n, groups, dim))
    for j, strength in planted:
        k[j] += strength * u
    v = k.copy() if shared_kv else rng.normal(size=(n, groups, vdim))
    return q, k, v


def plain_attention(q, k, v, visible, scale):
    n, heads, _ = q.shape
    groups = k.shape[1]
    out = np.zeros((n, heads, v.shape[2]))
    for h in range(heads):
        g = h // (heads // groups)
        out[:, h] = plain.softmax_masked(q[:, h] @ k[:, g].T * scale, visible) @ v[:, g]
    return out


MASKS = [("window", 37), ("chunk", 37), ("window", 1), ("chunk", 64), ("window", 200), ("chunk", 129)]


@pytest.mark.parametrize("kind, size", MASKS)
@pytest.mark.parametrize("dtype, heads, groups, dim, vdim, page, shared_kv", [
    (torch.float32, 4, 2, 16, 24, 16, False), (torch.float32, 3, 1, 40, 40, 8, True),
    (torch.bfloat16, 6, 3, 20, 8, 16, False), (torch.bfloat16, 4, 2, 64, 64, 16, False),
    (torch.bfloat16, 4, 2, 64, 64, 64, False), (torch.bfloat16, 3, 1, 128, 128, 64, False),
    (torch.bfloat16, 20, 1, 64, 64, 32, True), (torch.bfloat16, 5, 1, 128, 128, 64, True),
    (torch.bfloat16, 8, 1, 256, 256, 16, True)])
def test_attention_masks_at_their_edges(ops, kind, size, dtype, heads, groups, dim, vdim, page, shared_kv):
    """Keys planted at both sides of a window's and a chunk's edge, at a page's first and last
    slot and far back; every query position of a 300-token request, as a prompt (general and
    matrix-core prefill kernels) and token by token (general and matrix-core decode kernels)."""
    rng = np.random.default_rng(size * 7 + dim + heads)
    n, scale = 300, 0.4
    planted = [(0, 5.0), (page - 1, 6.0), (page, 7.0), (size - 1, 8.0) if size < n else (3, 8.0),
               (min(size, n - 1), 9.0), (2 * size if 2 * size < n else 5, 10.0), (n - 2 - size if n - 2 - size > 0 else 7, 11.0)]
    q, k, v = planted_case(rng, n, heads, groups, dim, vdim, planted, shared_kv)
    t = lambda a: torch.tensor(a, dtype=dtype)
    q, k, v = t(q), t(k), t(v)
    visible = plain.window_mask(n, size) if kind == "window" else plain.chunk_mask(n, size)
    want = plain_attention(q.double().numpy(), k.double().numpy(), v.double().numpy(), visible, scale)
    pages = -(-n // page)
    order = rng.permutation(pages + 3)[:pages]  # the request's pages lie scattered in a larger pool
    k_cache = torch.full((pages + 3, page, groups, dim), float("nan"), dtype=dtype)
    v_cache = torch.full((pages + 3, page, groups, vdim), float("nan"), dtype=dtype)
    slots = np.array([order[p // page] * page + p % page for p in range(n)])
    k_cache.view(-1, groups, dim)[slots] = k
    v_cache.view(-1, groups, vdim)[slots] = v
    k_cache, v_cache, qd = k_cache.to(DEV), v_cache.to(DEV), q.to(DEV)
    if shared_kv:
        v_cache = k_cache
    table = i32(order).view(1, pages)
    mask = {kind: size}
    bound = 2e-5 if dtype == torch.float32 else 2e-2
    positions = i32(range(n))
    rows = torch.zeros(n, dtype=torch.int32, device=DEV)
    got = ops.paged_attention(qd, k_cache, v_cache, table, rows, positions, page_size=page, scale=scale,
                              window=mask.get("window"), chunk=mask.get("chunk"))
    close(got.float().cpu().numpy(), want, bound, "general kernel")
    if dtype != torch.bfloat16 or dim not in ops.DECODE_HEAD_DIMS:
        return
    # prompt portions on the matrix cores: the whole request, and its second half over the cached first
    group = heads // groups
    for first in (0, 143):
        tile = ops.prefill_rows(n - first, heads, group) // group
        tiles = [(s, min(tile, n - s), 0, s) for s in range(first, n, tile)]
        out = torch.zeros_like(qd)
        ops.attention_prefill(qd, k_cache, v_cache, table, i32(np.array(tiles).reshape(-1)).view(-1, 4), page_size=page,
                              scale=scale, rows=ops.prefill_rows(n - first, heads, group), out=out,
                              window=mask.get("window"), chunk=mask.get("chunk"))
        close(out[first:].float().cpu().numpy(), want[first:], bound, f"prefill kernel from {first}")
    # single tokens on the matrix cores, every position a "request" of its own on the same pages
    if group > 16:
        per = max(g for g in range(1, 17) if heads % g == 0)
        qd = qd.view(n * (heads // per), per, dim)
        positions = positions.repeat_interleave(heads // per)
    rows = torch.zeros(positions.numel(), dtype=torch.int32, device=DEV)
    for cuts, splits in ((1, 1), (1, 4), (2, 2)):
        got = ops.attention_decode(qd, k_cache, v_cache, table, rows, positions, page_size=page, scale=scale,
                                   n_splits=splits, n_cuts=cuts, window=mask.get("window"), chunk=mask.get("chunk"))
        close(got.view(n, heads, dim).float().cpu().numpy(), want, bound, f"decode kernel, {cuts} cuts, {splits} waves")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("q_rank, kv_rank, gates", [(24, 40, 3), (8, 16, 1), (300, 513, 20), (64, 64, 0)])
def test_latent_preparation(ops, dtype, q_rank, kv_rank, gates):
    rng = np.random.default_rng(q_rank)
    n, eps = 7, 3e-6
    down = rng.normal(size=(n, q_rank + kv_rank + gates)) * 3
    qw, cw = rng.normal(size=q_rank), rng.normal(size=kv_rank)
    slots = [3, 11, 0, 6, 7, 19, 2]
    cache = torch.zeros((5, 4, 1, kv_rank), dtype=dtype, device=DEV)
    x = dev(down)
    q_latent, gate = ops.latent_prepare(x, cache, i32(slots), q_rank=q_rank, kv_rank=kv_rank, n_gate=gates,
                                        q_weight=dev(qw), c_weight=dev(cw), eps=eps, out_dtype=dtype)
    d = x.double().cpu().numpy()
    bound = 2e-5 if dtype == torch.float32 else 1e-2
    close(q_latent.float().cpu().numpy(), plain.norm_plain(d[:, :q_rank], qw, eps), bound, "query latent")
    close(cache.view(20, kv_rank)[slots].float().cpu().numpy(),
          plain.norm_plain(d[:, q_rank: q_rank + kv_rank], cw, eps), bound, "cached latent")
    if gates:
        close(gate.cpu().numpy(), plain.sigmoid(d[:, q_rank + kv_rank:]), 1e-5, "gates")
    else:
        assert gate is None
    # a run that reads another's cache stores nothing
    before = cache.clone()
    ops.latent_prepare(x, None, None, q_rank=q_rank, kv_rank=kv_rank, n_gate=gates, q_weight=dev(qw), c_weight=dev(cw),
                       eps=eps, out_dtype=dtype)
    assert torch.equal(before, cache)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("n, heads, n_in, n_out, gated", [(1, 3, 12, 40, False), (9, 2, 40, 20, True), (64, 5, 32, 64, True),
                                                          (65, 5, 32, 64, True), (200, 20, 64, 32, False), (3, 1, 300, 513, True)])
def test_products_head_by_head(ops, dtype, n, heads, n_in, n_out, gated):
    rng = np.random.default_rng(n + heads)
    x = torch.tensor(rng.normal(size=(n, heads, n_in)), dtype=dtype)
    m = torch.tensor(rng.normal(size=(heads, n_in, n_out)), dtype=dtype)
    gate = rng.uniform(size=(n, heads)) if gated else None
    want = np.einsum("thi,hio->tho", x.double().numpy(), m.double().numpy())
    if gated:
        want *= gate[:, :, None]
    got = ops.head_project(x.to(DEV), m.to(DEV), gate=dev(gate) if gated else None)
    close(got.float().cpu().numpy(), want, 1e-5 if dtype == torch.float32 else 1e-2, "per-head product")


@pytest.mark.parametrize("experts, top, shared", [(5, 2, True), (3, 1, False), (70, 7, True), (300, 32, False), (4, 4, True)])
def test_routing_takes_the_largest_logits_and_the_lower_index_among_equals(ops, experts, top, shared):
    rng = np.random.default_rng(experts)
    n = 37
    logits = rng.normal(size=(n, experts + (1 if shared else 0))).astype(np.float32)
    bias = (np.round(rng.normal(size=experts) * 8) / 8).astype(np.float32)  # eighths: sums with them are exact
    logits[1, : experts] = 0.25 - bias  # every sum the same number: the lowest indices win
    if experts > 3:
        logits[2, 1] = 1.5
        logits[2, 3] = logits[2, 1] + bias[1] - bias[3]  # one tie somewhere in the row
    z = (torch.tensor(logits[:, :experts]) + torch.tensor(bias)).double().numpy()  # the float32 sums the kernel forms
    order = np.argsort(-z, axis=-1, kind="stable")[:, :top]
    chosen = np.take_along_axis(z, order, axis=-1)
    e = np.exp(chosen - chosen.max(axis=-1, keepdims=True))
    got_experts, got_weights, gate = ops.route_top(dev(logits), dev(bias), n_experts=experts, top=top, shared_gate=shared)
    assert got_experts.cpu().numpy().tolist() == order.tolist()
    close(got_weights.cpu().numpy(), e / e.sum(axis=-1, keepdims=True), 1e-5, "weights")
    assert got_experts[1].tolist() == list(range(top))
    if shared:
        close(gate.cpu().numpy(), plain.sigmoid(logits[:, experts].astype(np.float64)), 1e-5, "shared gate")
    else:
        assert gate is None


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("width, experts, top, ff, shared", [(64, 5, 2, 24, 40), (48, 3, 1, 32, None), (512, 6, 4, 520, 64),
                                                             (100, 4, 4, 7, 3)])
def test_mixture_of_experts_against_the_plain_one(ops, dtype, width, experts, top, ff, shared):
    from pylon_amd.config.specs import MixtureFeedForwardSpec
    from pylon_amd.parts import build_part

    rng = np.random.default_rng(width + ff)
    spec = MixtureFeedForwardSpec(hidden_size=width, n_experts=experts, top=top, expert_size=ff, shared_size=shared,
                                  shared_gate=shared is not None, router_bias=True)
    part = build_part("feed_forward", spec, dtype=dtype, device=DEV)
    w = {"f.router": rng.normal(size=(experts, width)), "f.router.b": rng.normal(size=experts)}
    for e in range(experts):
        w[f"f.e{e}.gate"], w[f"f.e{e}.up"] = rng.normal(size=(ff, width)) * 0.2, rng.normal(size=(ff, width)) * 0.2
        w[f"f.e{e}.down"] = rng.normal(size=(width, ff)) * 0.2
    if shared is not None:
        w["f.shared.gate"], w["f.shared.up"] = rng.normal(size=(shared, width)) * 0.2, rng.normal(size=(shared, width)) * 0.2
        w["f.shared.down"], w["f.shared.sg"] = rng.normal(size=(width, shared)) * 0.2, rng.normal(size=(1, width)) * 0.3
    w = {k: torch.tensor(a).to(dtype).double().numpy() for k, a in w.items()}  # what the part will hold
    p = part.params
    p["router"][:experts] = dev(w["f.router"], dtype)
    p["router_bias"][:] = dev(w["f.router.b"])
    for e in range(experts):
        p["gate_up"][e * 2 * ff: e * 2 * ff + ff] = dev(w[f"f.e{e}.gate"], dtype)
        p["gate_up"][e * 2 * ff + ff: (e + 1) * 2 * ff] = dev(w[f"f.e{e}.up"], dtype)
        p["down"][e * width: (e + 1) * width] = dev(w[f"f.e{e}.down"], dtype)
    if shared is not None:
        p["router"][experts:] = dev(w["f.shared.sg"], dtype)
        p["shared_gate_up"][:shared] = dev(w["f.shared.gate"], dtype)
        p["shared_gate_up"][shared:] = dev(w["f.shared.up"], dtype)
        p["shared_down"][:] = dev(w["f.shared.down"], dtype)
    mlp = {"router": {"experts": experts, "top": top}, "shared": None if shared is None else {"ff": shared}}
    for n in (1, 5, 70, 150, 400):  # the products change kernels with the row count (400: the experts' tiles through LDS)
        h = torch.tensor(rng.normal(size=(n, width)), dtype=dtype)
        want = plain.mixture(h.double().numpy(), w, "f.", mlp)
        got = part.forward(h.to(DEV), None)
        assert got.dtype == torch.float32 and got.shape == (n, width)
        close(got.cpu().numpy(), want, 2e-5 if dtype == torch.float32 else 3e-2, f"{n} tokens")
        if n == 70:  # a token's result does not depend on its neighbours in the step
            alone = part.forward(h[3:4].to(DEV), None)
            if dtype == torch.float32:
                assert np.abs(alone.cpu().numpy() - got[3:4].cpu().numpy()).max() <= 2e-5 * np.abs(want).max()


@pytest.mark.parametrize("tokens", [300, 400])
def test_experts_sorted_by_expert_agree_with_token_by_token_at_tile_edges(ops, tokens):
    """The matrix-core path (pairs sorted by expert; tiles of 64 rows at 300 tokens, of 128 through LDS
    at 400) against the token-by-token kernels on routings made by hand: an expert nobody chose, experts
    with exactly one tile, one pair more, one pair, and the rest."""
    rng = np.random.default_rng(tokens)
    width, ff, experts, top = 72, 40, 5, 2
    pairs = tokens * top
    tile = 128 if pairs // experts >= 128 else 64
    counts = [0, tile, tile + 1, 1]
    counts.append(pairs - sum(counts))
    flat = np.repeat(np.arange(experts), counts)
    rng.shuffle(flat)  # (a token may meet an expert twice here, which a router never does and the kernels do not mind)
    chosen = flat.reshape(tokens, top)
    weights = rng.uniform(0.1, 1.0, size=(tokens, top)).astype(np.float32)
    x = torch.tensor(rng.normal(size=(tokens, width)), dtype=torch.bfloat16, device=DEV)
    gate_up = torch.tensor(rng.normal(size=(experts * 2 * ff, width)) * 0.2, dtype=torch.bfloat16, device=DEV)
    down = torch.tensor(rng.normal(size=(experts * width, ff)) * 0.2, dtype=torch.bfloat16, device=DEV)
    shared = torch.tensor(rng.normal(size=(tokens, width)), dtype=torch.float32, device=DEV)
    gate = torch.tensor(rng.uniform(size=tokens), dtype=torch.float32, device=DEV)
    e, w = i32(chosen.reshape(-1)).view(tokens, top), dev(weights)
    hidden = ops.expert_gate_up(x, gate_up, e, n_experts=experts, ff=ff)
    want = ops.expert_down(hidden, down, e, w, n_experts=experts, width=width, shared=shared, shared_gate=gate)
    got = ops.experts_grouped(x, gate_up, down, e, w, n_experts=experts, ff=ff, shared=shared, shared_gate=gate)
    close(got.cpu().numpy(), want.double().cpu().numpy(), 2e-2, "sorted by expert")
    # and without a shared expert
    want = ops.expert_down(hidden, down, e, w, n_experts=experts, width=width)
    got = ops.experts_grouped(x, gate_up, down, e, w, n_experts=experts, ff=ff)
    close(got.cpu().numpy(), want.double().cpu().numpy(), 2e-2, "sorted by expert, no shared expert")


def test_soft_cap(ops):
    x = torch.tensor([[-1e4, -30.0, -1.0, 0.0, 0.5, 29.0, 1e4]], device=DEV)
    want = 15.0 * np.tanh(x.double().cpu().numpy() / 15.0)
    close(ops.softcap_(x.clone(), 15.0).cpu().numpy(), want, 1e-6, "soft cap")


# ---- whole models ---------------------------------------------------------------------------------
class Case:
    def __init__(self, tmp, name, dtype, lengths, seed=3):
        self.folder = make_folder(tmp, name, dtype=dtype, seed=seed)
        self.cfg, self.weights = read_folder(self.folder)
        self.requests = {f"r{i}": tokens(self.cfg["vocab"], n, 50 + i) for i, n in enumerate(lengths)}
        self.want, self.clear = {}, {}
        for rid, toks in self.requests.items():
            margins = []
            self.want[rid] = plain.forward(self.cfg, self.weights, toks, margins=margins)
            # In bfloat16 a router's choice between two nearly equal logits is an accident of
            # rounding: positions at which some router's margin is that small are not compared.
            closest = np.min(margins, axis=0) if margins else np.full(len(toks), np.inf)
            self.clear[rid] = closest >= (0.0 if dtype == "float32" else ROUTER_MARGIN)
        self.dtype = dtype
        self.bound = F32_BOUND if dtype == "float32" else BF16_BOUND

    def runner(self, page_size=16, num_pages=40, max_requests=3):
        from pylon_amd.engine import Runner

        return Runner.from_folder(self.folder, dtype=self.dtype, page_size=page_size, num_pages=num_pages,
                                  max_requests=max_requests)

    def check(self, rid, got, label):
        clear = self.clear[rid][: len(got)]
        assert clear.mean() >= 0.3, "too few positions with clear routing to compare"
        got, want = got[clear], self.want[rid][: len(got)][clear]
        ok, worst, frac = rows_within(got, want, self.bound if self.dtype == "float32" else 3 * self.bound)
        assert ok, f"{label}: request {rid}, position {np.flatnonzero(clear)[worst]} is off by {frac:.2e} of its largest logit"
        if self.dtype != "float32":
            # A choice that rounding did flip at an unclear position also moves the positions that look
            # back at it: a few may be further off than rounding alone explains, none by much.
            over = np.abs(got - want).max(axis=1) > self.bound * np.abs(want).max(axis=1)
            assert over.mean() <= 0.05, f"{label}: request {rid}: {over.sum()} of {len(over)} positions are off by more than {self.bound}"


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


def test_every_layer_run_of_a_looped_model(tmp):
    """The stream after every run of a layer, a looped layer counted each time, in float32."""
    from pylon_amd.engine import StepEntry
    from pylon_amd.parts.base import summed

    case = Case(tmp, "U", "float32", (40,))
    runner = case.runner()
    kept = []
    for block in runner.model.blocks:
        def wrapped(resid, delta, ctx, cache, stores, inner=block.forward):
            resid, delta = inner(resid, delta, ctx, cache, stores)
            kept.append((resid + summed(delta)).cpu().numpy())
            return resid, delta
        block.forward = wrapped
    seq = runner.open("a")
    runner.step([StepEntry(seq, case.requests["r0"], [0])])
    _, want = plain.forward(case.cfg, case.weights, case.requests["r0"], keep_layers=True)
    assert len(kept) == len(want) == 8
    for run, (got, ref) in enumerate(zip(kept, want)):
        assert np.abs(got - ref).max() <= 1e-4 * np.abs(ref).max(), f"run {run}"


@pytest.mark.parametrize("name, dtype, page", [("U", "float32", 16), ("V", "float32", 16), ("W", "float32", 16),
                                                ("X", "float32", 32), ("W", "bfloat16", 16), ("W", "bfloat16", 64),
                                                ("X", "bfloat16", 64), ("U", "bfloat16", 16), ("V", "bfloat16", 32)])
def test_whole_token_by_token_and_in_portions(tmp, name, dtype, page):
    case = Case(tmp, name, dtype, (171, 38))
    runner = case.runner(page_size=page, num_pages=1280 // page)
    whole, _ = run_plan(runner, case, [{"r0": 171}, {"r0": 0, "r1": 38}])
    for rid, got in whole.items():
        case.check(rid, got, "whole")
    single, _ = run_plan(runner, case, [{"r1": 1} for _ in range(38)])
    case.check("r1", single["r1"], "token by token")
    cut, _ = run_plan(runner, case, [{"r0": n} for n in (2, 3, 2, 17, 1, 1, 30, 2, 13, 64, 5, 2, 29)])
    case.check("r0", cut["r0"], "portions")
    if dtype == "float32":  # how a request is cut moves nothing but the order of a product's sums
        assert np.abs(cut["r0"] - whole["r0"]).max() <= 2e-5 * np.abs(whole["r0"]).max()
        assert np.abs(single["r1"] - whole["r1"]).max() <= 2e-5 * np.abs(whole["r1"]).max()


@pytest.mark.parametrize("name, dtype, page", [("U", "float32", 16), ("V", "float32", 16), ("W", "bfloat16", 16),
                                                ("W", "bfloat16", 32), ("X", "bfloat16", 64), ("X", "float32", 16)])
def test_mixed_batches_over_pages_and_slots_that_are_used_again(tmp, name, dtype, page):
    case = Case(tmp, name, dtype, (60, 45, 33, 20))
    pages = 192 // page  # never room for all four requests at once
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


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding_over_pages_that_windows_and_chunks_give_back(tmp, dtype):
    """420 tokens through a pool of 4 pages of 64 a group: a chunk of 70 and a window of 100 never
    need more, because the pages they have passed go back while the request runs."""
    case = Case(tmp, "W", dtype, (420,))
    runner = case.runner(page_size=64, num_pages=4, max_requests=2)
    got, _ = run_plan(runner, case, [{"r0": 100}] + [{"r0": 1}] * 320)
    case.check("r0", got["r0"], "long decoding")
    assert runner.manager.free_pages == 4


def test_requests_do_not_see_what_a_freed_slot_or_page_held(tmp):
    """The same request, alone in a fresh runner and after others have used every page and slot."""
    case = Case(tmp, "U", "float32", (50, 64, 64))
    fresh, _ = run_plan(case.runner(num_pages=8, max_requests=2), case, [{"r0": 50}])
    runner = case.runner(num_pages=8, max_requests=2)
    for group in runner.manager.groups:
        for cache in list(group.k.values()) + [v for v in group.v.values() if v is not None]:
            cache.fill_(float("nan"))
    used, _ = run_plan(runner, case, [{"r1": 64, "r2": 64}, {"r1": 0, "r2": 0}, {"r0": 25}, {"r0": 25}])
    assert np.abs(used["r0"] - fresh["r0"]).max() <= 2e-5 * np.abs(fresh["r0"]).max()


@pytest.mark.parametrize("name, dtype, graphs, page", [("U", "float32", False, 16), ("V", "float32", True, 16),
                                                         ("W", "bfloat16", True, 16), ("W", "bfloat16", True, 64),
                                                         ("X", "bfloat16", True, 64)])
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
            row = plain.forward(cfg, weights, sequence)[-1]
            assert produced == int(row.argmax()) or row.max() - row[produced] <= slack * np.abs(row).max(), \
                (prompt[:3], result.output_ids)
            sequence.append(produced)
