"""The Rutevik design in the engine against the plain implementation: each mechanism alone at the
level of its op or part, then whole models through the step function (whole prompts, decoding
token by token, portions down to two tokens, mixed batches on a pool whose pages and slots are
used again), and greedy generation through the engine's own entry point and scheduler."""
import math

import pytest
import torch

import plain_rutevik as plain
import replay_lib as rl
from helpers import note_error, oracle_logits, random_tokens, read_config, rel_err, tol
from rutevik_models import RUTEVIK_LENGTHS, RUTEVIK_PAGE, clear_tokens

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
DTYPES = {"float32": torch.float32, "bfloat16": torch.bfloat16}
NAMES = ["rvA", "rvB", "rvC", "rvD"]
#: bfloat16: the share of a run's rows that may be over the tolerance, up to four times (rows at which the two
#: maps' outputs nearly cancel, where the norm over the head brings rounding up); the same rows in every way of
#: cutting.  A wrong page or a wrong map moves rows of these models by a tenth of the largest logit and more.
FEW = {"float32": 0.0, "bfloat16": 0.05}


def _ops():
    from tffinfer_amd.kernels import ops
    return ops


def _err(got, ref):
    got, ref = _ops().as_tensor(got).double().cpu(), ref.double().cpu()
    return float((got - ref).abs().max() / ref.abs().max().clamp_min(1e-30))


def _i32(v):
    return torch.tensor(v, dtype=torch.int32, device=DEV)


# ---------------------------------------------------------------- mechanisms, one by one ---

@pytest.mark.parametrize("W", [48, 321, 1030])
def test_norm_without_statistics(W):
    """resid += terms; tanh(alpha v) w + b element by element; or the norm of chosen rows with the stream
    left as it is; the same bits for a row whatever else the step holds."""
    ops = _ops()
    g = torch.Generator().manual_seed(W)
    n, alpha = 6, 0.37
    x = torch.randn(n, W, generator=g) * 3
    w, b = 1 + 0.3 * torch.randn(W, generator=g), torch.randn(W, generator=g)
    planes = torch.randn(3, n, W, generator=g)
    one = torch.randn(n, W, generator=g)
    for terms in (None, [one], [planes], [planes, one]):
        total = x.double()
        for t in terms or []:
            total = total + (t.double().sum(0) if t.dim() == 3 else t.double())
        resid = x.clone().to(DEV)
        delta = None if terms is None else (terms[0].to(DEV) if len(terms) == 1 else ops.PendingTerms([t.to(DEV) for t in terms]))
        out = ops.add_dyt(resid, delta, alpha, w.to(DEV), b.to(DEV), torch.float32)
        assert _err(resid, total) < 1e-6
        assert _err(out, plain.dyt(total, alpha, w.double(), b.double())) < 2e-6
    resid = x.clone().to(DEV)
    y = ops.add_dyt(resid, ops.PendingTerms([planes.to(DEV), one.to(DEV)]), alpha, w.to(DEV), b.to(DEV), torch.float32,
                    rows=_i32([4, 0, 2]))
    total = x.double() + planes.double().sum(0) + one.double()
    assert _err(y, plain.dyt(total, alpha, w.double(), b.double())[[4, 0, 2]]) < 2e-6
    assert torch.equal(resid.cpu(), x)
    resid = x.clone().to(DEV)
    h = ops.add_dyt(resid, one.to(DEV), alpha, w.to(DEV), b.to(DEV), torch.bfloat16)
    assert _err(h.float(), plain.dyt(x.double() + one.double(), alpha, w.double(), b.double())) < 5e-3
    many, mb = torch.randn(150, W, generator=g), torch.randn(150, W, generator=g)
    many[:n], mb[:n] = x, one
    r_many, r_few = many.to(DEV), x.clone().to(DEV)
    o_many = ops.add_dyt(r_many, mb.to(DEV), alpha, w.to(DEV), b.to(DEV), torch.float32)
    o_few = ops.add_dyt(r_few, one.to(DEV), alpha, w.to(DEV), b.to(DEV), torch.float32)
    assert torch.equal(o_many[:n], o_few) and torch.equal(r_many[:n], r_few)


@pytest.mark.parametrize("M,N,K", [(1, 256, 512), (8, 4096, 1024), (16, 320, 72), (5, 2048, 4096)])
def test_norm_in_the_epilogue_of_a_product_of_few_rows(M, N, K):
    """A product of up to 16 bfloat16 rows that has not run yet runs with the sum into the stream and the norm in
    its epilogue: the same stream and the same rows as the product followed by the norm's own kernel."""
    ops = _ops()
    g = torch.Generator().manual_seed(M * N + K)
    x = torch.randn(M, K, generator=g).to(torch.bfloat16).to(DEV)
    wm = (0.05 * torch.randn(N, K, generator=g)).to(torch.bfloat16)
    pw = ops.pack_weight(wm.to(DEV))
    resid0 = torch.randn(M, N, generator=g) * 2
    w, b, alpha = (1 + 0.3 * torch.randn(N, generator=g)).to(DEV), torch.randn(N, generator=g).to(DEV), 0.41
    pending = ops.linear(x, pw, out_dtype=torch.float32, partials=True)
    plain_run = ops.linear(x, pw, out_dtype=torch.float32)
    r1, r2 = resid0.clone().to(DEV), resid0.clone().to(DEV)
    fused = ops.add_dyt(r1, pending, alpha, w, b, torch.bfloat16)
    apart = ops.add_dyt(r2, plain_run, alpha, w, b, torch.bfloat16)
    if isinstance(pending, ops.PendingProduct):
        assert torch.equal(r1, r2) and torch.equal(fused, apart)
    total = resid0.double() + x.double().cpu() @ wm.double().T
    assert _err(r1, total) < 2e-6
    assert _err(fused.float(), plain.dyt(total, alpha, w.double().cpu(), b.double().cpu())) < 5e-3


def test_square_of_relu():
    ops = _ops()
    z = torch.linspace(-6, 6, 2001)
    assert _err(ops.relu_squared(z.to(DEV)), torch.relu(z.double()) ** 2) < 1e-6
    zb = z.to(torch.bfloat16)
    assert _err(ops.relu_squared(zb.to(DEV)).float(), torch.relu(zb.double()) ** 2) < 5e-3
    assert float(ops.relu_squared(z.to(DEV))[:1000].abs().max()) == 0.0


@pytest.mark.parametrize("E,top", [(8, 3), (2, 2), (5, 1), (40, 4)])
def test_experts_whose_scores_weigh_their_inputs(E, top):
    """s = sigmoid(router logits); the top largest chosen; the weights are the chosen scores as they are (they do
    not add up to one) and multiply what goes into the expert: silu(gate) * up is not linear, so a weight on the
    output gives another result, which the test shows to differ."""
    ops = _ops()
    g = torch.Generator().manual_seed(E)
    T, W, ff = 40, 48, 24
    x = torch.randn(T, W, generator=g).to(torch.bfloat16).float()
    P = {"router": (0.4 * torch.randn(E, W, generator=g)).double()}
    for e in range(E):
        for n, shape in (("gate", (ff, W)), ("up", (ff, W)), ("down", (W, ff))):
            P[f"e{e}.{n}"] = (0.3 * torch.randn(shape, generator=g)).to(torch.bfloat16).double()
    m = {"router": {"top": top, "experts": E}}
    ref = plain.routed_experts(m, P, x.double())
    idx, wts = ops.route_topk(x.to(DEV), P["router"].float().to(DEV), None, top, normalize=False)
    s = plain.sigmoid(x.double() @ P["router"].T)
    want = torch.topk(s, top).indices
    assert torch.equal(idx.cpu().long(), want)
    assert _err(wts, torch.gather(s, 1, want)) < 1e-6
    if top > 1:
        assert float((wts.sum(1) - 1).abs().max()) > 0.1
    stack = lambda n: ops.pad_expert_rows(torch.stack([P[f"e{e}.{n}"] for e in range(E)], 0).float()).to(DEV)   # noqa: E731
    out = ops.routed_experts(x.to(DEV), stack("gate"), stack("up"), stack("down"), idx, wts, float("inf"), 1.0,
                             up_offset=0.0, weight_input=True)
    assert _err(out, ref) < 2e-5
    wrong = ops.routed_experts(x.to(DEV), stack("gate"), stack("up"), stack("down"), idx, wts, float("inf"), 1.0,
                               up_offset=0.0, weight_input=False)
    assert _err(wrong, ref) > 1e-2
    b16 = lambda t: t.to(torch.bfloat16)        # noqa: E731
    for by_tiles in (False, True):
        out = ops.routed_experts(b16(x).to(DEV), b16(stack("gate")), b16(stack("up")), b16(stack("down")), idx, wts,
                                 float("inf"), 1.0, by_tiles=by_tiles, up_offset=0.0, weight_input=True)
        assert _err(out, ref) < 3e-2
    # a token alone gives the bits it gives among the others
    args = (stack("gate"), stack("up"), stack("down"))
    full = ops.as_tensor(ops.routed_experts(x.to(DEV), *args, idx, wts, float("inf"), 1.0, up_offset=0.0, weight_input=True))
    alone = ops.as_tensor(ops.routed_experts(x[7:8].to(DEV), *args, idx[7:8].contiguous(), wts[7:8].contiguous(),
                                             float("inf"), 1.0, up_offset=0.0, weight_input=True))
    assert torch.equal(alone[0], full[7])


def _view(cache, batch, cache_id, writes=True):
    from tffinfer_amd.engine.batch import KVView
    gi = cache.group_index(cache_id)
    k, v = cache.kv_tensors(cache_id)
    gt = batch.groups[gi]
    return KVView(k, v, gt.block_tables, gt.slot_mapping if writes else gt.no_slot_mapping, cache.page_size, gi)


def _ctx(cache, entries, act_dtype, max_positions=2048):
    """The context of a step with these entries (pages taken, nothing committed); the part's cache view is set by
    the caller."""
    from tffinfer_amd.engine.batch import build_step_batch
    from tffinfer_amd.engine.runner import LayerContext
    for e in entries:
        if not cache.has_request(e.req):
            cache.add_request(e.req)
        cache.reserve(e.req, len(e.tokens))
    return LayerContext(_ops(), act_dtype, build_step_batch(entries, cache, DEV), max_positions)


def _draw(part, seed, weights=None, scale=0.3):
    g = torch.Generator().manual_seed(seed)
    w = {}
    for k, s in part.weight_specs().items():
        t = torch.randn(s.shape, generator=g)
        w[k] = (1 + 0.2 * t) if s.init == "norm" else ((0.5 * t) if s.init == "norm_offset" else (t * scale).to(torch.bfloat16))
    w.update(weights or {})
    return w


def _run_parts(parts, x, cuts, dtype, page):
    """The parts (the writer of a cache, then readers of it) over rows x of one request in portions ``cuts``;
    returns each part's outputs [T, W]."""
    from tffinfer_amd.cache import CacheManager
    from tffinfer_amd.engine.batch import StepEntry
    T = x.shape[0]
    reqs = [(0, not getattr(p, "shared_cache", False), p.cache_spec(), None) for p in parts]
    cache = CacheManager(reqs, page, -(-T // page) + 2, 2, dtype=dtype, device=DEV)
    outs, at = [[] for _ in parts], 0
    for n in cuts:
        ctx = _ctx(cache, [StepEntry("r", [0] * n, [])], dtype)
        rows = x[at:at + n].to(dtype).to(DEV)
        for i, part in enumerate(parts):
            ctx.kv = _view(cache, ctx.batch, 0, writes=not getattr(part, "shared_cache", False))
            outs[i].append(_ops().as_tensor(part.forward(ctx, rows)).float())
        cache.commit("r", n)
        at += n
    assert at == T
    return [torch.cat(o, 0) for o in outs]


def _latent_part(W, H, D, R, E, rank, q_rank, scale, base, eps, dtype, seed, shared=False, weights=None):
    from tffinfer_amd.config.base import PartSpec
    from tffinfer_amd.parts import LatentAttention
    pos = PartSpec("rope", {"head_dim": R, "theta": base, "pairing": "half", "rotary_dim": R}) if R else None
    att = LatentAttention(hidden_size=W, num_heads=H, head_dim=D, rot_dim=R, value_dim=E, kv_rank=rank, scale=scale,
                          position=pos, latent_norm_eps=eps, sink=False, output_gate=False, q_rank=q_rank, shared_cache=shared)
    w = _draw(att, seed, weights)
    att.load_weights(w, dtype, DEV)
    m = {"heads": H, "dim": D, "rot_dim": R, "vdim": E, "kv_rank": rank, "q_rank": q_rank, "scale": scale,
         "rot": {"dims": R, "base": base}}
    return att, m, {k: v.double() for k, v in w.items()}


@pytest.mark.parametrize("dtype,limit", [(torch.float32, 2e-5), (torch.bfloat16, 3e-2)])
@pytest.mark.parametrize("H,D,R,E,rank,q_rank,page", [
    (3, 16, 8, 24, 40, 24, 16),
    (1, 64, 32, 64, 64, 16, 8),
    (5, 12, 6, 20, 30, 18, 32),          # no size a multiple of 8
    (8, 64, 32, 64, 160, 96, 16),        # a key of 192
    (2, 32, 64, 40, 272, 48, 16),        # a key of 336, beyond the sizes of the matrix-core attention
    (2, 16, 64, 24, 512, 32, 16)])       # a key of 576
def test_latent_attention_with_a_latent_query_and_a_reader(H, D, R, E, rank, q_rank, page, dtype, limit):
    """Queries through a normed latent vector, keys and values through another, the rotated part turned in halves;
    a second attention with its own queries and up-projections reads the cache the first one fills.  A prompt in
    one step, as portions down to two tokens, and as a portion followed by single tokens."""
    W, T, eps = 48, 150, 1e-5
    own, m, P = _latent_part(W, H, D, R, E, rank, q_rank, 0.2, 3000.0, eps, dtype, 11)
    reader, m2, P2 = _latent_part(W, max(1, H - 1), D + 4, R, E + 4, rank, q_rank + 2, 0.15, 3000.0, eps, dtype, 12, shared=True)
    assert "dkv" not in reader.weight_specs() and reader.cache_spec() == own.cache_spec()
    g = torch.Generator().manual_seed(7)
    x = torch.randn(T, W, generator=g).to(torch.bfloat16).float()
    cache = plain.latent_cache(m, P, x.double(), eps)
    refs = [plain.latent_attention(m, P, x.double(), eps, cache), plain.latent_attention(m2, P2, x.double(), eps, cache)]
    for cuts in ([T], [3, 2, 61, 64, 20], [90] + [1] * 60):
        for out, ref, who in zip(_run_parts([own, reader], x, cuts, dtype, page), refs, ("own", "reader")):
            err = _err(out, ref)
            assert err < limit, f"{who}, cut {cuts[:3]}: {err:.3e}"


def _diff_part(W, H, G, D, E, scale, diff, rot, softcap, scaling, eps, dtype, seed, weights=None):
    from tffinfer_amd.config.base import PartSpec
    from tffinfer_amd.parts import DifferentialAttention
    pos = None
    if rot:
        args = {"head_dim": D, "theta": rot[1], "pairing": "half", "rotary_dim": rot[0]}
        if scaling:
            args.update(dict(zip(("factor", "low", "high", "original"), scaling)))
        pos = PartSpec("rope_scaled" if scaling else "rope", args)
    att = DifferentialAttention(hidden_size=W, num_heads=H, num_kv_heads=G, head_dim=D, value_dim=E, position=pos,
                                scale=scale, softcap=softcap, diff=diff, norm_eps=eps)
    w = _draw(att, seed, weights)
    att.load_weights(w, dtype, DEV)
    m = {"heads": H, "kv_heads": G, "dim": D, "vdim": E, "scale": scale, "diff": diff,
         "rot": {"dims": rot[0], "base": rot[1]} if rot else {"dims": 0, "base": 1.0}}
    if softcap:
        m["softcap"] = softcap
    if scaling:
        m["rot"]["scaling"] = dict(zip(("factor", "low", "high", "original"), scaling))
    return att, m, {k: v.double() for k, v in w.items()}


@pytest.mark.parametrize("dtype,limit", [(torch.float32, 3e-5), (torch.bfloat16, 4e-2)])
@pytest.mark.parametrize("H,G,D,E,rot,softcap,scaling,page", [
    (4, 2, 16, 24, (8, 500.0), 5.0, (4.0, 1.0, 2.0, 32), 16),     # a part of every map rotated, long waves slowed down
    (2, 1, 32, 48, (32, 1e6), None, None, 8),                    # values narrower than two maps, no cap
    (6, 6, 8, 8, (8, 50.0), 2.0, None, 32),                      # heads that are not grouped, a tight cap
    (3, 1, 12, 20, (4, 1e4), 12.0, (2.0, 1.0, 3.0, 16), 16),     # no multiples of 8
    (8, 2, 64, 128, (64, 1e4), 20.0, (8.0, 1.0, 4.0, 64), 16),   # the sizes of a real model
    (2, 1, 128, 96, (32, 1e4), 9.0, None, 16),                   # a key row of 256: capped scores on the general kernel
    (2, 2, 24, 200, (24, 1e3), None, None, 8)])                  # values far wider than two maps
def test_differential_attention_part(H, G, D, E, rot, softcap, scaling, page, dtype, limit):
    """Two score maps a head with biases, rotation, a cap on the scores, the difference with lambda, the norm over
    the head, the gate: a prompt in one step, as portions down to two tokens, and as a portion followed by single
    tokens."""
    W, T, eps = 48, 150, 1e-5
    att, m, P = _diff_part(W, H, G, D, E, 0.4, 0.25, rot, softcap, scaling, eps, dtype, H * D + E)
    g = torch.Generator().manual_seed(7)
    x = torch.randn(T, W, generator=g).to(torch.bfloat16).float()
    ref = plain.differential_attention(m, P, x.double(), eps)
    for cuts in ([T], [3, 2, 61, 64, 20], [90] + [1] * 60):
        err = _err(_run_parts([att], x, cuts, dtype, page)[0], ref)
        assert err < limit, f"cut {cuts[:3]}: {err:.3e}"
    if softcap:       # the cap matters at these sizes: without it the result is another
        m2 = dict(m)
        del m2["softcap"]
        assert _err(plain.differential_attention(m2, P, x.double(), eps), ref) > 10 * limit


@pytest.mark.parametrize("decode", [False, True])
@pytest.mark.parametrize("which", [0, 1])
@pytest.mark.parametrize("far", [299, 288, 287, 16, 15, 1])
def test_a_loud_far_key_on_one_map(far, which, decode):
    """One key whose score with the last query stands far out among 300, on one of the two maps only (the other
    map's queries are zero and see all keys alike), up to 299 tokens back and on either side of a page's border.
    Without that key, and with the loud map being the other one, the plain result is far away: a key or a map
    that the engine loses shows.  In a prompt and in decoding."""
    W = 8
    H, G, D, E, T, page, eps, diff = 1, 1, 8, 12, 301, 16, 1e-6, 0.25
    j = T - 1 - far
    zero, eye = torch.zeros(D, W), torch.eye(D, W)

    def part(loud):
        fixed = {"q": (torch.cat([eye, zero]) if loud == 0 else torch.cat([zero, eye])).to(torch.bfloat16),
                 "k": torch.cat([eye, eye]).to(torch.bfloat16), "q.b": torch.zeros(2 * D), "k.b": torch.zeros(2 * D)}
        return _diff_part(W, H, G, D, E, 4.0, diff, None, 40.0, None, eps, torch.float32, 5, weights=fixed)

    att, m, P = part(which)
    g = torch.Generator().manual_seed(9)
    x = 0.05 * torch.randn(T, W, generator=g).to(torch.bfloat16).float()
    x[:, 3] = 0
    x[j] = 0
    x[j, 3] = 3.0                                   # token j's key lies along axis 3, and no other key's does ...
    x[j, 5], x[j, 6] = -4.0, 4.0                    # (its value is unlike any other's)
    x[T - 1, 3] = 3.0                               # ... but the last token's, whose query lies there too
    ref = plain.differential_attention(m, P, x.double(), eps)
    out = _run_parts([att], x, [T - 1, 1] if decode else [T], torch.float32, page)[0]
    assert _err(out, ref) < 3e-5
    without = x.clone()
    without[j, 3] = 0
    lost = plain.differential_attention(m, P, without.double(), eps)
    assert _err(lost[-1], ref[-1]) > 0.1
    _, m_other, P_other = part(1 - which)
    assert _err(plain.differential_attention(m_other, P_other, x.double(), eps)[-1], ref[-1]) > 0.1


def test_a_far_key_through_a_borrowed_cache():
    """A reader of another layer's cache finds keys up to 300 tokens back that the writer stored, across the
    borders of pages and portions; with the stored keys' positions one off the plain result is another, so the
    rotation that the writer applied is the one the reader's queries meet."""
    W, T, eps, page = 48, 300, 1e-5, 16
    own, m, P = _latent_part(W, 2, 16, 16, 8, 24, 16, 0.5, 40.0, eps, torch.float32, 21)
    reader, m2, P2 = _latent_part(W, 3, 8, 16, 12, 24, 20, 0.5, 40.0, eps, torch.float32, 22, shared=True)
    g = torch.Generator().manual_seed(3)
    x = torch.randn(T, W, generator=g).to(torch.bfloat16).float()
    cache = plain.latent_cache(m, P, x.double(), eps)
    ref = plain.latent_attention(m2, P2, x.double(), eps, cache)
    for cuts in ([T], [T - 20] + [1] * 20, [16, 1, 15, 250, 18]):
        out = _run_parts([own, reader], x, cuts, torch.float32, page)[1]
        assert _err(out, ref) < 3e-5
    raw = (x.double() @ P["dkv"].T)[:, 24:]
    shifted = (cache[0], plain.rotate(raw, plain.frequencies(16, 40.0), first_pos=1))
    assert _err(plain.latent_attention(m2, P2, x.double(), eps, shifted), ref) > 1e-2


def test_batches_of_unequal_requests_share_the_mixers():
    """Three requests in one step (a prompt's portion, a single token, a whole short prompt) through a differential
    attention and through a latent attention with a reader give what each gives alone; freed pages are used again."""
    from tffinfer_amd.cache import CacheManager
    from tffinfer_amd.engine.batch import StepEntry
    W, eps, page = 40, 1e-5, 8
    att, m, P = _diff_part(W, 4, 2, 16, 24, 0.3, 0.2, (8, 100.0), 6.0, None, eps, torch.float32, 31)
    own, lm, LP = _latent_part(W, 2, 16, 8, 12, 24, 16, 0.3, 100.0, eps, torch.float32, 32)
    reader, rm, RP = _latent_part(W, 3, 8, 8, 20, 24, 12, 0.3, 100.0, eps, torch.float32, 33, shared=True)
    g = torch.Generator().manual_seed(2)
    lengths = [60, 41, 7]
    xs = [torch.randn(n, W, generator=g).to(torch.bfloat16).float() for n in lengths]

    def refs_of(x):
        c = plain.latent_cache(lm, LP, x.double(), eps)
        return [plain.differential_attention(m, P, x.double(), eps), plain.latent_attention(lm, LP, x.double(), eps, c),
                plain.latent_attention(rm, RP, x.double(), eps, c)]

    refs = [refs_of(x) for x in xs]
    cache = CacheManager([(0, True, att.cache_spec(), None), (1, True, own.cache_spec(), None), (1, False, reader.cache_spec(), None)],
                         page, 18, 3, dtype=torch.float32, device=DEV)

    def step(parts):
        entries = [StepEntry(f"r{r}", [0] * (hi - lo), []) for r, lo, hi in parts]
        rows = torch.cat([xs[r][lo:hi] for r, lo, hi in parts], 0).to(DEV)
        ctx = _ctx(cache, entries, torch.float32)
        outs = []
        for part, cache_id, writes in ((att, 0, True), (own, 1, True), (reader, 1, False)):
            ctx.kv = _view(cache, ctx.batch, cache_id, writes)
            outs.append(_ops().as_tensor(part.forward(ctx, rows)))
        at = 0
        for (r, lo, hi), e in zip(parts, entries):
            for i, o in enumerate(outs):
                assert _err(o[at:at + hi - lo], refs[r][i][lo:hi]) < 3e-5, (r, lo, hi, i)
            at += hi - lo
            cache.commit(e.req, hi - lo)

    step([(0, 0, 35), (1, 0, 40)])
    step([(0, 35, 60), (1, 40, 41), (2, 0, 7)])
    for r in range(3):
        cache.release(f"r{r}")
    xs[0], xs[1] = xs[1], xs[0]
    refs[0], refs[1] = refs[1], refs[0]
    step([(1, 0, 2), (0, 0, 30)])
    step([(1, 2, 60), (0, 30, 41)])
    cache.check()


# ---------------------------------------------------------------------- whole models ---

def requests_for(name, model_dir):
    V = read_config(model_dir)["vocab"]
    # (sequences in which no choice of experts is a close call that rounding could turn)
    return {f"{name}{i}": list(clear_tokens(model_dir, n, V, 3000 + 13 * i + n)) for i, n in enumerate(RUTEVIK_LENGTHS[name])}


def make_runner(model_dir, dtype, page_size, num_pages, max_seqs=4, use_graphs=False):
    from tffinfer_amd.engine.runner import ModelRunner
    from tffinfer_amd.models import load_model
    model = load_model(model_dir, DTYPES[dtype], DEV)
    return ModelRunner(model, page_size=page_size, num_pages=num_pages, max_seqs=max_seqs, max_model_len=512,
                       use_graphs=use_graphs)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", NAMES)
def test_residual_stream_after_every_layer(rutevik_dirs, name, dtype):
    """Layer by layer, so that a fault names its layer.  A block leaves its feed-forward's output to the norm
    after it; the stream after a layer is the stream plus what is pending."""
    from tffinfer_amd.engine.batch import StepEntry, build_step_batch
    from tffinfer_amd.engine.runner import StepContext
    d = rutevik_dirs[name]
    toks = list(clear_tokens(d, 45, read_config(d)["vocab"], 77))
    want = []
    plain.forward(*plain.load(d), toks, want)
    runner = make_runner(d, dtype, RUTEVIK_PAGE[name], 16)
    model, ops = runner.model, runner.ops
    runner.add_request("a")
    e = [StepEntry("a", toks, [])]
    runner.reserve(e)
    batch = build_step_batch(e, runner.cache, runner.device, runner._pinned)
    ctx = StepContext(ops, runner.act_dtype, batch, runner.max_model_len, runner._calls, runner.cache)
    resid, pending = model.embedding.forward(ctx, batch.token_ids), None
    assert len(model.schedule) == len(want)
    for it, call in enumerate(model.schedule):
        pending = model.blocks[call.layer].forward(ctx.for_call(it), resid, pending)
        after = resid + ops.as_tensor(pending) if pending is not None else resid
        err = _err(after, want[it])
        assert err < (4e-5 if dtype == "float32" else 5e-2), f"layer {it}: {err:.3e}"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", NAMES)
@pytest.mark.parametrize("mode", ["whole", "tail", "chunks", "mixed"])
def test_replay_modes(rutevik_dirs, name, dtype, mode):
    model_dir = rutevik_dirs[name]
    reqs = requests_for(name, model_dir)
    steps = {"whole": rl.trace_whole, "tail": rl.trace_tail, "chunks": rl.trace_chunks,
             "mixed": rl.trace_mixed}[mode](reqs)
    ps = RUTEVIK_PAGE[name]
    # the pool holds what is live at the worst moment and no more, so pages and slots are used again
    num_pages = rl.max_live_tokens(steps, unit=ps) // ps
    runner = make_runner(model_dir, dtype, ps, num_pages)
    results = rl.run_steps_in_process(runner, steps)
    worst = rl.check_against_oracle(model_dir, reqs, steps, results, tol(dtype, name), dtype, few_over=FEW[dtype])
    print(f"{name} {dtype} {mode}: worst rel. error {worst:.3e} over {len(steps)} steps, {num_pages} pages")
    assert all(g.pool.num_used == 0 for g in runner.cache.groups)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["rvA", "rvD"])
def test_long_decoding_through_captured_graphs(rutevik_dirs, name, dtype):
    """Three requests decode some 150 tokens each as replays of captured HIP graphs beside eager prompt steps."""
    model_dir = rutevik_dirs[name]
    V = read_config(model_dir)["vocab"]
    reqs = {f"g{i}": list(clear_tokens(model_dir, n, V, 300 + n)) for i, n in enumerate((160, 171, 190))}
    steps = rl.trace_mixed(reqs, max_live=3, prompt_frac=0.1, want_all=True)
    ps = RUTEVIK_PAGE[name]
    runner = make_runner(model_dir, dtype, ps, rl.max_live_tokens(steps, unit=ps) // ps, use_graphs=True)
    results = rl.run_steps_in_process(runner, steps)
    rl.check_against_oracle(model_dir, reqs, steps, results, tol(dtype, name), dtype, few_over=FEW[dtype])
    assert runner._graphs, "no decode step ran as a graph"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_run_program(rutevik_dirs, tmp_path, dtype):
    """The program itself, as a user calls it, on a model of this architecture."""
    model_dir = rutevik_dirs["rvB"]
    reqs = requests_for("rvB", model_dir)
    steps = rl.trace_mixed(reqs, want_all=False)
    out = rl.run_steps_subprocess(model_dir, dtype, steps, str(tmp_path / "out"), rl.max_live_tokens(steps, 64))
    rl.check_against_oracle(model_dir, reqs, steps, out, tol(dtype, "rvB"), dtype, few_over=FEW[dtype])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["rvA", "rvC"])
def test_greedy_generation_through_the_engine(rutevik_dirs, name, dtype):
    """The engine's own entry point: scheduler, portions beside decoding requests, graphs, sampler.
    Every kept row of logits matches the plain logits of the engine's own sequence (rows whose routers make a
    close call apart), and every token is the first maximum of its row."""
    from tffinfer_amd import EngineOptions, LLMEngine
    from rutevik_models import MIN_MARGIN
    d = rutevik_dirs[name]
    V = read_config(d)["vocab"]
    prompts = [list(clear_tokens(d, n, V, 80 + n)) for n in (1, 9, 40, 70)]
    eng = LLMEngine.from_model_dir(d, EngineOptions(dtype=dtype, page_size=16, kv_tokens=512, max_num_seqs=3,
                                                    max_num_batched_tokens=48, prefill_chunk=24, max_model_len=256))
    eng.keep_logits = True
    res = eng.generate(prompts, max_new_tokens=40, ignore_eos=True)
    cfg, Wt = plain.load(d)
    over = 0
    for r in res:
        assert len(r.output) == 40 and r.finish_reason == "length"
        margins = []
        ref = plain.forward(cfg, Wt, r.prompt + r.output, margins=margins)
        gap = torch.stack(margins, 0).min(0).values if margins else torch.full((len(r.prompt) + 40,), math.inf)
        # a close call turns an expert for that token and, through the cache, may move every later row
        close = (gap < MIN_MARGIN).nonzero()
        upto = int(close[0]) if (close.numel() and dtype == "bfloat16") else len(gap)
        for i, (row, tok) in enumerate(zip(r.logits, r.output)):
            assert tok == int(torch.argmax(row))
            at = len(r.prompt) + i - 1
            if at >= upto:
                break
            err = rel_err(row, ref[at])
            if FEW[dtype] and tol(dtype, d) < err <= 4 * tol(dtype, d):
                over += 1
                continue
            note_error(dtype, d, err)
            assert err <= tol(dtype, d), f"output {i}: {err:.3e}"
    assert over <= max(1, int(FEW[dtype] * 160))
    if dtype == "float32":
        toks = list(prompts[1])
        for _ in range(8):
            toks.append(int(torch.argmax(plain.forward(cfg, Wt, toks)[-1])))
        assert res[1].output[:8] == toks[len(prompts[1]):]


def test_the_command_line_with_a_configuration_file_of_this_architecture(tmp_path):
    """--config FILE --random-weights through bin/tffinfer: the weights are those of the folder that
    --save-model writes, the dumped rows are the logits that chose each token."""
    import json
    import os
    import subprocess
    import sys
    import numpy as np
    from rutevik_models import RV_B
    prog = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "bin", "tffinfer")
    cfg = tmp_path / "config.json"
    cfg.write_text(json.dumps(RV_B))
    folder, dump = str(tmp_path / "rvB"), str(tmp_path / "logits.f32")
    cmd = [sys.executable, prog, "--config", str(cfg), "--random-weights", "--seed", "5", "--fp32", "--n-ctx", "256",
           "--n-predict", "12", "--ignore-eos", "--json", "--random-prompts", "3:30", "--page-size", "8",
           "--max-batches", "3", "--save-model", folder, "--dump-logits", dump, "--kv-tokens", "512"]
    p = subprocess.run(cmd, capture_output=True, text=True, timeout=300)
    assert p.returncode == 0, p.stderr[-3000:]
    recs = [json.loads(ln) for ln in p.stdout.strip().splitlines()]
    meta = json.load(open(dump + ".json"))
    V = RV_B["vocab"]
    rows = np.fromfile(dump, dtype="<f4").reshape(meta["shape"])
    assert meta["shape"] == [36, V]
    for i, r in enumerate(recs):
        ref = oracle_logits(folder, r["prompt"] + r["output"])
        first = meta["requests"][i]["first_row"]
        for j, tok in enumerate(r["output"]):
            row = torch.from_numpy(rows[first + j].copy())
            assert rel_err(row, ref[len(r["prompt"]) - 1 + j]) <= tol("float32", "rvB")
            assert tok == int(torch.argmax(row))
