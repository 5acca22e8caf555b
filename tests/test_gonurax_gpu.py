"""Gonurax on the GPU: each new kernel against the plain implementation's function for the same mechanism, then whole
models of the tests' own sizes through the engine's step function, cache manager and scheduler, cut in every way."""

from __future__ import annotations

import pytest
import torch

import gonurax_helpers as gh
import plain_gonurax as plain
import trace_helpers as th

pytestmark = pytest.mark.gpu

F64 = torch.float64
TOL = {torch.float32: 2e-5, torch.bfloat16: 2e-2}


def rel_err(got: torch.Tensor, want: torch.Tensor) -> float:
    """Largest error of a row against that row's largest value."""
    got, want = got.detach().cpu().to(F64), want.detach().cpu().to(F64)
    return float(((got - want).abs().amax(-1) / want.abs().amax(-1).clamp_min(1e-30)).max())


# ------------------------------------------------------------------------------------------------ norm
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("dim,groups", [(96, 3), (80, 5), (256, 1), (1024, 2), (40, 40)])
def test_grouped_norm_with_a_scaled_delta(dim, groups, dtype):
    from mini_engine_amd.ops import kernels as K

    g = torch.Generator().manual_seed(dim + groups)
    x = torch.randn(7, dim, generator=g)
    delta = torch.randn(7, dim, generator=g).to(dtype)
    w = 1.0 + 0.3 * torch.randn(dim, generator=g)
    xs = x.cuda()
    got = K.add_group_rmsnorm(xs, delta.cuda(), w.cuda(), 1e-5, dtype, groups=groups, delta_scale=0.7)
    s = x.to(F64) + 0.7 * delta.to(F64)
    assert rel_err(xs, s) < 1e-6  # the stream holds the sum
    assert rel_err(got, plain.grouped_rms_norm(s, w, groups, 1e-5)) < TOL[dtype]
    # partial sums, rows picked, nothing written
    parts = torch.randn(3, 7, dim, generator=g)
    rows = torch.tensor([5, 0, 6], dtype=torch.int32)
    xs2 = x.cuda()
    got = K.add_group_rmsnorm(xs2, K.PartialSums(parts.cuda()), w.cuda(), 1e-6, dtype, groups=groups, delta_scale=1.5,
                              rows=rows.cuda(), write_x=False)
    s = (x.to(F64) + 1.5 * parts.to(F64).sum(0))[rows.long()]
    assert torch.equal(xs2.cpu(), x)
    assert rel_err(got, plain.grouped_rms_norm(s, w, groups, 1e-6)) < TOL[dtype]
    # no delta at all
    got = K.add_group_rmsnorm(x.cuda(), None, w.cuda(), 1e-6, dtype, groups=groups)
    assert rel_err(got, plain.grouped_rms_norm(x.to(F64), w, groups, 1e-6)) < TOL[dtype]
    y = x.cuda()
    K.residual_add_scaled(y, delta.cuda(), -0.25)
    assert rel_err(y, x.to(F64) - 0.25 * delta.to(F64)) < 1e-6


# ------------------------------------------------------------------------------------------- attention
def plain_attention_rows(qkv, start, nh, nkv, d, dv, q_w, k_w, eps, rd, base, pairing, turn_values, scale, size, keep):
    """What the kernels should give for one sequence whose projections are ``qkv`` ``[L, nh d + nkv d + nkv dv]``: rows
    from ``start`` on."""
    L = qkv.shape[0]
    p = torch.arange(L)
    q = qkv[:, : nh * d].reshape(L, nh, d).to(F64)
    k = qkv[:, nh * d : (nh + nkv) * d].reshape(L, nkv, d).to(F64)
    v = qkv[:, (nh + nkv) * d :].reshape(L, nkv, dv).to(F64)
    if q_w is not None:
        q, k = plain.unit_rms(q, eps) * q_w.to(F64), plain.unit_rms(k, eps) * k_w.to(F64)
    if rd:
        q, k = plain.rotate_pairs(q, p, rd, base, pairing), plain.rotate_pairs(k, p, rd, base, pairing)
    if turn_values:
        v = plain.rotate_pairs(v, p, dv, base, pairing)
    out = torch.zeros(L, nh, dv, dtype=F64)
    for i in range(start, L):
        js = [j for j in range(L) if plain.visible(i, j, size, keep)]
        for h in range(nh):
            kv = h // (nh // nkv)
            out[i, h] = torch.softmax((k[js, kv] @ q[i, h]) * scale, 0) @ v[js, kv]
    if turn_values:
        out = plain.rotate_pairs(out, p, dv, base, pairing, sign=-1.0)
    return out[start:].reshape(L - start, nh * dv)


def angle_table(n, base, positions):
    j = torch.arange(n // 2, dtype=F64)
    ang = torch.arange(positions, dtype=F64)[:, None] * torch.exp(-(2.0 * j / n) * torch.log(torch.tensor(base, dtype=F64)))
    return torch.stack((torch.cos(ang), torch.sin(ang)), 1).float().contiguous().cuda()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("nh,nkv,d,dv,rd,pairing,size,keep,bs,normed,turned", [
    (4, 2, 32, 48, 16, "interleaved", 24, 5, 16, True, True),
    (3, 3, 24, 20, 24, "interleaved", 17, 17, 8, True, True),
    (6, 1, 64, 32, 32, "halves", 300, 3, 32, False, True),
    (2, 2, 16, 16, 16, "interleaved", 40, 0, 16, True, False),
    (4, 1, 128, 72, 64, "halves", 70, 9, 16, True, True),
])
def test_window_attention_in_portions_with_one_key_that_stands_out(nh, nkv, d, dv, rd, pairing, size, keep, bs, normed, turned,
                                                                 dtype):
    """A sequence of 330 tokens through the scatter and attention kernels in portions cut in the middle of pages and of the
    window, pages in random order. One key far back, one among the kept first ones, one at a page border and one per
    window edge are made large and every query leans towards them, so that a key seen or missed by one position moves
    the output by far more than the tolerance."""
    from mini_engine_amd.ops import kernels as K

    L, base, eps, scale = 330, 500.0, 1e-5, 0.3
    g = torch.Generator().manual_seed(nh * 1000 + d)
    qkv = torch.randn(L, nh * d + nkv * (d + dv), generator=g) * 0.5
    u = torch.randn(d, generator=g)
    loud = [0, max(keep - 1, 0), keep, 63, 64, 150, L - size, L - size - 1, L - 2]
    if not rd or rd < d:  # elements that the rotation leaves alone carry the signal at any distance
        u[:rd] = 0
    for j in loud:
        if 0 <= j < L:
            qkv[j, nh * d + (j % nkv) * d : nh * d + (j % nkv + 1) * d] += 3.0 * u
    qkv[:, : nh * d] += 0.7 * u.repeat(nh)
    qkv = qkv.to(dtype)
    q_w = (1.0 + 0.2 * torch.randn(d, generator=g)) if normed else None
    k_w = (1.0 + 0.2 * torch.randn(d, generator=g)) if normed else None
    want = plain_attention_rows(qkv.float(), 0, nh, nkv, d, dv, q_w, k_w, eps, rd, base, pairing, turned, scale, size, keep)

    pages = -(-L // bs)
    order = torch.randperm(pages + 3, generator=g)[:pages].to(torch.int32)
    k_cache = torch.zeros(pages + 3, nkv, bs, d, dtype=dtype, device="cuda")
    v_cache = torch.zeros(pages + 3, nkv, dv, bs, dtype=dtype, device="cuda")
    table = order[None, :].contiguous().cuda()
    rope = angle_table(rd, base, 512) if rd else None
    vt = angle_table(dv, base, 512) if turned else None
    code = 0 if pairing == "halves" else 1
    cuts = [0, 1, 3, 70, 71, 200, 233, 235, L]
    outs = []
    for lo, hi in zip(cuts, cuts[1:]):
        pos = torch.arange(lo, hi, dtype=torch.int32, device="cuda")
        item = torch.zeros(hi - lo, dtype=torch.int32, device="cuda")
        q = K.qkv_rotate_scatter(qkv[lo:hi].cuda().contiguous(), None if q_w is None else q_w.cuda(),
                                 None if k_w is None else k_w.cuda(), rope, code, vt, code, pos, item, table, k_cache, v_cache,
                                 nh, nkv, d, dv, eps)
        outs.append(K.attention_general(q, k_cache, v_cache, pos, item, table, scale, size, keep_first=keep, unturn=vt,
                                        un_pairing=code))
    got = torch.cat(outs)
    assert rel_err(got, want) < TOL[dtype] * 2
    # the loud keys matter: the same rows with a window one key shorter are far off where an edge passes one of them
    other = plain_attention_rows(qkv.float(), 0, nh, nkv, d, dv, q_w, k_w, eps, rd, base, pairing, turned, scale, size - 1, keep)
    assert rel_err(other, want) > 0.05


@pytest.mark.parametrize("nh,nkv,d,rd,pairing,size,keep", [(4, 2, 64, 32, "interleaved", 50, 6), (8, 8, 32, 32, "halves", 100, 70),
                                                          (6, 1, 128, 128, "interleaved", 70, 1), (2, 1, 64, 64, "halves", 200, 130)])
def test_tiled_prompt_attention_sees_the_kept_first_keys(nh, nkv, d, rd, pairing, size, keep):
    """bfloat16 prompts and portions with keys and values of one size go to the tiled matrix-core kernel, whose work
    list gives the kept first keys an entry of their own: two sequences side by side, in portions that start behind the
    kept keys, with the same loud keys as above."""
    from mini_engine_amd.ops import kernels as K

    dtype, base, eps, scale, bs = torch.bfloat16, 500.0, 1e-5, 0.3, 16
    g = torch.Generator().manual_seed(nh * 100 + d)
    lens = [330, 205]
    u = torch.randn(d, generator=g)
    seqs, wants = [], []
    for L in lens:
        qkv = torch.randn(L, (nh + 2 * nkv) * d, generator=g) * 0.5
        for j in (0, max(keep - 1, 0), keep, 63, 64, 150, L - size, L - size - 1, L - 2):
            if 0 <= j < L:
                qkv[j, nh * d + (j % nkv) * d : nh * d + (j % nkv + 1) * d] += 3.0 * u
        qkv[:, : nh * d] += 0.7 * u.repeat(nh)
        qkv = qkv.to(dtype)
        seqs.append(qkv)
        wants.append(plain_attention_rows(qkv.float(), 0, nh, nkv, d, d, None, None, eps, rd, base, pairing, True, scale, size, keep))
    pages = [-(-L // bs) for L in lens]
    order = torch.randperm(sum(pages) + 2, generator=g).to(torch.int32)
    table = torch.full((2, max(pages)), int(order[-1]), dtype=torch.int32)
    table[0, : pages[0]] = order[: pages[0]]
    table[1, : pages[1]] = order[pages[0] : pages[0] + pages[1]]
    table = table.cuda()
    k_cache = torch.zeros(sum(pages) + 2, nkv, bs, d, dtype=dtype, device="cuda")
    v_cache = torch.zeros(sum(pages) + 2, nkv, d, bs, dtype=dtype, device="cuda")
    rope, vt = angle_table(rd, base, 512), angle_table(d, base, 512)
    code = 0 if pairing == "halves" else 1
    got = [[], []]
    for cuts in ([(0, 130), (0, 5)], [(130, 331 - 1), (5, 205)]):
        qlens = [hi - lo for lo, hi in cuts]
        starts = [lo for lo, _ in cuts]
        pos = torch.cat([torch.arange(lo, hi) for lo, hi in cuts]).to(torch.int32).cuda()
        item = torch.cat([torch.full((n,), i) for i, n in enumerate(qlens)]).to(torch.int32).cuda()
        item_start = torch.tensor([0, qlens[0], sum(qlens)], dtype=torch.int32).cuda()
        rows = torch.cat([seqs[i][lo:hi] for i, (lo, hi) in enumerate(cuts)]).cuda().contiguous()
        # (the values go to their pages a segment of 16 slots at a time)
        q = K.qkv_rotate_scatter(rows, None, None, rope, code, vt, code, pos, item, table, k_cache, v_cache, nh, nkv, d, d, eps,
                                 item_start=item_start, starts=starts, qlens=qlens)
        out = K.attention_prefill_bf16(q, k_cache, v_cache, pos, item_start, qlens, table, scale, size, starts=starts,
                                       keep_first=keep)
        K.unturn_rows(out, vt, code, pos, nh)
        got[0].append(out[: qlens[0]].cpu())
        got[1].append(out[qlens[0] :].cpu())
        # the kernel that takes every size, on the same pages: the two differ by the rounding of the weights alone
        same = K.attention_general(q, k_cache, v_cache, pos, item, table, scale, size, keep_first=keep, unturn=vt, un_pairing=code)
        assert rel_err(out, same) < 2e-2
    # one new token per item over the same pages: the split-context kernel deals the kept keys' tiles to its splits too
    for ends in ((330, 205), (329, 201), (215, 78)):
        pos = torch.tensor([e - 1 for e in ends], dtype=torch.int32).cuda()
        item = torch.tensor([0, 1], dtype=torch.int32).cuda()
        rows = torch.stack([seqs[i][e - 1] for i, e in enumerate(ends)]).cuda().contiguous()
        q = K.qkv_rotate_scatter(rows, None, None, rope, code, vt, code, pos, item, table, k_cache, v_cache, nh, nkv, d, d, eps)
        ctx = torch.tensor(list(ends), dtype=torch.int32).cuda()
        out = K.attention_decode_bf16(q, k_cache, v_cache, ctx, table, scale, size, table.shape[1] * bs, keep_first=keep)
        K.unturn_rows(out, vt, code, pos, nh)
        same = K.attention_general(q, k_cache, v_cache, pos, item, table, scale, size, keep_first=keep, unturn=vt, un_pairing=code)
        assert rel_err(out, same) < 2e-2
        for i, e in enumerate(ends):
            assert rel_err(out[i : i + 1], wants[i][e - 1 : e]) < 8e-2
    for i in range(2):
        # (scores this loud feel the rounding of the turned q and k: both kernels are up to 6% of a row's largest value off)
        assert rel_err(torch.cat(got[i]), wants[i]) < 8e-2
    missed = plain_attention_rows(seqs[0].float(), 0, nh, nkv, d, d, None, None, eps, rd, base, pairing, True, scale, size, 0)
    assert rel_err(missed, wants[0]) > 0.1  # without the kept keys the longer sequence's rows are somewhere else


# ------------------------------------------------------------------------------------------ decay state
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads,d,dv,rd,pairing,act,norm_kind,gate", [
    (3, 32, 16, 16, "halves", "none", "per_head", "silu"),
    (2, 16, 24, 0, "halves", "silu", "all_heads", "sigmoid"),
    (5, 40, 12, 20, "interleaved", "none", "per_head", "sigmoid"),
    (1, 72, 136, 0, "halves", "silu", "all_heads", "silu"),
    (2, 130, 70, 130, "halves", "none", "all_heads", "silu"),
])
def test_decay_state_kernels_in_portions_and_beside_other_items(heads, d, dv, rd, pairing, act, norm_kind, gate, dtype):
    """Three sequences of unequal length walk through the kernels in steps that hold portions of some beside single
    tokens of others, in slots that are not in order; a fourth then takes over a used slot. One head decays so slowly
    that a large first key is still felt hundreds of tokens later."""
    from mini_engine_amd.ops import kernels as K
    from mini_engine_amd.parts.decay_state import GATE_ACTIVATIONS, INPUT_ACTIVATIONS, OUTPUT_NORMS

    g = torch.Generator().manual_seed(heads * 100 + d)
    decay = [0.9995, 0.6, 0.97, 1.0, 0.0][:heads]
    lens = {"a": 420, "b": 37, "c": 150, "d": 33}
    cols = 2 * heads * (d + dv)
    base, eps, key_scale = 1000.0, 1e-5, d ** -0.5
    proj = {r: (torch.randn(n, cols, generator=g) * 0.7).to(dtype) for r, n in lens.items()}
    proj["a"][0, heads * d : 2 * heads * d] *= 6.0  # a first key that a slow decay carries far
    norm_w = (1.0 + 0.2 * torch.randn(heads * dv, generator=g)) if norm_kind == "all_heads" else None

    def plain_rows(pr):
        n = pr.shape[0]
        x = pr.float().to(F64)
        f = plain.silu if act == "silu" else (lambda z: z)
        q, k = f(x[:, : heads * d]).reshape(n, heads, d), f(x[:, heads * d : 2 * heads * d]).reshape(n, heads, d)
        v = f(x[:, 2 * heads * d : 2 * heads * d + heads * dv]).reshape(n, heads, dv)
        gt = x[:, 2 * heads * d + heads * dv :]
        p = torch.arange(n)
        if rd:
            q, k = plain.rotate_pairs(q, p, rd, base, pairing), plain.rotate_pairs(k, p, rd, base, pairing)
        o, _ = plain.decayed_state_scan(q, k * key_scale, v, decay, None)
        o = plain.unit_rms(o, eps).reshape(n, -1) if norm_kind == "per_head" else plain.unit_rms(o.reshape(n, -1), eps) * norm_w.to(F64)
        return o * (plain.silu(gt) if gate == "silu" else torch.sigmoid(gt))

    want = {r: plain_rows(pr) for r, pr in proj.items()}
    hi = torch.tensor(decay, dtype=F64).float()
    lo = (torch.tensor(decay, dtype=F64) - hi.to(F64)).float()
    dec = torch.stack((hi, lo)).cuda()
    rope = angle_table(rd, base, 512) if rd else None
    state = torch.full((6, heads, d, dv), 7.0, device="cuda")  # stale values: a fresh request's slot is zeroed by the caller
    slot = {"a": 4, "b": 1, "c": 2}
    fed = {r: 0 for r in lens}
    got = {r: [] for r in lens}
    # (steps whose longest portion has more than two chunks of 64 tokens walk all chunks side by side: the first two)
    plan = [[("a", 300), ("b", 1), ("c", 2)], [("b", 30), ("a", 1), ("c", 147)], [("a", 119), ("c", 1), ("b", 6)], [("d", 33)]]
    for step in plan:
        if step[0][0] == "d":
            slot["d"] = slot.pop("b")  # b is over: its slot is used again
        rows, pos, starts, slots = [], [], [0], []
        for r, n in step:
            if fed[r] == 0:
                state[slot[r]].zero_()
            rows.append(proj[r][fed[r] : fed[r] + n])
            pos += list(range(fed[r], fed[r] + n))
            starts.append(starts[-1] + n)
            slots.append(slot[r])
        out = K.decay_state(torch.cat(rows).cuda().contiguous(), rope, 0 if pairing == "halves" else 1,
                            torch.tensor(pos, dtype=torch.int32).cuda(), dec, None if norm_w is None else norm_w.cuda(), state,
                            torch.tensor(starts, dtype=torch.int32).cuda(), torch.tensor(slots, dtype=torch.int32).cuda(), heads, d,
                            dv, INPUT_ACTIVATIONS[act], key_scale, OUTPUT_NORMS[norm_kind], GATE_ACTIVATIONS[gate], eps,
                            longest_item=max(n for _, n in step))
        at = 0
        for r, n in step:
            got[r].append(out[at : at + n].cpu())
            fed[r] += n
            at += n
    for r in lens:
        assert fed[r] == lens[r]
        assert rel_err(torch.cat(got[r]), want[r]) < TOL[dtype] * 2, r


# --------------------------------------------------------------------------------- models through the engine
def assert_logits_close(got, want, dtype, what):
    """float32: the bound of the other models' tests. bfloat16, row by row: no element further off than 4% of the row's
    largest logit and a root-mean-square error of at most 3% of the row's root mean square: these models round the
    projections of q, k, v and the gate, the normed outputs and three products per layer, and their random weights give
    rows whose largest logit is two to three times their root mean square. One row in a hundred (at least one) may miss
    that: a head's output is divided by its own root mean square, so where q . k nearly vanishes (the first token of a
    sequence, whose state is k v^T alone: o = (q . k) v) a rounding decides the sign of what the norm hands on."""
    if dtype == "float32":
        return th.assert_logits_close(got, want, dtype, what)
    err = (got - want).abs()
    bad = (err.max(dim=-1).values > 0.04 * want.abs().max(dim=-1).values) | (
        err.pow(2).mean(dim=-1).sqrt() > 0.03 * want.pow(2).mean(dim=-1).sqrt())
    if int(bad.sum()) > max(1, got.shape[0] // 100):
        pos = int(bad.nonzero()[0])
        raise AssertionError(f"{what}: {int(bad.sum())} rows off, the first at {pos} of {got.shape[0]}: error {err[pos].max().item():.3e}, the row's "
                             f"largest logit {want[pos].abs().max().item():.3e}, its root mean square "
                             f"{want[pos].pow(2).mean().sqrt().item():.3e}, the error's {err[pos].pow(2).mean().sqrt().item():.3e}")


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    return {n: gh.write_folder(str(tmp_path_factory.mktemp(f"gonurax_{n}")), cfg, seed=31 + i)
            for i, (n, cfg) in enumerate(gh.configs().items())}


def requests_for(cfg, seed, lengths=(1, 23, 97, 150, 61)):
    g = torch.Generator().manual_seed(seed)
    return {f"r{i}": torch.randint(0, cfg["vocab"], (n,), generator=g).tolist() for i, n in enumerate(lengths)}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["P", "Q", "R", "S", "T"])
def test_every_way_of_cutting_gives_the_plain_logits(folders, name, dtype):
    """Whole prompts; most of a prompt and its tail token by token (replayed graphs); portions down to two tokens; up
    to four live requests in a pool and in slots that are used again: all against the plain implementation."""
    from mini_engine_amd.engine.trace import TraceSession, build_session

    cfg = gh.configs()[name]
    reqs = requests_for(cfg, seed=7)
    want = gh.plain_logits(cfg, gh.read_weights(folders[name]), reqs)
    bs = gh.BLOCK_SIZES[name]
    biggest = max(th.round_up(len(t)) for t in reqs.values())
    for build, max_tokens, live in ((th.whole, biggest, 4), (lambda r: th.tail_one_by_one(r, tail=40), biggest, 4),
                                    (th.portions, biggest, 4), (lambda r: th.mixed(r, 448, seed=3, max_live=3), 448, 3)):
        session = TraceSession(build_session(folders[name], dtype, max_tokens, block_size=bs, max_live=live))
        steps = build(reqs)
        got = th.collect(steps, th.replay_in_process(session, steps))
        for rid in reqs:
            assert_logits_close(got[rid], want[rid], dtype, f"{name} {dtype} {rid}")
        if live == 3:  # five requests went through three slots
            assert session.engine.runner.num_state_slots == 3
    assert len({int(t) for t in want["r3"].argmax(-1)}) > 10


def test_float32_logits_do_not_depend_on_the_cut_or_the_company(folders):
    """In float32 the same position gives the same logits to a few units in the last place however it was reached."""
    from mini_engine_amd.engine.trace import TraceSession, build_session

    cfg = gh.configs()["P"]
    reqs = requests_for(cfg, seed=9, lengths=(130, 45, 77))
    outs = []
    for build in (th.whole, th.portions, lambda r: th.mixed(r, 320, seed=5, max_live=3)):
        session = TraceSession(build_session(folders["P"], "float32", 320, block_size=16, max_live=3))
        steps = build(reqs)
        outs.append(th.collect(steps, th.replay_in_process(session, steps)))
    for rid in reqs:
        for other in outs[1:]:
            assert rel_err(other[rid], outs[0][rid]) < 2e-5


def test_long_decoding_from_a_short_prompt(folders):
    """Three tokens of prompt, then 300 tokens one by one: past every window, far beyond the kept first keys, through
    pages that the window gives back."""
    from mini_engine_amd.engine.trace import TraceSession, build_session

    cfg = gh.configs()["R"]
    reqs = requests_for(cfg, seed=13, lengths=(303,))
    want = gh.plain_logits(cfg, gh.read_weights(folders["R"]), reqs)
    session = TraceSession(build_session(folders["R"], "float32", 320, block_size=8, max_live=2))
    steps = th.tail_one_by_one(reqs, tail=300)
    got = th.collect(steps, th.replay_in_process(session, steps))
    th.assert_logits_close(got["r0"], want["r0"], "float32", "long decoding")
    assert session.engine.runner.graph_replays >= 299


@pytest.mark.parametrize("name", ["P", "Q"])
def test_greedy_generation_through_the_scheduler(folders, name):
    """Unequal prompts through ``LLMEngine.generate``: a token budget that cuts prompts into portions, a pool that
    fits two of the three requests at a time. float32 picks the plain implementation's tokens."""
    from mini_engine_amd import EngineConfig, LLMEngine, SamplingParams

    cfg = gh.configs()[name]
    w = gh.read_weights(folders[name])
    prompts = list(requests_for(cfg, seed=17, lengths=(40, 9, 75)).values())
    new = 12
    want = []
    for p in prompts:
        toks = list(p)
        for _ in range(new):
            toks.append(int(plain.forward(cfg, w, toks)[0][-1].argmax()))
        want.append(toks[len(p):])
    bs = gh.BLOCK_SIZES[name]
    engine = LLMEngine.from_pretrained(folders[name], EngineConfig(dtype="float32", block_size=bs, num_blocks=160 // bs,
                                                                   max_num_seqs=3, max_num_batched_tokens=32, max_model_len=128,
                                                                   enable_prefix_caching=False))
    got = engine.generate(prompts, SamplingParams(max_tokens=new, ignore_eos=True))
    assert got == want
