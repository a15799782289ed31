"""Zokepel on the GPU against the plain implementation, in 32-bit and in bfloat16: every mixer kind alone; whole
prompts; most of a prompt in one step and its last tokens one by one; portions of changing size down to two tokens;
mixed batches in a pool so small that pages and slots are used again; long decoding; the first tokens; kernels with
inputs made so that one far key, one distance bucket or one old write stands out; generation through the scheduler,
the replay program and the command line."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

from tests import helpers as H
from tests import zokepel_helpers as ZH
from tests.plain import zokepel_plain as Z
from tests.test_engine_gpu import mixed_schedule, portions, run_steps

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
DTYPES = ["float32", "bfloat16"]
NAMES = ["P", "Q", "R", "S"]
LENGTHS = {"P": 150, "Q": 210, "R": 120, "S": 330}
# bfloat16 against the plain implementation, per row: relative L2 error of the logits (1.5 x the worst row measured
# for these models; a wrong bucket, a lost state or a missing scale shows as tens of percent)
BF16_REL_L2 = 0.06
# A sequence's first token gets more: every state is empty there, so each recurrent head's read-out is one outer
# product, (k . q) u for the delta rule and (sum_i bonus_i k_i r_i) v for the time mixing, and dividing it by its root
# mean square leaves a direction times a factor that depends on that one inner product and the norm's eps alone:
# where the products' terms cancel, their bfloat16 rounding is amplified (measured up to 8.4 % for one sequence,
# the same in every batching; 32-bit is not affected).
BF16_REL_L2_FIRST = 0.15
# The same amplification happens at single later tokens where a head's read-out nearly cancels before it is divided
# by its root mean square (random weights; measured: one row in some sequences at 10 % between neighbours at 1 %, bit
# for bit the same alone, in portions, decoded and beside other requests).  One row in fifty may therefore exceed
# the bound, none twice the first token's.
BF16_ROWS_OVER = 0.02
BF16_REL_L2_WORST = 0.3


@pytest.fixture(scope="module")
def dirs(tmp_path_factory):
    root = tmp_path_factory.mktemp("zokepel")
    out = {n: ZH.make_model_dir(str(root), ZH.MODELS[n], n, seed=31 + i) for i, n in enumerate(NAMES)}
    for kind in ("delta", "channel_delta", "parallel"):
        out[kind] = ZH.make_model_dir(str(root), ZH.single_layer(kind), kind, seed=5)
    return out


def make_engine(model_dir, dtype, **kw):
    from gibbs_amd import Engine
    kw.setdefault("max_tokens", 2048)
    kw.setdefault("max_requests", 4)
    return Engine(model_dir, dtype=dtype, **kw)


def close(got, want, dtype, what, places=None):
    """`places`: the rows' positions in their sequence (position 0 has a bound of its own in bfloat16)."""
    got, want = np.asarray(got, dtype=np.float64), np.asarray(want, dtype=np.float64)
    assert got.shape == want.shape, (what, got.shape, want.shape)
    if dtype == "float32":
        err = np.abs(got - want).max(-1)
        bound = 2e-5 * np.abs(want).max()
        assert err.max() <= bound, f"{what}: max error {err.max():.3e} at row {int(err.argmax())} above {bound:.3e}; first bad row {int((err > bound).argmax())}"
        return
    rel = np.sqrt(((got - want) ** 2).sum(-1) / (want ** 2).sum(-1))
    bound = np.full(rel.shape, BF16_REL_L2)
    if places is not None:
        bound[np.asarray(places) == 0] = BF16_REL_L2_FIRST
    over = int((rel > bound).sum())
    assert over <= max(1, int(BF16_ROWS_OVER * rel.size)) and rel.max() <= BF16_REL_L2_WORST, (
        f"{what}: {over} of {rel.size} rows over their bound, relative L2 error {rel.max():.3e} at row {int(rel.argmax())}; "
        f"first bad row {int((rel > bound).argmax())}")


def check(model_dir, seqs, got, dtype, what):
    for rid, ids in seqs.items():
        want = ZH.plain_logits(model_dir, ids)
        places = sorted(p for r, p in got if r == rid)
        assert places, f"{what}: no logits for {rid}"
        close(np.stack([got[(rid, p)] for p in places]), want[places], dtype, f"{what} request {rid}", places)


def vocab_of(model_dir):
    with open(os.path.join(model_dir, "config.json")) as f:
        return json.load(f)["vocab"]


# ----------------------------------------------------------------------------------------------- whole models
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("kind", ["delta", "channel_delta", "parallel"])
def test_each_mixer_alone(dirs, kind, dtype):
    d = dirs[kind]
    ids = ZH.tokens(1, 90, vocab_of(d))
    eng = make_engine(d, dtype)
    got = run_steps(eng, [([("r", ids[:61], list(range(61)))], []), ([("r", ids[61:], list(range(29)))], ["r"])])
    check(d, {"r": ids}, got, dtype, f"{kind} alone {dtype}")
    assert eng.cache.free_slots() == 4


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", NAMES)
def test_whole(dirs, name, dtype):
    d = dirs[name]
    ids = ZH.tokens(2, LENGTHS[name], vocab_of(d))
    eng = make_engine(d, dtype)
    got = run_steps(eng, [([("r", ids, list(range(len(ids))))], ["r"])])
    check(d, {"r": ids}, got, dtype, f"whole {name} {dtype}")
    eng.cache.check()
    assert all(eng.cache.free_pages(g) == eng.cache.pools[g].num_pages for g in range(eng.cache.n_groups))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", NAMES)
def test_bulk_then_last_32_one_by_one(dirs, name, dtype):
    d = dirs[name]
    ids = ZH.tokens(3, LENGTHS[name], vocab_of(d))
    cut = len(ids) - 32
    steps = [([("r", ids[:cut], list(range(cut)))], [])] + [([("r", [t], [0])], []) for t in ids[cut:]]
    got = run_steps(make_engine(d, dtype), steps)
    check(d, {"r": ids}, got, dtype, f"bulk+tail {name} {dtype}")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", NAMES)
def test_changing_portions_down_to_two_tokens(dirs, name, dtype):
    d = dirs[name]
    ids = ZH.tokens(4, LENGTHS[name], vocab_of(d))
    cuts = portions(len(ids) - 9, [7, 2, 13, 3, 2, 64, 5, 2, 17, 1, 2]) + [(len(ids) - 9 + i, len(ids) - 8 + i) for i in range(9)]
    steps = [([("r", ids[a:b], list(range(b - a)))], []) for a, b in cuts]
    got = run_steps(make_engine(d, dtype), steps)
    check(d, {"r": ids}, got, dtype, f"portions {name} {dtype}")


@pytest.mark.parametrize("name", NAMES)
def test_cutting_changes_no_bit_in_32_bit(dirs, name):
    """The recurrences add in one order per token and the products in ascending k, so 32-bit logits do not depend on how
    the prompt was cut or on what else was in the batch."""
    d = dirs[name]
    ids = ZH.tokens(5, 77, vocab_of(d))
    other = ZH.tokens(6, 41, vocab_of(d))
    whole = run_steps(make_engine(d, "float32"), [([("r", ids, list(range(77)))], [])])
    eng = make_engine(d, "float32")
    steps = [([("o", other[:20], []), ("r", ids[:2], [0, 1])], []), ([("r", ids[2:50], list(range(48))), ("o", other[20:21], [])], []),
             ([("o", other[21:], []), ("r", ids[50:51], [0])], ["o"]), ([("r", ids[51:], list(range(26)))], [])]
    cut = run_steps(eng, steps)
    for p in range(77):
        assert np.abs(cut[("r", p)] - whole[("r", p)]).max() <= 2e-6 * np.abs(whole[("r", p)]).max(), p


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", NAMES)
def test_mixed_batches_with_pages_and_slots_used_again(dirs, name, dtype):
    d = dirs[name]
    rng = np.random.default_rng(7)
    seqs = {f"q{i}": ZH.tokens(100 + i, int(n), vocab_of(d)) for i, n in enumerate([70, 45, 90, 33, 64, 81, 50, 3, 2])}
    steps = mixed_schedule(seqs, rng)
    assert max(len(e) for e, _ in steps) >= 3
    assert any(len(t) > 1 for e, _ in steps for _, t, _ in e) and any(len(t) == 1 for e, _ in steps for _, t, _ in e)
    eng = make_engine(d, dtype, max_tokens=384, max_requests=4, page_size=16)
    assert sum(-(-len(s) // 16) for s in seqs.values()) > eng.cache.pools[0].num_pages, "the pool must be too small to avoid reuse"
    got = run_steps(eng, steps)
    check(d, seqs, got, dtype, f"mixed {name} {dtype}")
    eng.cache.check()
    assert eng.cache.free_slots() == 4 and all(eng.cache.free_pages(g) == eng.cache.pools[g].num_pages for g in range(eng.cache.n_groups))


@pytest.mark.parametrize("dtype", DTYPES)
def test_long_decoding(dirs, dtype):
    d = dirs["P"]
    ids = ZH.tokens(9, 330, vocab_of(d))
    steps = [([("r", ids[:5], list(range(5)))], [])] + [([("r", [t], [0])], []) for t in ids[5:]]
    got = run_steps(make_engine(d, dtype), steps)
    check(d, {"r": ids}, got, dtype, f"long decoding {dtype}")


@pytest.mark.parametrize("dtype", DTYPES)
def test_first_tokens(dirs, dtype):
    """Sequences of one, two and three tokens, alone and side by side: zeros before the start in the convolutions
    and the shift, empty states, a single visible key."""
    d = dirs["P"]
    seqs = {f"s{n}": ZH.tokens(20 + n, n, vocab_of(d)) for n in (1, 2, 3, 5)}
    got = run_steps(make_engine(d, dtype), [([(r, ids, list(range(len(ids)))) for r, ids in seqs.items()], list(seqs))])
    check(d, seqs, got, dtype, f"first tokens together {dtype}")
    eng = make_engine(d, dtype)
    for r, ids in seqs.items():
        got = run_steps(eng, [([(r, ids[:1], [0])], [])] + [([(r, [t], [0])], []) for t in ids[1:]] + [([], [r])][:0])
        check(d, {r: ids}, got, dtype, f"first tokens one by one {dtype}")
        eng.release(r)


# ----------------------------------------------------------------------------------------------- kernels with made-up inputs
def paged(keys, values, page_size, n_pages, order):
    """Key and value pages [page, 1, slot, size] of one request whose logical pages lie at `order` in the pool."""
    T = keys.shape[0]
    kp = torch.zeros((n_pages, 1, page_size, keys.shape[1]), dtype=keys.dtype, device="cuda")
    vp = torch.zeros((n_pages, 1, page_size, values.shape[1]), dtype=keys.dtype, device="cuda")
    for t in range(T):
        kp[order[t // page_size], 0, t % page_size] = keys[t]
        vp[order[t // page_size], 0, t % page_size] = values[t]
    return kp, vp


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_attention_far_key_and_every_distance_of_the_bias(dtype):
    """One query head over 700 keys in pages of 16 scattered over the pool, values of a size of their own.  A single key
    far back is made to dominate (its score stands out by 12), at a page's border and in the middle of one; then the
    bias alone decides: a table whose row for one distance stands out, for distances just inside and just beyond the
    table's end (all longer distances share the last row)."""
    from gibbs_amd import ops
    rng = np.random.default_rng(0)
    T, hd, vd, ps = 700, 24, 40, 16
    n_pages = 64
    order = rng.permutation(n_pages)[:-(-T // ps)].tolist()
    keys = torch.tensor(rng.normal(size=(T, hd)) * 0.1, dtype=dtype, device="cuda")
    values = torch.tensor(rng.normal(size=(T, vd)), dtype=dtype, device="cuda")
    table = torch.tensor([order], dtype=torch.int32, device="cuda")
    rows = torch.tensor([T - 1, T - 2, 300], dtype=torch.int32, device="cuda")
    row_req = torch.zeros(3, dtype=torch.int32, device="cuda")
    q = torch.tensor(rng.normal(size=(3, hd)) * 0.1, dtype=dtype, device="cuda")
    flat = torch.zeros((50, 1), dtype=torch.float32, device="cuda")
    for far in (15, 16, 17, 200, 0):
        k2 = keys.clone()
        k2[far] = (q[0].float() / q[0].float().norm() ** 2 * 12.0).to(dtype)     # q0 . k = 12
        kp, vp = paged(k2, values, ps, n_pages, order)
        out = ops.attention_plain(q, 3, 1, 1, hd, kp, vp, table, 1, rows, row_req, 1.0, bias=flat).float().cpu().numpy()
        s = (q.float() @ k2.float().T).cpu().numpy()
        for i, p in enumerate(rows.tolist()):
            w = np.exp(s[i, :p + 1] - s[i, :p + 1].max())
            want = (w / w.sum()) @ values.float().cpu().numpy()[:p + 1]
            assert np.abs(out[i] - want).max() <= (2e-5 if dtype == torch.float32 else 2e-2), (far, i)
        assert np.abs(out[0] - values[far].float().cpu().numpy()).max() < 0.05, f"the far key {far} does not dominate"
    kp, vp = paged(keys * 0, values, ps, n_pages, order)
    for length, hot in ((50, 48), (50, 49), (50, 7), (3, 2), (3, 1)):
        bias = torch.zeros((length, 1), dtype=torch.float32, device="cuda")
        bias[hot, 0] = 14.0
        out = ops.attention_plain(q, 3, 1, 1, hd, kp, vp, table, 1, rows, row_req, 1.0, bias=bias).float().cpu().numpy()
        for i, p in enumerate(rows.tolist()):
            dist = np.minimum(p - np.arange(p + 1), length - 1)
            w = np.exp(np.where(dist == hot, 14.0, 0.0))
            want = (w / w.sum()) @ values.float().cpu().numpy()[:p + 1]
            assert np.abs(out[i] - want).max() <= (2e-5 if dtype == torch.float32 else 2e-2), (length, hot, i)


def test_unit_norm_temperature_and_cache_write():
    from gibbs_amd import ops
    rng = np.random.default_rng(1)
    nh, nkv, hd, vd, ps = 4, 2, 24, 40, 16
    pos = torch.tensor([0, 7, 8, 15, 16, 31, 250], dtype=torch.int32, device="cuda")
    n = pos.numel()
    rows = torch.tensor(rng.normal(size=(n, (nh + nkv) * hd + nkv * vd)), dtype=torch.float32, device="cuda")
    before = rows.cpu().numpy().copy()
    kp = torch.zeros((20, nkv, ps, hd), dtype=torch.float32, device="cuda")
    vp = torch.zeros((20, nkv, ps, vd), dtype=torch.float32, device="cuda")
    table = torch.arange(19, -1, -1, dtype=torch.int32, device="cuda").view(1, 20).contiguous()
    ops.qk_unit_kv(rows, nh, nkv, hd, vd, kpages=kp, vpages=vp, table=table, pos=pos, row_req=torch.zeros(n, dtype=torch.int32, device="cuda"),
                   eps=1e-5, unit=True, temp_coef=0.7, temp_every=8)
    after = rows.cpu().numpy()
    for i, p in enumerate(pos.tolist()):
        heads = before[i, :(nh + nkv) * hd].reshape(nh + nkv, hd)
        unit = heads / np.sqrt((heads ** 2).mean(-1, keepdims=True) + 1e-5)
        unit[:nh] *= 1.0 + 0.7 * np.log((p + 1) // 8 + 1.0)             # positions 7 and 8, 15 and 16 lie on both sides of a step
        assert np.allclose(after[i, :(nh + nkv) * hd].reshape(nh + nkv, hd), unit, rtol=2e-6, atol=1e-6)
        page = 19 - p // ps
        assert np.allclose(kp[page, :, p % ps].cpu().numpy(), unit[nh:], rtol=2e-6, atol=1e-6)
        assert np.array_equal(vp[page, :, p % ps].cpu().numpy().reshape(-1), before[i, (nh + nkv) * hd:])


def test_heads_of_unequal_sizes_are_stored_padded_in_bfloat16_only(dirs):
    """Keys of 24 and values of 40 (model P) run as heads of 48 in a bfloat16 engine (zeros behind each head's channels, in
    the projections and in the pages: what the matrix-core attention kernels take) and at their own sizes in 32-bit; the
    logits of both are held against the plain implementation by the tests above."""
    for dtype, sizes in (("bfloat16", (48, 48)), ("float32", (24, 40))):
        eng = make_engine(dirs["P"], dtype)
        left = eng.model.blocks[1].left
        assert left.stored_dims() == sizes and (left.head_dim, left.v_head_dim) == (24, 40)
        group = eng.cache.group_needs.index(left.cache_need())
        assert eng.device_cache.kpages[group].shape[-1] == sizes[0] and eng.device_cache.vpages[group].shape[-1] == sizes[1]
        assert left.w_qkv.shape[0] == 6 * sizes[0] + 3 * sizes[0] + 3 * sizes[1] and left.w_out.shape[1] == 6 * sizes[1]
        if dtype == "bfloat16":
            q = left.w_qkv[:6 * 48].view(6, 48, -1)
            assert float(q[:, 24:].abs().max()) == 0.0 and float(left.w_out.view(-1, 6, 48)[:, :, 40:].abs().max()) == 0.0


def test_unit_norm_of_padded_heads_divides_by_the_true_size():
    from gibbs_amd import ops
    rng = np.random.default_rng(8)
    nh, nkv, true, pad = 2, 1, 24, 32
    rows = np.zeros((3, (nh + 2 * nkv) * pad), dtype=np.float32)
    rows.reshape(3, nh + 2 * nkv, pad)[:, :, :true] = rng.normal(size=(3, nh + 2 * nkv, true))
    dev = torch.tensor(rows, device="cuda")
    pos = torch.tensor([0, 1, 2], dtype=torch.int32, device="cuda")
    ops.qk_unit_kv(dev, nh, nkv, pad, pad, kpages=None, vpages=None, table=None, pos=pos, row_req=torch.zeros(3, dtype=torch.int32, device="cuda"),
                   eps=1e-6, unit=True, norm_dim=true)
    heads = rows.reshape(3, nh + 2 * nkv, pad)[:, :nh + nkv]
    want = heads / np.sqrt((heads[:, :, :true] ** 2).mean(-1, keepdims=True) + 1e-6)
    got = dev.cpu().numpy().reshape(3, nh + 2 * nkv, pad)[:, :nh + nkv]
    assert np.allclose(got, want, rtol=2e-6, atol=1e-6) and np.abs(got[:, :, true:]).max() == 0.0


@pytest.mark.parametrize("per_channel", [False, True])
def test_delta_rule_keeps_an_old_write_through_portions_and_slots(per_channel):
    """A value written at the first token with a key of its own is read back 500 tokens later (no decay on that key's
    channel, random writes on the others in between), whole, in portions of 1, 2, 7 and 64 tokens, and in a slot that
    another request used before; the kernel's result equals the plain rule's."""
    from gibbs_amd import ops
    rng = np.random.default_rng(2)
    T, H, G, D, V = 501, 4, 2, 20, 24
    k = rng.normal(size=(T, G, D)); k[:, :, 0] = 0; k[0] = 0; k[0, :, 0] = 1
    k /= np.linalg.norm(k, axis=-1, keepdims=True)
    q = rng.normal(size=(T, G, D)) * 0.2; q[-1] = 0; q[-1, :, 0] = 1
    v = rng.normal(size=(T, H, V))
    beta = rng.uniform(0.2, 1.0, size=(T, H)); beta[0] = 1
    decay = rng.uniform(0.8, 1.0, size=(T, H, D) if per_channel else (T, H))
    if per_channel:
        decay[:, :, 0] = 1
    want = np.stack([Z.delta_rule(q[:, h // 2], k[:, h // 2], v[:, h], beta[:, h], decay[:, h]) for h in range(H)], axis=1)
    if per_channel:
        assert np.allclose(want[-1], v[0]), "the plain rule itself must recall the first write"
    dev = lambda a: torch.tensor(a.reshape(T, -1), dtype=torch.float32, device="cuda")
    dq, dk, dv, db, dd = dev(q), dev(k), dev(v), dev(beta), dev(decay)
    state = torch.zeros((3, H, D, V), dtype=torch.float32, device="cuda")
    for slot, sizes in ((1, [T]), (2, [1, 2, 7, 64, 1, 1, 300, 2]), (1, [64, 63, 2])):
        state[slot].zero_()                       # (a slot is cleared when a request takes it)
        at, outs, i = 0, [], 0
        while at < T:
            n = min(sizes[i % len(sizes)], T - at)
            cu = torch.tensor([0, n], dtype=torch.int32, device="cuda")
            outs.append(ops.delta_rule(dq[at:at + n].contiguous(), dk[at:at + n].contiguous(), dv[at:at + n].contiguous(),
                                       db[at:at + n].contiguous(), dd[at:at + n].contiguous(), state, cu,
                                       torch.tensor([slot], dtype=torch.int32, device="cuda"), H, G))
            at += n; i += 1
        got = torch.cat(outs).cpu().numpy().reshape(T, H, V)
        assert np.abs(got - want).max() <= 2e-5 * np.abs(want).max(), (slot, sizes)


def test_decayed_outer_rule_two_requests_side_by_side():
    from gibbs_amd import ops
    rng = np.random.default_rng(3)
    H, D = 3, 12
    lens = [37, 5]
    r, k, v = (rng.normal(size=(sum(lens), H, D)) * 0.5 for _ in range(3))
    w = rng.uniform(0.5, 1.0, size=(sum(lens), H, D)); w[:, :, 1] = 1.0          # channel 1 never forgets
    bonus = rng.normal(size=(H, D))
    want = np.zeros((sum(lens), H, D))
    at = 0
    for n in lens:
        for h in range(H):
            S = np.zeros((D, D))
            for t in range(at, at + n):
                kv = np.outer(k[t, h], v[t, h])
                want[t, h] = (S + bonus[h][:, None] * kv).T @ r[t, h]
                S = w[t, h][:, None] * S + kv
        at += n
    dev = lambda a: torch.tensor(a.reshape(a.shape[0], -1), dtype=torch.float32, device="cuda")
    state = torch.zeros((4, H, D, D), dtype=torch.float32, device="cuda")
    slot = torch.tensor([3, 0], dtype=torch.int32, device="cuda")
    dr, dk, dv, dw = dev(r), dev(k), dev(v), dev(w)
    # first 30 + 2 tokens in one call, the rest in another (rows of the two requests side by side)
    idx1 = list(range(30)) + [37, 38]
    idx2 = list(range(30, 37)) + [39, 40, 41]
    outs = {}
    for idx, cu in ((idx1, [0, 30, 32]), (idx2, [0, 7, 10])):
        sel = torch.tensor(idx, device="cuda")
        o = ops.decayed_outer_rule(dr[sel].contiguous(), dk[sel].contiguous(), dv[sel].contiguous(), dw[sel].contiguous(),
                                   torch.tensor(bonus, dtype=torch.float32, device="cuda"), state,
                                   torch.tensor(cu, dtype=torch.int32, device="cuda"), slot, H)
        for i, t in enumerate(idx):
            outs[t] = o[i].cpu().numpy().reshape(H, D)
    got = np.stack([outs[t] for t in range(sum(lens))])
    assert np.abs(got - want).max() <= 2e-5 * np.abs(want).max()


def test_short_convolution_across_portions_shorter_than_its_taps():
    from gibbs_amd import ops
    rng = np.random.default_rng(4)
    T, C, K = 23, 70, 5
    x = rng.normal(size=(T, C))
    taps = rng.normal(size=(C, K))
    want = Z.silu(Z.causal_conv(x, taps))
    dx = torch.tensor(x, dtype=torch.float32, device="cuda")
    dt = torch.tensor(taps, dtype=torch.float32, device="cuda")
    state = torch.zeros((2, K - 1, C), dtype=torch.float32, device="cuda")
    slot = torch.tensor([1], dtype=torch.int32, device="cuda")
    at, outs = 0, []
    for n in [1, 1, 2, 3, 1, 9, 2, 4]:
        cu = torch.tensor([0, n], dtype=torch.int32, device="cuda")
        outs.append(ops.causal_conv_silu(dx[at:at + n].contiguous(), dt, state, torch.zeros(n, dtype=torch.int32, device="cuda"), cu, slot))
        at += n
    assert at == T
    assert np.abs(torch.cat(outs).cpu().numpy() - want).max() <= 1e-5


# ----------------------------------------------------------------------------------------------- entry points
def plain_greedy(model_dir, prompt, n):
    seq, out = list(prompt), []
    for _ in range(n):
        t = int(np.argmax(ZH.plain_logits(model_dir, seq)[-1]))
        out.append(t); seq.append(t)
    return out


@pytest.mark.parametrize("dtype", DTYPES)
def test_greedy_generation_through_the_scheduler(dirs, dtype):
    """`generate` (scheduler, prompt steps, bursts of captured decode steps) gives the plain implementation's greedy
    tokens; in bfloat16 wherever the plain logits' lead exceeds the precision's error."""
    from gibbs_amd import Engine, generate
    held = 0
    for name, lens in (("P", [7, 13, 2]), ("R", [5])):
        d = dirs[name]
        eng = Engine(d, dtype=dtype, max_tokens=512, max_requests=4)
        prompts = [ZH.tokens(40 + i, n, vocab_of(d)) for i, n in enumerate(lens)]
        outs = generate(eng, prompts, max_tokens=20, temperature=0.0, ignore_eos=True)
        for p, o in zip(prompts, outs):
            assert o.finish_reason == "length" and len(o.tokens) == 20
            if dtype == "float32":
                assert o.tokens == plain_greedy(d, p, 20)
                held += 20
                continue
            logits = ZH.plain_logits(d, list(p) + list(o.tokens))
            for i, t in enumerate(o.tokens):
                row = logits[len(p) - 1 + i]
                best, second = np.sort(row)[[-1, -2]]
                margin = 2 * 0.04 * np.abs(row).max()
                if best - second > margin:
                    held += 1
                    assert t == int(np.argmax(row)), f"token {i}"
                else:
                    assert row[t] >= best - margin, f"token {i}"
        eng.cache.check()
        assert eng.cache.free_slots() == 4
    assert held >= 20


def test_decode_bursts_change_nothing(dirs):
    from gibbs_amd import Engine, Generator, SamplingParams
    d = dirs["Q"]
    prompts = [ZH.tokens(70 + i, n, vocab_of(d)) for i, n in enumerate([9, 21, 5])]
    runs = []
    for burst in (0, 16):
        eng = Engine(d, dtype="float32", max_tokens=1024, max_requests=4)
        gen = Generator(eng, decode_burst=burst, eos_token_ids=())
        rids = [gen.submit(p, SamplingParams(temperature=0.0, max_new_tokens=n), rid=f"r{i}") for i, (p, n) in enumerate(zip(prompts, [37, 20, 9]))]
        res = gen.run()
        runs.append([res[r].tokens for r in rids])
    assert runs[0] == runs[1]
    assert runs[0][0] == plain_greedy(d, prompts[0], 37)


@pytest.mark.parametrize("dtype", DTYPES)
def test_replay_program(dirs, dtype, tmp_path):
    d = dirs["R"]
    ids = ZH.tokens(50, 40, vocab_of(d))
    other = ZH.tokens(51, 9, vocab_of(d))
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": ids[:17], "want": [0, 16]}, {"id": "b", "tokens": other[:2], "want": []}], "end": []},
             {"step": 1, "entries": [{"id": "b", "tokens": other[2:], "want": [6]}], "end": ["b"]},
             {"step": 2, "entries": [{"id": "a", "tokens": ids[17:39], "want": [21]}], "end": []},
             {"step": 3, "entries": [{"id": "a", "tokens": ids[39:], "want": [0]}], "end": ["a"]}]
    out = tmp_path / "out"
    proc = subprocess.run([os.path.join(ROOT, "bin", "trace_run"), "--model", d, "--dtype", dtype, "--out", str(out), "--max-tokens", "128"],
                          input="\n".join(json.dumps(s) for s in steps) + "\n", capture_output=True, text=True, timeout=600)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert [l for l in proc.stdout.splitlines() if l.startswith("done")] == [f"done {i}" for i in range(4)]
    want_a, want_b = ZH.plain_logits(d, ids), ZH.plain_logits(d, other)
    read = lambda i: np.fromfile(out / f"{i}.f32", dtype="<f4").reshape(-1, vocab_of(d))
    close(read(0), want_a[[0, 16]], dtype, "step 0", [0, 16])
    close(read(1), want_b[[8]], dtype, "step 1")
    close(read(2), want_a[[38]], dtype, "step 2")
    close(read(3), want_a[[39]], dtype, "step 3")


def test_command_line(dirs):
    d = dirs["P"]
    prompt = ZH.tokens(60, 6, vocab_of(d))
    proc = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "gibbs"), "--model", d, "--dtype", "float32", "--prompt-ids",
                           ",".join(map(str, prompt)), "--max-tokens", "8", "--temperature", "0", "--ignore-eos"],
                          capture_output=True, text=True, timeout=600)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert "⚡ Prefill: 6 tokens" in proc.stdout and "📈 Roofline:" in proc.stdout
    line = proc.stdout.split("✨ Output:\n")[1].splitlines()[0]
    assert [int(t) for t in line.split()] == plain_greedy(d, prompt, 8)
    proc = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "gibbs"), "--model", d, "--arch-dump"], capture_output=True, text=True, timeout=600)
    dump = json.loads(proc.stdout)
    assert dump["architecture"] == "Zokepel" and dump["unconsumed"] == [] and dump["missing"] == []
    assert dump["derived"]["order"] == [0, 1, 2, 1, 2, 1, 2, 3]
