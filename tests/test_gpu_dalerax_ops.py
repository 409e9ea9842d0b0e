"""Dalerax's mechanisms one by one, each kernel against the plain function of ``plain_dalerax`` (float64), at
sizes of the tests' own: the mixing of a token's input with the input before it, the wkv recurrence, the
router, the sorting of (token, choice) pairs by expert, the experts' grouped product in both of its forms, the
weighted sum back into the rows, and attention's kept first keys and sink with inputs made so that a single key
(or the sink) decides the output."""

import math

import numpy as np
import pytest
import torch

import plain_dalerax as plain

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
DTYPES = [torch.float32, torch.bfloat16]


@pytest.fixture(scope="module")
def ops():
    from flyweight_amd.kernels import ops
    ops.library()
    return ops


def dev(a, dtype=torch.float32):
    return torch.tensor(np.asarray(a), dtype=dtype, device=DEV).contiguous()


def ints(a):
    return torch.tensor(np.asarray(a, dtype=np.int32), device=DEV)


def host(t):
    return t.detach().float().cpu().numpy().astype(np.float64)


def segments_of(lengths):
    seg_row0 = np.concatenate([[0], np.cumsum(lengths)]).astype(np.int32)
    row_seg = np.concatenate([np.full(n, i) for i, n in enumerate(lengths)]).astype(np.int32)
    return seg_row0, row_seg


# ---- the input of the token before -------------------------------------------------------------------------
@pytest.mark.parametrize("out_dtype", DTYPES)
@pytest.mark.parametrize("hidden,lengths,normed", [(40, [1, 5, 1, 2], True), (300, [3], True), (2048, [1, 1, 1], True), (96, [2, 7], False)])
def test_token_shift_mix(ops, hidden, lengths, normed, out_dtype):
    rng = np.random.default_rng(hidden)
    rows, eps = sum(lengths), 1e-5
    slots = [3, 0, 2, 5][:len(lengths)]
    x = rng.normal(size=(rows, hidden)).astype(np.float32) * 2
    weight = rng.normal(size=hidden).astype(np.float32) * 0.1
    mu = rng.uniform(size=(5, hidden)).astype(np.float32)
    last = rng.normal(size=(6, hidden)).astype(np.float32)
    seg_row0, row_seg = segments_of(lengths)
    h = plain.norm_around_zero(x.astype(np.float64), weight.astype(np.float64), eps) if normed else x.astype(np.float64)
    before = np.zeros_like(h)
    for s, slot in enumerate(slots):
        a, b = seg_row0[s], seg_row0[s + 1]
        before[a] = last[slot]
        before[a + 1:b] = h[a:b - 1]
    expected = np.stack([h + (before - h) * mu[s] for s in range(5)])
    state = dev(last)
    found = ops.token_shift_mix(dev(x), dev(weight) if normed else None, eps, True, dev(mu), state, ints(row_seg), ints(seg_row0),
                                ints(slots), len(lengths), out_dtype)
    limit = 1e-5 if out_dtype == torch.float32 else 1e-2
    assert np.abs(host(found) - expected).max() <= limit * np.abs(expected).max()
    moved = host(state)
    for s, slot in enumerate(slots):
        assert np.abs(moved[slot] - h[seg_row0[s + 1] - 1]).max() <= 1e-5 * np.abs(h).max()
    untouched = [slot for slot in range(6) if slot not in slots]
    assert np.array_equal(moved[untouched], last[untouched].astype(np.float64))


# ---- the recurrence ----------------------------------------------------------------------------------------
def plain_recurrence(r, k, v, decay, u, S, heads, dim):
    """One segment, token by token and head by head, through ``plain.wkv_read_write``; S [heads, dim, dim] moves on."""
    out = np.zeros_like(r)
    for t in range(r.shape[0]):
        for head in range(heads):
            cut = slice(head * dim, (head + 1) * dim)
            out[t, cut], S[head] = plain.wkv_read_write(S[head], r[t, cut], k[t, cut], v[t, cut], decay[t, cut], u[cut])
    return out


@pytest.mark.parametrize("heads,dim", [(3, 4), (2, 24), (4, 64), (1, 100), (2, 128), (1, 256)])
def test_wkv_recurrence(ops, heads, dim):
    """Segments of 1, 4, 5, 8, 9, 16, 17, 31, 32, 33 and 70 tokens (the edges of chunks of every length the kernel
    takes) on slots in no order, from states that are not zero; then every request goes on by one token (the state of
    the first call carried)."""
    rng = np.random.default_rng(dim)
    lengths, slots = [1, 4, 5, 8, 9, 16, 17, 31, 32, 33, 70], [4, 0, 5, 2, 1, 11, 7, 12, 6, 9, 10]
    width, rows = heads * dim, sum(lengths)
    seg_row0, _ = segments_of(lengths)
    state = rng.normal(size=(13, heads, dim, dim)).astype(np.float32) * 0.3
    w0 = rng.normal(size=width).astype(np.float32) - 1.0
    u = rng.normal(size=width).astype(np.float32)
    device_state = dev(state)
    S = state.astype(np.float64).copy()
    for lengths_now in (lengths, [1] * len(lengths)):
        seg_row0, _ = segments_of(lengths_now)
        rows = sum(lengths_now)
        r, k, v = (rng.normal(size=(rows, width)).astype(np.float32) * dim ** -0.25 for _ in range(3))
        a = rng.normal(size=(rows, width)).astype(np.float32)
        decay = np.exp(-np.exp(a.astype(np.float64) + w0))
        expected = np.zeros((rows, width))
        for s, slot in enumerate(slots):
            cut = slice(seg_row0[s], seg_row0[s + 1])
            expected[cut] = plain_recurrence(r[cut].astype(np.float64), k[cut].astype(np.float64), v[cut].astype(np.float64), decay[cut],
                                             u.astype(np.float64), S[slot], heads, dim)
        found = ops.wkv_recurrence(dev(r), dev(k), dev(v), dev(a), dev(w0), dev(u), device_state, ints(seg_row0), ints(slots),
                                   len(slots), heads, dim)
        assert np.abs(host(found) - expected).max() <= 2e-5 * max(1.0, np.abs(expected).max())
        assert np.abs(host(device_state) - S).max() <= 2e-5 * max(1.0, np.abs(S).max())
        assert np.array_equal(host(device_state)[3], state[3].astype(np.float64)), "a slot of no request was touched"


def test_wkv_recurrence_gives_the_same_bits_however_the_tokens_are_cut(ops):
    heads, dim, rows = 2, 48, 70
    rng = np.random.default_rng(1)
    width = heads * dim
    r, k, v, a = (dev(rng.normal(size=(rows, width)).astype(np.float32) * 0.5) for _ in range(4))
    w0, u = dev(rng.normal(size=width) - 1.0), dev(rng.normal(size=width))

    def run(cuts):
        state = torch.zeros((2, heads, dim, dim), dtype=torch.float32, device=DEV)
        out, at = [], 0
        for n in cuts:
            out.append(ops.wkv_recurrence(r[at:at + n], k[at:at + n], v[at:at + n], a[at:at + n], w0, u, state, ints([0, n]), ints([1]), 1, heads, dim))
            at += n
        return torch.cat(out), state

    whole, state = run([rows])
    for cuts in ([1] * rows, [16, 16, 16, 16, 6], [2, 31, 1, 17, 19]):
        found, other = run(cuts)
        assert torch.equal(found, whole) and torch.equal(other, state), f"cut as {cuts}"


def test_wkv_bonus_counts_for_the_current_token_only(ops):
    """A state of zeros and one token: the read-out is (r . (u k)) v; the token after it sees k v^T without u."""
    dim = 16
    r = np.zeros((2, dim), dtype=np.float32); k = np.zeros((2, dim), dtype=np.float32); v = np.zeros((2, dim), dtype=np.float32)
    r[:, 3] = 2.0; k[0, 3] = 1.5; v[0, 7] = 4.0
    u = np.zeros(dim, dtype=np.float32); u[3] = 10.0
    a = np.full((2, dim), -30.0, dtype=np.float32)          # a decay of exp(-exp(-30)) = 1 to float32
    state = torch.zeros((1, 1, dim, dim), dtype=torch.float32, device=DEV)
    out = host(ops.wkv_recurrence(dev(r), dev(k), dev(v), dev(a), dev(np.zeros(dim)), dev(u), state, ints([0, 2]), ints([0]), 1, 1, dim))
    assert out[0, 7] == pytest.approx(2.0 * 10.0 * 1.5 * 4.0) and out[1, 7] == pytest.approx(2.0 * 1.5 * 4.0)
    assert np.count_nonzero(out) == 2


# ---- the router --------------------------------------------------------------------------------------------
@pytest.mark.parametrize("experts,top", [(2, 1), (7, 3), (12, 12), (64, 4), (200, 9)])
def test_moe_route(ops, experts, top):
    rng = np.random.default_rng(experts)
    rows = 50
    logits = rng.normal(size=(rows, experts)).astype(np.float32)
    logits[3] = 0.25                                        # all equal: the lowest ids, in order
    logits[4, : experts // 2] = logits[4, experts // 2: 2 * (experts // 2)]     # pairs of equal logits
    bias = rng.normal(size=experts).astype(np.float32)
    identity = np.eye(experts)
    want_chosen, want_weight = plain.route(logits.astype(np.float64), identity, bias.astype(np.float64), top)
    chosen, weight = ops.moe_route(dev(logits), dev(bias), top)
    summed = logits.astype(np.float64) + bias
    for row in range(rows):
        found = chosen[row].cpu().numpy()
        if len(set(np.round(summed[row], 6))) == experts:       # no ties after the bias in float32
            assert list(found) == list(want_chosen[row])
            assert np.abs(host(weight[row]) - want_weight[row]).max() < 1e-5
        assert len(set(found.tolist())) == top and abs(float(weight[row].sum()) - 1.0) < 1e-5
    no_bias = ops.moe_route(dev(logits), None, top)[0].cpu().numpy()
    assert list(no_bias[3]) == list(range(top))


def test_moe_arrange_keeps_an_experts_pairs_in_their_order(ops):
    rng = np.random.default_rng(5)
    for rows, experts, top in ((1, 4, 2), (37, 5, 3), (700, 12, 4), (3000, 130, 2)):
        chosen = np.stack([rng.permutation(experts)[:top] for _ in range(rows)]).astype(np.int32)
        begin, place_row, pair_place = (t.cpu().numpy() for t in ops.moe_arrange(ints(chosen), experts))
        flat = chosen.reshape(-1)
        assert begin[0] == 0 and begin[-1] == rows * top
        for e in range(experts):
            mine = np.nonzero(flat == e)[0]
            assert begin[e + 1] - begin[e] == len(mine)
            assert list(pair_place.reshape(-1)[mine]) == list(range(begin[e], begin[e + 1])), f"expert {e}: places out of order"
            assert list(place_row[begin[e]:begin[e + 1]]) == list(mine // top)


# ---- the experts' products ---------------------------------------------------------------------------------
def plain_grouped(a, rows_of_places, w, begin, gated):
    out = []
    for e in range(len(begin) - 1):
        x = a[rows_of_places[begin[e]:begin[e + 1]]]
        if gated:
            half = w.shape[1] // 2
            out.append(plain.silu(x @ w[e, :half].T) * (x @ w[e, half:].T))
        else:
            out.append(x @ w[e].T)
    return np.concatenate(out)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("rows,experts,top,K,N", [
    (5, 6, 2, 40, 24),          # few places: tiles of 32, experts without a place
    (9, 3, 3, 64, 100),         # every expert has every row; N no multiple of a tile
    (300, 4, 2, 96, 200),       # hundreds of places an expert: tiles of 128, the last one not full
    (70, 9, 4, 50, 12),         # K no multiple of 8: the plain form in either dtype
    (129, 2, 1, 264, 136),      # one place more than a tile
    (200, 130, 3, 64, 40),      # more experts than a wave has lanes
    (2100, 70, 2, 32, 72),      # tiles of 128 places over more than 64 experts, K of half a slab
])
def test_grouped_gemm(ops, dtype, rows, experts, top, K, N):
    rng = np.random.default_rng(rows + N)
    pool = experts - 1 if experts > 4 else experts         # the last expert of many has no place at all
    chosen = np.stack([rng.permutation(pool)[:top] for _ in range(rows)]).astype(np.int32)
    begin, place_row, _ = ops.moe_arrange(ints(chosen), experts)
    places = rows * top
    a = dev(rng.normal(size=(rows, K)), dtype)
    gate_up = dev(rng.normal(size=(experts, 2 * N, K)) * K ** -0.5, dtype)
    down = dev(rng.normal(size=(experts, K, N)) * N ** -0.5, dtype)
    hidden = ops.grouped_gemm(a, place_row, gate_up, begin, places, gated=True, out_dtype=dtype)
    b, pr = begin.cpu().numpy(), place_row.cpu().numpy()
    want_hidden = plain_grouped(host(a), pr, host(gate_up), b, True)
    limit = 2e-5 if dtype == torch.float32 else 1.5e-2
    assert hidden.shape == (places, N) and np.abs(host(hidden) - want_hidden).max() <= limit * np.abs(want_hidden).max()
    out = ops.grouped_gemm(hidden, None, down, begin, places, gated=False, out_dtype=torch.float32)
    want = plain_grouped(host(hidden), np.arange(places), host(down), b, False)
    assert out.shape == (places, K) and np.abs(host(out) - want).max() <= limit * np.abs(want).max()


def test_grouped_gemm_rows_do_not_depend_on_the_step(ops):
    """A row's products through the tiles of 32 places (alone with a few others) and through the tiles of 128 (among
    hundreds): the same bits."""
    rng = np.random.default_rng(2)
    experts, top, K, N, rows = 4, 2, 128, 192, 400
    chosen = np.stack([rng.permutation(experts)[:top] for _ in range(rows)]).astype(np.int32)
    a = dev(rng.normal(size=(rows, K)), torch.bfloat16)
    gate_up = dev(rng.normal(size=(experts, 2 * N, K)) * K ** -0.5, torch.bfloat16)
    down = dev(rng.normal(size=(experts, K, N)) * N ** -0.5, torch.bfloat16)

    def run(first, count):
        begin, place_row, pair_place = ops.moe_arrange(ints(chosen[first:first + count]), experts)
        hidden = ops.grouped_gemm(a[first:first + count], place_row, gate_up, begin, count * top, gated=True, out_dtype=torch.bfloat16)
        out = ops.grouped_gemm(hidden, None, down, begin, count * top, gated=False, out_dtype=torch.float32)
        return out[pair_place.long()]           # [rows, top, K] in the order of the rows

    everything = run(0, rows)
    for first, count in ((0, 3), (77, 1), (390, 10)):
        assert torch.equal(run(first, count), everything[first:first + count])


def test_moe_combine(ops):
    rng = np.random.default_rng(3)
    rows, top, hidden = 23, 3, 72
    x = rng.normal(size=(rows, hidden)).astype(np.float32)
    y = rng.normal(size=(rows * top, hidden)).astype(np.float32)
    weight = rng.uniform(size=(rows, top)).astype(np.float32)
    pair_place = rng.permutation(rows * top).reshape(rows, top).astype(np.int32)
    expected = x.astype(np.float64) + np.einsum("rt,rth->rh", weight.astype(np.float64), y.astype(np.float64)[pair_place])
    target = dev(x)
    ops.moe_combine_(target, dev(y), dev(weight), ints(pair_place))
    assert np.abs(host(target) - expected).max() <= 1e-5 * np.abs(expected).max()


# ---- attention: the kept first keys and the sink -----------------------------------------------------------
def paged(keys, values, dtype, pages):
    """[T, G, d] keys and [T, G, dv] values -> pages of 64 tokens in the order ``pages``; the rest is NaN."""
    T, G, d = keys.shape
    dv = values.shape[2]
    k_pages = torch.full((max(pages) + 1, G, 64, d), float("nan"), dtype=torch.float64)
    v_pages = torch.full((max(pages) + 1, G, dv, 64), float("nan"), dtype=torch.float64)
    for t in range(T):
        k_pages[pages[t // 64], :, t % 64, :] = torch.from_numpy(keys[t])
        v_pages[pages[t // 64], :, :, t % 64] = torch.from_numpy(values[t])
    return k_pages.to(dtype).to(DEV), v_pages.to(dtype).to(DEV)


def every_kernel(ops, q, H, G, d, dv, k_pages, v_pages, table, position, scale, window, keep_first, sinks, dtype):
    """The one row ``q`` at ``position`` through the generic kernel and, in bfloat16, the two of the matrix cores."""
    found = [ops.attention_generic(q, H, G, d, k_pages, v_pages, table, ints([0]), ints([position]), scale, window, v_dim=dv,
                                   keep_first=keep_first, sinks=sinks)]
    if dtype == torch.bfloat16:
        found.append(ops.attention_decode(q, H, G, d, k_pages, v_pages, table, ints([0]), ints([position]), scale, position + 1, window,
                                          v_dim=dv, keep_first=keep_first, sinks=sinks))
        found.append(ops.attention_prefill(q, H, G, d, k_pages, v_pages, table, ints([0]), ints([0]), ints([0, 1]), ints([position]), scale,
                                           window, v_dim=dv, keep_first=keep_first, sinks=sinks))
    return [host(f)[0].reshape(H, dv) for f in found]


@pytest.mark.parametrize("dtype", DTYPES)
def test_attention_sees_the_kept_first_keys_and_the_window_and_nothing_between(ops, dtype):
    """One key is made to match the query far better than all others. The row at 699 with a window of 100 that keeps
    5 first keys sees key 600 and key 4, not key 599 and not key 5; a sink far below the scores changes nothing."""
    H, G, d, dv, T = 4, 2, 64, 32, 700
    rng = np.random.default_rng(0)
    pages = [7, 2, 9, 0, 4, 11, 1, 8, 3, 10, 6]
    table = ints([pages])
    values = rng.normal(size=(T, G, dv))
    values = host(dev(values, dtype)).reshape(T, G, dv)
    q = np.zeros((1, H * d)); q[0, 5::d] = 60.0
    sinks = dev(np.full(H, -20.0))
    for target, seen in ((600, True), (599, False), (4, True), (5, False), (0, True), (699, True), (640, True), (300, False)):
        keys = rng.normal(size=(T, G, d)) * 0.1
        keys[target, :, :] = 0.0
        keys[target, :, 5] = 8.0
        k_pages, v_pages = paged(keys, values, dtype, pages)
        for found in every_kernel(ops, dev(q, dtype), H, G, d, dv, k_pages, v_pages, table, T - 1, d ** -0.5, 100, 5, sinks, dtype):
            for head in range(H):
                hit = np.abs(found[head] - values[target, head // 2]).max() < 0.05
                assert hit == seen, f"key {target}, head {head}"


@pytest.mark.parametrize("dtype", DTYPES)
def test_attention_sink_takes_its_share_and_has_no_value(ops, dtype):
    """One key decides the row (its score 60 above the rest). A sink equal to that score halves the output, a sink
    ln 3 above it leaves a quarter, each head by its own sink; the sink is not scaled with the scores."""
    H, G, d, dv, T = 2, 1, 32, 48, 130
    rng = np.random.default_rng(1)
    pages = [2, 0, 1]
    keys = rng.normal(size=(T, G, d)) * 0.05
    keys[70, 0, :] = 0.0
    keys[70, 0, 3] = 8.0
    values = host(dev(rng.normal(size=(T, G, dv)), dtype)).reshape(T, G, dv)
    q = np.zeros((1, H * d)); q[0, 3::d] = 16.0
    scale = 0.5
    score = 16.0 * 8.0 * scale
    sinks = dev([score, score + math.log(3.0)])
    k_pages, v_pages = paged(keys, values, dtype, pages)
    for window, keep_first in ((0, 0), (64, 2)):
        for found in every_kernel(ops, dev(q, dtype), H, G, d, dv, k_pages, v_pages, ints([pages]), T - 1, scale, window, keep_first, sinks, dtype):
            assert np.abs(found[0] - values[70, 0] / 2).max() < 0.03
            assert np.abs(found[1] - values[70, 0] / 4).max() < 0.03


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,G,d,dv,window,keep_first", [(4, 2, 32, 48, 40, 3), (6, 3, 16, 16, 33, 70), (2, 1, 64, 128, 1, 2), (3, 3, 48, 16, 0, 0)])
def test_attention_with_a_sink_against_the_plain_heads(ops, dtype, H, G, d, dv, window, keep_first):
    """Rows at several positions of a sequence of 200 (in the first window, across page borders, at the end)."""
    T = 200
    rng = np.random.default_rng(H + d)
    pages = [3, 1, 0, 2]
    q_all = host(dev(rng.normal(size=(T, H, d)), dtype)).reshape(T, H, d)
    keys = host(dev(rng.normal(size=(T, G, d)), dtype)).reshape(T, G, d)
    values = host(dev(rng.normal(size=(T, G, dv)), dtype)).reshape(T, G, dv)
    sink = rng.normal(size=H) * 2
    scale = 1.7 * d ** -0.5
    expected = plain.sink_heads(q_all, keys, values, scale, window or None, keep_first, sink)
    k_pages, v_pages = paged(keys, values, dtype, pages)
    for position in (0, 1, keep_first, window, 63, 64, 65, 128, 199):
        q = dev(q_all[position].reshape(1, H * d), dtype)
        limit = 2e-5 if dtype == torch.float32 else 2e-2
        for found in every_kernel(ops, q, H, G, d, dv, k_pages, v_pages, ints([pages]), position, scale, window, keep_first, dev(sink), dtype):
            assert np.abs(found - expected[position]).max() <= limit * max(1.0, np.abs(expected[position]).max()), f"position {position}"


@pytest.mark.parametrize("H,G,d,dv,window,keep_first", [(4, 2, 32, 48, 40, 3), (6, 3, 16, 16, 33, 70), (2, 1, 64, 128, 1, 2), (8, 2, 64, 64, 64, 1)])
def test_prompt_attention_with_kept_keys_and_a_sink_over_whole_tiles(ops, H, G, d, dv, window, keep_first):
    """A prompt of 200 rows in one call of the matrix-core prompt kernel (tiles of 64 rows: a window's edge and the
    kept keys' edge lie inside tiles and across pages), and its rows from 130 on as a portion behind cached keys;
    scores with a spread of several units, so that a key wrongly seen or missed moves the output."""
    T = 200
    rng = np.random.default_rng(H * d + window)
    pages = [3, 1, 0, 2]
    dtype = torch.bfloat16
    q_all = host(dev(rng.normal(size=(T, H, d)), dtype)).reshape(T, H, d)
    keys = host(dev(rng.normal(size=(T, G, d)), dtype)).reshape(T, G, d)
    values = host(dev(rng.normal(size=(T, G, dv)), dtype)).reshape(T, G, dv)
    sink = rng.normal(size=H) * 2
    scale = 3.0 * d ** -0.5
    expected = plain.sink_heads(q_all, keys, values, scale, window, keep_first, sink).reshape(T, H * dv)
    k_pages, v_pages = paged(keys, values, dtype, pages)
    for first in (0, 130):
        seg_row0 = [0, T - first]
        tile_seg, tile_row0 = ops.query_tiles(seg_row0)
        q = dev(q_all[first:].reshape(T - first, H * d), dtype)
        found = ops.attention_prefill(q, H, G, d, k_pages, v_pages, ints([pages]), ints(tile_seg), ints(tile_row0), ints(seg_row0),
                                      ints(np.arange(first, T)), scale, window, v_dim=dv, keep_first=keep_first, sinks=dev(sink))
        assert np.abs(host(found) - expected[first:]).max() <= 2e-2 * max(1.0, np.abs(expected).max()), f"rows from {first}"
        generic = ops.attention_generic(q, H, G, d, k_pages, v_pages, ints([pages]), ints(np.zeros(T - first)), ints(np.arange(first, T)),
                                        scale, window, v_dim=dv, keep_first=keep_first, sinks=dev(sink))
        assert np.abs(host(generic) - expected[first:]).max() <= 2e-2 * max(1.0, np.abs(expected).max()), f"plain kernel, rows from {first}"
