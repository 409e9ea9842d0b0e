"""Telapel's mechanisms one by one, each kernel against the plain function of ``plain_telapel`` (float64), at sizes of
the tests' own: the short causal convolution over mixed segments and slots, the gated linear recurrence, the router with
groups, the experts' clamped unit, the latent's store with its rotated part and the queries' side of it, the factor on the
queries, and attention with a bias by distance and a term of 1 in the softmax, with inputs made so that a single key
decides the output just inside and just outside the window."""

import math

import numpy as np
import pytest
import torch

import plain_telapel as plain

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
    row0 = np.concatenate([[0], np.cumsum(lengths)])
    row_seg = np.concatenate([np.full(n, s) for s, n in enumerate(lengths)])
    return ints(row_seg), ints(row0)


# ---- the convolution ---------------------------------------------------------------------------------------
@pytest.mark.parametrize("channels,taps,lengths", [(40, 4, [1, 5, 1, 2]), (300, 3, [70]), (7, 7, [2, 1, 9]), (64, 1, [3, 3]), (130, 2, [1, 1, 1])])
def test_causal_conv_over_segments_and_slots(ops, channels, taps, lengths):
    """Three steps over the same requests: every segment continues what its slot remembers, segments shorter than the
    taps reach back through several earlier steps, a step of single rows takes the one-launch path; some channels leave twice."""
    rng = np.random.default_rng(channels)
    w, bias = rng.normal(size=(channels, taps)), rng.normal(size=channels)
    slots = [5, 0, 3, 2][:len(lengths)]
    state = torch.zeros((7, channels, taps - 1), dtype=torch.float32, device=DEV)
    before = {slot: None for slot in slots}
    echo = (channels // 3, channels // 4)
    for step, single in ((0, False), (1, False), (2, True)):
        now = [1] * len(lengths) if single else [n + step for n in lengths]
        x = rng.normal(size=(sum(now), channels + 3))           # rows wider than the channels read
        row_seg, seg_row0 = segments_of(now)
        found = ops.causal_conv(dev(x)[:, :channels], dev(w), dev(bias), state, row_seg, seg_row0, ints(slots), len(now), single_rows=single,
                                echo=echo)
        at = 0
        for slot, n in zip(slots, now):
            want, before[slot] = plain.causal_conv(x[at:at + n, :channels], w, before[slot])
            got = host(found[at:at + n])
            assert np.abs(got[:, :channels] - (want + bias)).max() < 1e-5, f"step {step} slot {slot}"
            assert np.array_equal(got[:, channels:], got[:, echo[0]:echo[0] + echo[1]])
            at += n
    for slot in slots:
        if taps > 1:
            assert np.abs(host(state[slot]) - before[slot].T).max() < 1e-6


# ---- the recurrence ----------------------------------------------------------------------------------------
def plain_scan(u, gates, y, r_bias, i_bias, lam, S, block):
    C = u.shape[1]
    r_col = np.array([c // block * 2 * block + c % block for c in range(C)])
    r = plain.sigmoid(gates[:, r_col] + r_bias)
    i = plain.sigmoid(gates[:, r_col + block] + i_bias)
    out, S = plain.gated_recurrence(u, r, i, lam, S)
    return out * plain.gelu_tanh(y), S


@pytest.mark.parametrize("out_dtype", DTYPES)
@pytest.mark.parametrize("channels,block,lengths", [(12, 4, [1, 5, 1, 2]), (300, 100, [70, 9]), (64, 64, [1, 1, 1]), (50, 1, [17]),
                                                    (96, 32, [700, 3, 257, 256]), (40, 8, [1000])])
def test_rglru_scan(ops, channels, block, lengths, out_dtype):
    """Two steps over the same requests: decays from barely forgetting to forgetting at once, states carried in slots;
    segments of more than 256 rows are walked in chunks side by side, beside short ones walked in order."""
    rng = np.random.default_rng(channels + block)
    lam, r_bias, i_bias = rng.uniform(-6.0, 1.5, channels), rng.normal(size=channels), rng.normal(size=channels)
    slots = [4, 1, 0, 2][:len(lengths)]
    state = torch.zeros((6, channels), dtype=torch.float32, device=DEV)
    carried = {slot: None for slot in slots}
    for step in range(2):
        rows = sum(lengths)
        u, y, gates = rng.normal(size=(rows, channels)) * 2, rng.normal(size=(rows, channels)) * 2, rng.normal(size=(rows, 2 * channels)) * 2
        _, seg_row0 = segments_of(lengths)
        found = host(ops.rglru_scan(dev(u), dev(gates), dev(y), dev(r_bias), dev(i_bias), dev(lam), 8.0, state, seg_row0, ints(slots),
                                    len(lengths), block, out_dtype))
        at = 0
        for slot, n in zip(slots, lengths):
            want, carried[slot] = plain_scan(u[at:at + n], gates[at:at + n], y[at:at + n], r_bias, i_bias, lam, carried[slot], block)
            limit = 2e-5 if out_dtype == torch.float32 else 1e-2
            assert np.abs(found[at:at + n] - want).max() <= limit * max(1.0, np.abs(want).max()), f"step {step} slot {slot}"
            assert np.abs(host(state[slot]) - carried[slot]).max() <= 2e-5 * max(1.0, np.abs(carried[slot]).max())
            at += n


@pytest.mark.parametrize("rows", [1, 8, 16, 17])
@pytest.mark.parametrize("blocks,width", [(3, 40), (10, 256), (1, 7)])
def test_the_gates_maps_per_block(ops, rows, blocks, width):
    """Both gates of a block from one map per block, float32 inputs against bfloat16 weights: few rows (a wave per
    output) and more (tiles), the same numbers to float32 rounding."""
    rng = np.random.default_rng(rows + width)
    u = rng.normal(size=(rows, blocks * width))
    maps = host(dev(rng.normal(size=(blocks, 2 * width, width)) * width ** -0.5, torch.bfloat16))
    found = host(ops.head_linear(dev(u), dev(maps, torch.bfloat16), torch.float32))
    want = np.einsum("bnk,rbk->rbn", maps, host(dev(u)).reshape(rows, blocks, width)).reshape(rows, -1)
    assert np.abs(found - want).max() <= 1e-5 * max(1.0, np.abs(want).max())


def test_rglru_scan_gives_the_same_bits_however_the_tokens_are_cut(ops):
    rng = np.random.default_rng(7)
    channels, block, T = 96, 32, 150
    lam, r_bias, i_bias = rng.uniform(-6.0, 1.5, channels), rng.normal(size=channels), rng.normal(size=channels)
    u, y, gates = (dev(rng.normal(size=(T, width))) for width in (channels, channels, 2 * channels))

    def run(cuts):
        state = torch.zeros((2, channels), dtype=torch.float32, device=DEV)
        out, at, i = [], 0, 0
        while at < T:
            n = min(cuts[i % len(cuts)], T - at)
            out.append(ops.rglru_scan(u[at:at + n], gates[at:at + n], y[at:at + n], dev(r_bias), dev(i_bias), dev(lam), 8.0, state, ints([0, n]),
                                      ints([1]), 1, block, torch.float32))
            at, i = at + n, i + 1
        return torch.cat(out), state[1].clone()
    whole, last = run([T])
    for cuts in ([1], [2], [7, 8, 9, 64, 1]):
        rows, state = run(cuts)
        assert torch.equal(rows, whole) and torch.equal(state, last)


# ---- the router and the clamped unit -------------------------------------------------------------------------
@pytest.mark.parametrize("experts,top,groups,keep", [(2, 1, 2, 1), (12, 3, 3, 2), (16, 2, 2, 1), (9, 4, 3, 2), (64, 4, 8, 3), (200, 9, 4, 4), (6, 6, 1, 1)])
def test_moe_route_in_groups(ops, experts, top, groups, keep):
    rng = np.random.default_rng(experts + top)
    rows = 57
    logits = rng.normal(size=(rows, experts)).astype(np.float32) * 2
    logits[3] = 0.0                                           # all equal: the lowest groups, then the lowest ids
    logits[4, :] = np.round(logits[4, :])                     # many ties
    chosen, weight = ops.moe_route(dev(logits), None, top, groups, keep, score_all=True)
    want_chosen, want_weight = plain.route(np.eye(experts), logits.astype(np.float64).T, top, groups, keep) if False else (None, None)
    # the plain router reads h @ router.T: h = the logits themselves through an identity
    want_chosen, want_weight = plain.route(logits.astype(np.float64), np.eye(experts), top, groups, keep)
    assert np.array_equal(host(chosen).astype(np.int64), want_chosen)
    assert np.abs(host(weight) - want_weight).max() < 2e-6
    per_group = experts // groups
    assert all(len({e // per_group for e in row}) <= keep for row in host(chosen).astype(np.int64))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("rows,experts,top,K,N", [(5, 4, 2, 64, 40), (300, 6, 3, 96, 64), (33, 3, 1, 50, 12)])
def test_grouped_gemm_with_clamped_units(ops, dtype, rows, experts, top, K, N):
    rng = np.random.default_rng(rows)
    chosen = np.stack([rng.permutation(experts)[:top] for _ in range(rows)]).astype(np.int32)
    begin, place_row, _ = ops.moe_arrange(ints(chosen), experts)
    a = dev(rng.normal(size=(rows, K)) * 2, dtype)
    gate_up = dev(rng.normal(size=(experts, 2 * N, K)) * K ** -0.5, dtype)
    limit, alpha, shift = 1.3, 1.702, 1.0
    found = host(ops.grouped_gemm(a, place_row, gate_up, begin, rows * top, gated=True, out_dtype=dtype, glu=(limit, alpha, shift)))
    b, pr = begin.cpu().numpy(), place_row.cpu().numpy()
    A, W = host(a), host(gate_up)
    for e in range(experts):
        for place in range(b[e], b[e + 1]):
            g = np.minimum(W[e, :N] @ A[pr[place]], limit)
            u = np.clip(W[e, N:] @ A[pr[place]], -limit, limit)
            want = g * plain.sigmoid(alpha * g) * (u + shift)
            assert np.abs(found[place] - want).max() <= (2e-5 if dtype == torch.float32 else 2e-2) * max(1.0, np.abs(want).max())
    assert (np.abs(W[:, :N] @ A.T) > limit).any()           # the clamp bites somewhere


# ---- the latent's store, the queries' side, the factor on the queries ----------------------------------------------
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("rank,rot,turn", [(48, 16, 16), (32, 32, 8), (100, 2, 2), (24, 6, 0)])
def test_latent_store_with_a_rotated_part(ops, dtype, rank, rot, turn):
    rng = np.random.default_rng(rank)
    positions = np.array([0, 1, 63, 64, 130, 700])
    rows = len(positions)
    raw = rng.normal(size=(rows, rank + rot + 5))
    weight = rng.uniform(0.5, 1.5, rank)
    table = ints([[3, 0, 2, 5, 1, 4, 6, 7, 8, 9, 10]] * rows)
    k_pages = torch.full((11, 1, 64, rank + rot), float("nan"), dtype=dtype, device=DEV)
    v_pages = torch.full((11, 1, rank, 64), float("nan"), dtype=dtype, device=DEV)
    inv_freq = dev(100.0 ** (-2.0 * np.arange(turn // 2) / max(turn, 1)), torch.float64)
    cos, sin = ops.rope_table(ints(positions), inv_freq) if turn else (None, None)
    ops.latent_norm_write(dev(raw)[:, :rank + rot], dev(weight), 1e-5, k_pages, v_pages, table, ints(np.arange(rows)), ints(positions), rot=rot,
                          cos=cos, sin=sin, turn=turn)
    c = plain.rms_norm(raw[:, :rank], weight, 1e-5)
    part = plain.rotate_pairs(raw[:, rank:rank + rot], positions, turn, 100.0)
    limit = 1e-5 if dtype == torch.float32 else 1e-2
    pages = [3, 0, 2, 5, 1, 4, 6, 7, 8, 9, 10]
    for r, p in enumerate(positions):
        key = host(k_pages[pages[p // 64], 0, p % 64])
        assert np.abs(key[:rank] - c[r]).max() <= limit * np.abs(c[r]).max() and np.abs(key[rank:] - part[r]).max() <= limit * max(1.0, np.abs(part[r]).max())
        assert np.abs(host(v_pages[pages[p // 64], 0, :, p % 64]) - c[r]).max() <= limit * np.abs(c[r]).max()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("rows", [3, 40])
@pytest.mark.parametrize("heads,dim,rot,rank", [(4, 16, 16, 48), (3, 24, 8, 40), (1, 12, 2, 25)])
def test_queries_against_a_latent_with_a_rotated_part(ops, dtype, rows, heads, dim, rot, rank):
    """[W_uk^T q_plain | q_rot turned] head by head: the map per head reads the first channels of a head's vector and writes
    the first channels of a wider one, the rotation fills the rest."""
    rng = np.random.default_rng(heads * dim + rows)
    q = host(dev(rng.normal(size=(rows, heads * (dim + rot))), dtype))
    uk_t = host(dev(rng.normal(size=(heads, rank, dim)) * dim ** -0.5, dtype))
    positions = rng.integers(0, 900, size=rows)
    cos, sin = ops.rope_table(ints(positions), dev(1000.0 ** (-2.0 * np.arange(rot // 2) / rot), torch.float64))
    out = torch.full((rows, heads * (rank + rot)), float("nan"), dtype=dtype, device=DEV)
    ops.head_linear(dev(q, dtype), dev(uk_t, dtype), dtype, in_head=dim + rot, out=out, out_head=rank + rot)
    ops.rotate_place(dev(q, dtype), heads, dim, rot, cos, sin, out, rank)
    found = host(out).reshape(rows, heads, rank + rot)
    per_head = q.reshape(rows, heads, dim + rot)
    want_plain = np.einsum("hnk,rhk->rhn", uk_t, per_head[..., :dim])
    want_rot = plain.rotate_pairs(per_head[..., dim:], positions, rot, 1000.0)
    limit = 2e-5 if dtype == torch.float32 else 1.5e-2
    assert np.abs(found[..., :rank] - want_plain).max() <= limit * max(1.0, np.abs(want_plain).max())
    assert np.abs(found[..., rank:] - want_rot).max() <= limit * max(1.0, np.abs(want_rot).max())


def test_query_temperature(ops):
    positions = np.array([0, 1, 2, 3, 46, 47, 48, 95, 96, 4799, 100000])
    for coef, every in ((0.4, 48), (1.0, 1), (0.1, 3)):
        found = host(ops.query_temperature(ints(positions), coef, every))
        want = np.array([plain.query_factor(int(p), coef, every) for p in positions])
        assert np.abs(found - want).max() < 1e-6
    assert host(ops.query_temperature(ints([46, 47]), 0.4, 48)).tolist() == pytest.approx([1.0, 1.0 + 0.4 * math.log(2.0)])


# ---- attention: the window's edges, the bias by distance, the term of 1 -------------------------------------------
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


def slopes_of(heads, exponent=8.0):
    return 2.0 ** (-exponent * np.arange(1, heads + 1) / heads)


def every_kernel(ops, q, H, G, d, k_pages, v_pages, table, position, scale, window, softcap, dtype):
    """The one row ``q`` at ``position`` through the generic kernel and, in bfloat16 with heads in steps of 16 channels,
    the two of the matrix cores."""
    more = {"sinks": dev(np.zeros(H)), "slopes": dev(slopes_of(H)), "softcap": softcap}
    found = [ops.attention_generic(q, H, G, d, k_pages, v_pages, table, ints([0]), ints([position]), scale, window, **more)]
    if dtype == torch.bfloat16 and d % 16 == 0:
        found.append(ops.attention_decode(q, H, G, d, k_pages, v_pages, table, ints([0]), ints([position]), scale, position + 1, window, **more))
        found.append(ops.attention_prefill(q, H, G, d, k_pages, v_pages, table, ints([0]), ints([0]), ints([0, 1]), ints([position]), scale,
                                           window, **more))
    return [host(f)[0].reshape(H, d) for f in found]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("window", [40, 64, 65, 1, 130, 0])
def test_a_key_just_inside_and_just_outside_the_window(ops, dtype, window):
    """One key is made to match the query far better than all others: the row at 299 sees it at 299 - window + 1 and not
    one place earlier; at page borders; far back without a window. The bias by distance and the term of 1 are small
    beside that key's score."""
    H, G, d, T = 4, 2, 32, 300
    rng = np.random.default_rng(window)
    pages = [7, 2, 9, 0, 4]
    values = host(dev(rng.normal(size=(T, G, d)), dtype)).reshape(T, G, d)
    q = np.zeros((1, H * d)); q[0, 5::d] = 60.0
    edge = T - window if window else 0
    targets = [(edge, True), (edge - 1, False), (T - 1, True), (256, window == 0 or T - 1 - 256 < window), (255, window == 0 or T - 1 - 255 < window),
               (3, window == 0)]
    for target, seen in targets:
        if target < 0:
            continue
        keys = rng.normal(size=(T, G, d)) * 0.1
        keys[target, :, :] = 0.0
        keys[target, :, 5] = 8.0
        k_pages, v_pages = paged(keys, values, dtype, pages)
        for found in every_kernel(ops, dev(q, dtype), H, G, d, k_pages, v_pages, ints([pages]), T - 1, d ** -0.5, window, 0.0, dtype):
            for head in range(H):
                hit = np.abs(found[head] - values[target, head // 2]).max() < 0.05
                assert hit == seen, f"window {window}, key {target}, head {head}"


@pytest.mark.parametrize("dtype", DTYPES)
def test_the_term_of_one_and_the_bias_by_distance(ops, dtype):
    """All keys equal and orthogonal to the query (every score 0): the weights are exp(-slope_h * distance) / (1 + their
    sum), head by head; one value differs, so the output tells that key's weight."""
    H, G, d, T = 4, 1, 16, 200
    pages = [2, 0, 1, 3]
    keys = np.zeros((T, G, d)); keys[:, :, 0] = 1.0
    values = np.zeros((T, G, d)); values[150, 0, :] = 1.0
    q = np.zeros((1, H * d)); q[0, 1::d] = 3.0
    k_pages, v_pages = paged(keys, values, dtype, pages)
    for window in (0, 100):
        first = 0 if not window else T - window
        for found in every_kernel(ops, dev(q, dtype), H, G, d, k_pages, v_pages, ints([pages]), T - 1, 0.7, window, 20.0, dtype):
            for head, slope in enumerate(slopes_of(H)):
                weights = np.exp(-slope * (T - 1 - np.arange(first, T)))
                want = weights[150 - first] / (1.0 + weights.sum())
                assert abs(found[head, 0] - want) <= (1e-6 if dtype == torch.float32 else 3e-3 * want + 1e-4), f"window {window} head {head}"


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,G,d,window,softcap", [(6, 2, 32, 50, 20.0), (4, 4, 16, 33, 8.0), (2, 1, 48, 64, 0.0), (3, 1, 20, 0, 50.0), (8, 2, 64, 150, 30.0), (10, 2, 32, 40, 20.0)])
def test_attention_against_the_plain_heads(ops, dtype, H, G, d, window, softcap):
    """Rows at several positions of a sequence of 200 (in the first window, across page borders, at the end), and in
    bfloat16 the whole sequence as one prompt and as a portion behind cached keys, through the prompt kernel."""
    T = 200
    rng = np.random.default_rng(H + d)
    pages = [3, 1, 0, 2]
    q_all = host(dev(rng.normal(size=(T, H, d)), dtype)).reshape(T, H, d)
    keys = host(dev(rng.normal(size=(T, G, d)), dtype)).reshape(T, G, d)
    values = host(dev(rng.normal(size=(T, G, d)), dtype)).reshape(T, G, d)
    scale = 1.7 * d ** -0.5
    expected = plain.biased_heads(q_all, keys, values, 0, scale, window or None, softcap or None)
    k_pages, v_pages = paged(keys, values, dtype, pages)
    limit = 2e-5 if dtype == torch.float32 else 2e-2
    for position in (0, 1, max(window - 1, 0), window, 63, 64, 65, 128, 199):
        q = dev(q_all[position].reshape(1, H * d), dtype)
        for found in every_kernel(ops, q, H, G, d, k_pages, v_pages, ints([pages]), position, scale, window, softcap, dtype):
            assert np.abs(found - expected[position]).max() <= limit * max(1.0, np.abs(expected[position]).max()), f"position {position}"
    if dtype == torch.bfloat16 and d % 16 == 0:
        for first in (0, 130):
            seg_row0 = [0, T - first]
            tile_seg, tile_row0 = ops.query_tiles(seg_row0)
            q = dev(q_all[first:].reshape(T - first, H * d), dtype)
            # one query head to a workgroup, and four heads of a key head together where the kernel has that form
            for together in (1, 4) if d <= 64 and H // G >= 4 else (1,):
                found = ops.attention_prefill(q, H, G, d, k_pages, v_pages, ints([pages]), ints(tile_seg), ints(tile_row0), ints(seg_row0),
                                              ints(np.arange(first, T)), scale, window, heads_together=together, softcap=softcap,
                                              sinks=dev(np.zeros(H)), slopes=dev(slopes_of(H)))
                assert np.abs(host(found).reshape(-1, H, d) - expected[first:]).max() <= limit * max(1.0, np.abs(expected).max()), \
                    f"rows from {first}, {together} heads together"


@pytest.mark.parametrize("dtype", DTYPES)
def test_the_factor_on_the_queries_through_the_cache_write_and_the_fused_step(ops, dtype):
    """Normed queries times a factor per row: through the kernel that norms and stores (a wave a vector and eight rows a
    wave), and through the decode step that does both and attends in one kernel; the keys take no factor."""
    H, G, d = 4, 2, 32
    rng = np.random.default_rng(11)
    for rows in (3, 70):
        qkv = rng.normal(size=(rows, (H + 2 * G) * d))
        factor = rng.uniform(0.5, 4.0, rows)
        wq, wk = rng.uniform(0.5, 1.5, d), rng.uniform(0.5, 1.5, d)
        k_pages = torch.zeros((rows + 1, G, 64, d), dtype=dtype, device=DEV)
        v_pages = torch.zeros((rows + 1, G, d, 64), dtype=dtype, device=DEV)
        table = ints(np.arange(rows).reshape(rows, 1))
        positions = rng.integers(0, 64, size=rows)
        q = ops.qk_norm_rope_kv_write(dev(qkv), H, G, d, dev(wq), dev(wk), 1e-6, None, None, 0, k_pages, v_pages, table, ints(np.arange(rows)),
                                      ints(positions), q_row_scale=dev(factor))
        want_q = plain.rms_norm(qkv[:, :H * d].reshape(rows, H, d), wq, 1e-6) * factor[:, None, None]
        want_k = plain.rms_norm(qkv[:, H * d:(H + G) * d].reshape(rows, G, d), wk, 1e-6)
        limit = 1e-5 if dtype == torch.float32 else 1e-2
        assert np.abs(host(q).reshape(rows, H, d) - want_q).max() <= limit * np.abs(want_q).max()
        for r in range(rows):
            assert np.abs(host(k_pages[r, :, positions[r]]) - want_k[r]).max() <= limit * np.abs(want_k).max()
        if dtype == torch.bfloat16 and rows <= 16:
            more = {"sinks": dev(np.zeros(H)), "slopes": dev(slopes_of(H)), "softcap": 20.0}
            apart = ops.attention_decode(q, H, G, d, k_pages, v_pages, table, ints(np.arange(rows)), ints(positions), 0.3, 64, 0, **more)
            k_pages.zero_(); v_pages.zero_()
            fused = ops.attention_decode_fused(dev(qkv), H, G, d, dev(wq), dev(wk), 1e-6, None, None, 0, k_pages, v_pages, table,
                                               ints(np.arange(rows)), ints(positions), 0.3, 64, 0, q_row_scale=dev(factor), **more)
            assert torch.equal(fused, apart)
