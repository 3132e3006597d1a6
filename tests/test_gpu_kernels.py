"""Each HIP kernel alone against its plain PyTorch reference (tests/ref_ops.py), at sizes
other than the tiny models': head sizes in steps of 16, odd head and group counts, widths
and vocabularies that are no power of two, several page sizes; and inputs built so that a
fault that random data would hide (a far key, a window's edge, a page's edge) shows."""
import math

import pytest
import torch

import ref_ops

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
DTYPES = [torch.float32, torch.bfloat16]


@pytest.fixture(scope="module")
def ops():
    from macllm_infer_amd.kernels import build, ops as module
    module.require_gpu(DEV)
    build.ensure_modules(build.MODULES)
    return module


def rand(*shape, seed=0, scale=1.0, dtype=torch.float32):
    return (torch.randn(*shape, generator=torch.Generator().manual_seed(seed)) * scale).to(dtype)


def tol(dtype, scale=1.0):
    return (3e-5 if dtype == torch.float32 else 2.5e-2) * scale


def gpu(*tensors):
    return [None if t is None else t.to(DEV) for t in tensors]


def i32(values):
    return torch.tensor(values, dtype=torch.int32)


def close(got, want, dtype, scale=1.0):
    got, want = got.float().cpu(), want.float()
    assert got.shape == want.shape
    if got.numel() == 0:
        return
    assert torch.isfinite(got).all()
    error = (got - want).abs().max().item()
    assert error <= tol(dtype, scale), f"max error {error}"


# ------------------------------------------------------------------ common
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("d", [40, 1000, 4100])
def test_embed_and_add_rmsnorm(ops, dtype, d):
    T, V = 7, 203
    table = rand(V, d, seed=1, dtype=dtype)
    ids = i32([0, 202, 5, 5, 17, 100, 1])
    want_h = torch.empty(T, d)
    ref_ops.embed(ids, table, 1.7, want_h)
    h = torch.empty(T, d, device=DEV)
    ops.embed(ids.to(DEV), table.to(DEV), 1.7, h)
    close(h, want_h, torch.float32)
    deltas = [rand(T, d, seed=2, dtype=dtype), rand(T, d, seed=3, dtype=dtype)]
    weight = rand(d, seed=4) + 1.0
    for count in (0, 1, 2):
        want_h2, want_out = want_h.clone(), torch.empty(T, d, dtype=dtype)
        ref_ops.add_rmsnorm(want_h2, deltas[:count], weight, 3e-6, want_out)
        h2, out = h.clone(), torch.empty(T, d, dtype=dtype, device=DEV)
        ops.add_rmsnorm(h2, gpu(*deltas[:count]), weight.to(DEV), 3e-6, out)
        close(h2, want_h2, torch.float32)
        close(out, want_out, dtype, 4.0)
    rows = i32([6, 0, 3])
    want_out = torch.empty(3, d, dtype=dtype)
    keep = want_h.clone()
    ref_ops.add_rmsnorm(keep, deltas[:1], weight, 1e-5, want_out, rows)
    h3, out = h.clone(), torch.empty(3, d, dtype=dtype, device=DEV)
    ops.add_rmsnorm(h3, gpu(deltas[0]), weight.to(DEV), 1e-5, out, rows.to(DEV))
    close(out, want_out, dtype, 4.0)
    assert torch.equal(h3, h)                                   # with rows the stream is left alone


def test_rmsnorm_refuses_a_width_beyond_its_limit(ops):
    h = torch.zeros(1, 20000, device=DEV)
    with pytest.raises(ops.KernelError, match="size not supported"):
        ops.add_rmsnorm(h, [], torch.ones(20000, device=DEV), 1e-5, torch.empty(1, 20000, device=DEV))


@pytest.mark.parametrize("dtype", DTYPES)
def test_swiglu_and_scale(ops, dtype):
    gu = rand(9, 2 * 77, seed=5, scale=2.0, dtype=dtype)
    want = torch.empty(9, 77, dtype=dtype)
    ref_ops.swiglu(gu, want)
    out = torch.empty(9, 77, dtype=dtype, device=DEV)
    ops.swiglu(gu.to(DEV), out)
    close(out, want, dtype, 4.0)
    for width, tile in ((77, 7), (80, 8), (2048, 8)):          # gate and up interleaved in tiles
        tiled = rand(9, 2 * width, seed=6, scale=2.0, dtype=dtype)
        want = torch.empty(9, width, dtype=dtype)
        ref_ops.swiglu(tiled, want, tile)
        first = (torch.nn.functional.silu(tiled[:, :tile].float()) * tiled[:, tile:2 * tile].float()).to(dtype).float()
        assert torch.allclose(want[:, :tile].float(), first, rtol=1e-2 if dtype == torch.bfloat16 else 1e-6, atol=1e-6)
        out = torch.empty(9, width, dtype=dtype, device=DEV)
        ops.swiglu(tiled.to(DEV), out, tile)
        close(out, want, dtype, 4.0)
    logits = torch.empty(9, 154, device=DEV)
    ops.scale_to_f32(gu.to(DEV), 0.6, logits)
    close(logits, gu.float() * 0.6, torch.float32)


@pytest.mark.parametrize("shape", [(1, 64, 32), (5, 130, 97), (67, 100, 260), (130, 33, 1000), (40, 70, 3), (200, 257, 708)])
def test_float32_product_is_true_float32(ops, shape):
    M, N, K = shape
    x, w, b = rand(M, K, seed=6), rand(N, K, seed=7), rand(N, seed=8)
    want = (x.double() @ w.double().T + b.double()).float()
    got = ops.linear(x.to(DEV), w.to(DEV), b.to(DEV))
    assert (got.cpu() - want).abs().max() < 2e-5 * math.sqrt(K)       # float32 rounding only
    # a row's result does not depend on the rows beside it, nor on the tiling that the number of rows selects
    for rows in (1, 9, 17, 33, 65):
        if rows <= M:
            fewer = ops.linear(x[:rows].to(DEV), w.to(DEV), b.to(DEV))
            assert torch.equal(fewer, got[:rows]), rows
    last = ops.linear(x[M - 1:].to(DEV), w.to(DEV), b.to(DEV))
    assert torch.equal(last[0], got[M - 1])
    # a strided input (a column block of a wider matrix)
    wide = rand(M, K + 24, seed=9)
    got = ops.linear(wide.to(DEV)[:, 8:8 + K], w.to(DEV), None)
    assert (got.cpu() - (wide[:, 8:8 + K].double() @ w.double().T).float()).abs().max() < 2e-5 * math.sqrt(K)


def test_mixed_product_keeps_a_32bit_weight(ops):
    x, w = rand(4, 96, seed=10, dtype=torch.bfloat16), rand(50, 96, seed=11)
    got = ops.linear(x.to(DEV), w.to(DEV), None)
    assert got.dtype == torch.bfloat16
    close(got, (x.float() @ w.T).to(torch.bfloat16), torch.bfloat16, 10.0)
    both = ops.linear(x.to(DEV), w.to(torch.bfloat16).to(DEV), rand(50, seed=12).to(DEV))
    close(both, x.float() @ w.to(torch.bfloat16).float().T + rand(50, seed=12), torch.bfloat16, 10.0)


def test_bfloat16_product_adds_its_bias_in_float32(ops):
    """A bias that 16 bits cannot hold: 1 + 2^-8 rounds to 1 in bfloat16, and a product of 2^-8 added to that
    rounds to 1 again; added to the float32 sum it gives 1 + 2^-7, which bfloat16 holds."""
    x = torch.zeros(3, 32, dtype=torch.bfloat16)
    x[:, 0] = 2.0 ** -8
    w = torch.zeros(5, 32, dtype=torch.bfloat16)
    w[:, 0] = 1.0
    bias = torch.full((5,), 1.0 + 2.0 ** -8)
    got = ops.linear(x.to(DEV), w.to(DEV), bias.to(DEV))
    assert got.dtype == torch.bfloat16 and bool((got.float().cpu() == 1.0 + 2.0 ** -7).all())


def test_the_cap_on_the_logits_is_a_scaled_tanh(ops):
    """cap * tanh(x / cap), in place, at a size that is no multiple of the workgroup; small logits pass nearly as
    they are, large ones end at the cap, and the sign stays."""
    x = torch.randn(3, 1031, generator=torch.Generator().manual_seed(4)) * 6.0
    x[0, :4] = torch.tensor([0.0, 1e-3, -400.0, 400.0])
    got = x.to(DEV)
    ops.tanh_softcap(got, 2.5)
    want = 2.5 * torch.tanh(x.double() / 2.5)
    assert (got.cpu().double() - want).abs().max() < 1e-6
    assert got[0, :4].cpu().tolist() == pytest.approx([0.0, 1e-3, -2.5, 2.5], abs=1e-7)
    with pytest.raises(ops.KernelError):
        ops.tanh_softcap(got, 0.0)


# ------------------------------------------------------------------ attention
def paged_setup(lengths, page_size, Hkv, dh, dtype, layers=2, seed=0):
    """A pool of shuffled pages [page, layer, K|V, Hkv, page_size*dh] and a block table per lane."""
    generator = torch.Generator().manual_seed(seed)
    pages_per_lane = [-(-length // page_size) for length in lengths]
    total = sum(pages_per_lane) + 3
    order = torch.randperm(total, generator=generator).tolist()
    table = torch.zeros(len(lengths), max(pages_per_lane), dtype=torch.int32)
    cursor = 0
    for lane, count in enumerate(pages_per_lane):
        table[lane, :count] = torch.tensor(order[cursor:cursor + count], dtype=torch.int32)
        cursor += count
    pool = torch.full((total, layers, 2, Hkv, page_size * dh), float("nan"), dtype=dtype)
    return pool, table


def views(pool, page_size, layer=1):
    """One layer's K pages [pages, Hkv, page_size, dh] and transposed V pages [pages, Hkv, dh, page_size]."""
    dh = pool.shape[-1] // page_size
    return (pool[:, layer, 0].unflatten(-1, (page_size, dh)), pool[:, layer, 1].unflatten(-1, (dh, page_size)))


def fill_cache(pool, table, lane, keys, values, page_size, layer=1):
    k_pages, v_pages = views(pool, page_size, layer)
    for position in range(keys.shape[0]):
        page = int(table[lane, position // page_size])
        k_pages[page, :, position % page_size, :] = keys[position]
        v_pages[page, :, :, position % page_size] = values[position]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("Hq, Hkv, dh, page_size, rotary", [
    (4, 2, 16, 8, 16), (5, 5, 48, 16, 48), (6, 2, 80, 4, 32), (8, 2, 64, 64, 64), (3, 1, 128, 16, 128),
    (2, 1, 256, 32, 256)])
def test_rope_store_and_attention_over_pages(ops, dtype, Hq, Hkv, dh, page_size, rotary):
    """Three lanes: a prompt portion that continues a cached prefix, a single decoded token,
    and a fresh prompt.  Every unwritten cache cell holds NaN, so reading a cell that is
    not the request's shows."""
    starts, counts = [21, 70, 0], [13, 1, 37]
    lengths = [s + c for s, c in zip(starts, counts)]
    pool, table = paged_setup(lengths, page_size, Hkv, dh, dtype)
    for lane, start in enumerate(starts):       # prefixes already in the cache (post-rotation keys)
        fill_cache(pool, table, lane, rand(start, Hkv, dh, seed=20 + lane, dtype=dtype),
                   rand(start, Hkv, dh, seed=30 + lane, dtype=dtype), page_size)
    T = sum(counts)
    width = (Hq + 2 * Hkv) * dh
    qkv = rand(T, width + 8, seed=40, dtype=dtype)            # wider than needed: a row stride
    positions = torch.cat([torch.arange(s, s + c) for s, c in zip(starts, counts)]).to(torch.int32)
    lane_of_token = torch.repeat_interleave(torch.arange(3), torch.tensor(counts)).to(torch.int32)
    slot_mapping = torch.tensor([int(table[l, p // page_size]) * page_size + p % page_size
                                 for l, p in zip(lane_of_token.tolist(), positions.tolist())], dtype=torch.int32)
    inv_freq = torch.tensor([1.0 / (1e4 ** (i / rotary)) for i in range(0, rotary, 2)], dtype=torch.float64).float()
    want_qkv, want_pool = qkv.clone(), pool.clone()
    ref_ops.rope_kv_store(want_qkv, Hq, Hkv, dh, positions, inv_freq, rotary, slot_mapping,
                          *views(want_pool, page_size))
    got_qkv, got_pool = qkv.to(DEV), pool.to(DEV)
    ops.rope_kv_store(got_qkv, Hq, Hkv, dh, positions.to(DEV), inv_freq.to(DEV), rotary, slot_mapping.to(DEV),
                      *views(got_pool, page_size))
    close(got_qkv[:, :Hq * dh], want_qkv[:, :Hq * dh], dtype, 4.0)
    assert torch.equal(got_qkv[:, Hq * dh:].cpu(), qkv[:, Hq * dh:])         # k, v columns untouched
    written = ~torch.isnan(want_pool.float())
    assert torch.equal(torch.isnan(got_pool.float().cpu()), ~written)          # exactly the same cells
    close(torch.nan_to_num(got_pool.float()), torch.nan_to_num(want_pool.float()), dtype, 4.0)
    assert torch.isnan(got_pool[:, 0].float()).all()                           # the other layer is untouched
    slopes = torch.tensor([0.4 / (head + 1) for head in range(Hq)])
    for window, bias in ((None, None), (9, None), (None, slopes), (9, slopes)):     # bias: a slope per head times the distance
        want = torch.empty(T, Hq * dh, dtype=dtype)
        ref_ops.paged_attention(want_qkv, Hq, Hkv, dh, *views(want_pool, page_size), table,
                                lane_of_token, positions, 0.37, window, want, slopes=bias)
        got = torch.empty(T, Hq * dh, dtype=dtype, device=DEV)
        ops.paged_attention(got_qkv, Hq, Hkv, dh, *views(got_pool, page_size), table.to(DEV),
                            lane_of_token.to(DEV), positions.to(DEV), 0.37, window, got,
                            slopes=None if bias is None else bias.to(DEV))
        close(got, want, dtype, 3.0)
        if bias is not None and window is None:
            plain = torch.empty(T, Hq * dh, dtype=dtype)
            ref_ops.paged_attention(want_qkv, Hq, Hkv, dh, *views(want_pool, page_size), table,
                                    lane_of_token, positions, 0.37, window, plain)
            assert (plain.float() - want.float()).abs().max() > 0.05          # the bias changes the result


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("page_size", [16, 64])
def test_one_far_key_among_hundreds_is_found(ops, dtype, page_size):
    """One decoded token over 700 cached keys.  The query and one chosen key are scaled so that
    this key takes all the weight: the output must be that key's value, for keys at the
    start, at both sides of page edges, and at the end."""
    Hq, Hkv, dh, length = 4, 2, 64, 700
    pool, table = paged_setup([length], page_size, Hkv, dh, dtype, seed=3)
    values = rand(length, Hkv, dh, seed=50, dtype=dtype)
    base_keys = rand(length, Hkv, dh, seed=51, scale=0.1, dtype=dtype)
    direction = torch.zeros(dh)
    direction[5] = 1.0
    for chosen in (0, 1, page_size - 1, page_size, 63, 64, 65, 255, 256, 257, 511, 512, length - 2, length - 1):
        keys = base_keys.clone()
        keys[chosen] = (direction * 30.0).to(dtype)
        fill_cache(pool, table, 0, keys, values, page_size)
        q = (direction * 30.0).repeat(Hq)[None].to(dtype)
        out = torch.empty(1, Hq * dh, dtype=dtype, device=DEV)
        dev_pool = pool.to(DEV)
        ops.paged_attention(q.to(DEV), Hq, Hkv, dh, *views(dev_pool, page_size), table.to(DEV),
                            i32([0]).to(DEV), i32([length - 1]).to(DEV), 1.0 / math.sqrt(dh), None, out)
        expected = values[chosen].float()[[0, 0, 1, 1]].reshape(-1)
        assert (out.float().cpu()[0] - expected).abs().max() < 1e-2, f"key {chosen} was missed"


@pytest.mark.parametrize("dtype", DTYPES)
def test_window_edge(ops, dtype):
    """Window 37 at query position 299: key 263 is the last one inside, key 262 the first one
    outside.  Whichever is made to stand out, the output tells whether it was seen."""
    Hq, Hkv, dh, length, window, page_size = 2, 1, 32, 300, 37, 16
    pool, table = paged_setup([length], page_size, Hkv, dh, dtype, seed=4)
    values = rand(length, Hkv, dh, seed=52, dtype=dtype)
    direction = torch.zeros(dh)
    direction[0] = 1.0
    q = (direction * 30.0).repeat(Hq)[None].to(dtype).to(DEV)
    for chosen, visible in ((263, True), (262, False), (299, True), (0, False)):
        keys = rand(length, Hkv, dh, seed=53, scale=0.1, dtype=dtype)
        keys[chosen] = (direction * 30.0).to(dtype)
        fill_cache(pool, table, 0, keys, values, page_size)
        dev_pool = pool.to(DEV)
        out = torch.empty(1, Hq * dh, dtype=dtype, device=DEV)
        ops.paged_attention(q, Hq, Hkv, dh, *views(dev_pool, page_size), table.to(DEV), i32([0]).to(DEV),
                            i32([length - 1]).to(DEV), 1.0 / math.sqrt(dh), window, out)
        hit = (out.float().cpu()[0, :dh] - values[chosen, 0].float()).abs().max() < 1e-2
        assert hit == visible, f"key {chosen} should be {'visible' if visible else 'masked'}"
        want = torch.empty(1, Hq * dh, dtype=dtype)
        ref_ops.paged_attention(q.cpu(), Hq, Hkv, dh, *views(pool, page_size), table, i32([0]),
                                i32([length - 1]), 1.0 / math.sqrt(dh), window, want)
        close(out, want, dtype, 3.0)


@pytest.mark.parametrize("dtype", DTYPES)
def test_window_across_the_edge_of_a_run_of_keys(ops, dtype):
    """The general kernel cuts the keys into runs of 256 by position: a window of 60 at position 299 holds
    keys 240..299, on both sides of that edge; and one at position 600 of window 300 spans two edges."""
    Hq, Hkv, dh, page_size = 3, 1, 48, 16
    for length, window, cases in ((300, 60, ((240, True), (239, False), (255, True), (256, True))),
                                  (601, 300, ((301, True), (300, False), (511, True), (512, True), (600, True)))):
        pool, table = paged_setup([length], page_size, Hkv, dh, dtype, seed=14)
        values = rand(length, Hkv, dh, seed=54, dtype=dtype)
        direction = torch.zeros(dh)
        direction[3] = 1.0
        q = (direction * 30.0).repeat(Hq)[None].to(dtype).to(DEV)
        for chosen, visible in cases:
            keys = rand(length, Hkv, dh, seed=55, scale=0.1, dtype=dtype)
            keys[chosen] = (direction * 30.0).to(dtype)
            fill_cache(pool, table, 0, keys, values, page_size)
            dev_pool = pool.to(DEV)
            out = torch.empty(1, Hq * dh, dtype=dtype, device=DEV)
            ops.paged_attention(q, Hq, Hkv, dh, *views(dev_pool, page_size), table.to(DEV), i32([0]).to(DEV),
                                i32([length - 1]).to(DEV), 1.0 / math.sqrt(dh), window, out)
            hit = (out.float().cpu()[0, :dh] - values[chosen, 0].float()).abs().max() < 1e-2
            assert hit == visible, f"key {chosen} should be {'visible' if visible else 'masked'}"
            want = torch.empty(1, Hq * dh, dtype=dtype)
            ref_ops.paged_attention(q.cpu(), Hq, Hkv, dh, *views(pool, page_size), table, i32([0]),
                                    i32([length - 1]), 1.0 / math.sqrt(dh), window, want)
            close(out, want, dtype, 3.0)


def test_general_attention_does_not_depend_on_the_step_around_a_token(ops):
    """float32: a token's attended row is bit for bit the same alone, among the tokens of a prompt portion,
    beside another request, and whatever bound of the longest context sizes the launch."""
    Hq, Hkv, dh, page_size = 4, 2, 40, 16
    lengths = [700, 90]
    pool, table = paged_setup(lengths, page_size, Hkv, dh, torch.float32, seed=15)
    for lane, length in enumerate(lengths):
        fill_cache(pool, table, lane, rand(length, Hkv, dh, seed=56 + lane), rand(length, Hkv, dh, seed=58 + lane), page_size)
    dev_pool, dev_table = pool.to(DEV), table.to(DEV)
    positions = i32(list(range(500, 700)) + list(range(60, 90)))
    lane_of_token = i32([0] * 200 + [1] * 30)
    q = rand(230, Hq * dh, seed=60).to(DEV)
    whole = torch.empty(230, Hq * dh, device=DEV)
    ops.paged_attention(q, Hq, Hkv, dh, *views(dev_pool, page_size), dev_table, lane_of_token.to(DEV),
                        positions.to(DEV), 0.2, None, whole)
    want = torch.empty(230, Hq * dh)
    ref_ops.paged_attention(q.cpu(), Hq, Hkv, dh, *views(pool, page_size), table, lane_of_token, positions, 0.2, None, want)
    close(whole, want, torch.float32, 3.0)
    for row, bound in ((0, None), (199, 700), (199, 704), (200, 90), (229, None), (12, 513)):
        alone = torch.empty(1, Hq * dh, device=DEV)
        ops.paged_attention(q[row:row + 1], Hq, Hkv, dh, *views(dev_pool, page_size), dev_table,
                            lane_of_token[row:row + 1].to(DEV), positions[row:row + 1].to(DEV), 0.2, None, alone, bound)
        assert torch.equal(alone[0], whole[row]), (row, bound)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("Hq, Hkv, dh, page_size, tile", [(4, 2, 64, 16, 64), (6, 2, 48, 8, 16), (3, 1, 128, 4, 32),
                                                           (2, 2, 256, 64, 64), (5, 5, 16, 16, 48)])
def test_tiled_general_attention_gives_the_per_token_kernels_bits(ops, dtype, Hq, Hkv, dh, page_size, tile):
    """Lanes of several tokens go through the kernel that fetches a run of keys once for sixteen queries; a
    position's attended row must be the per-token kernel's, bit for bit, in both dtypes, with a window, with a
    bias by distance, for portions that cross the edges of pages, of 64-key groups and of 256-key runs, beside a
    single token and a short fresh prompt, with rows of the table that hold nothing, and with NaN in every cache
    cell that no request wrote."""
    starts, counts = [300, 0, 519, 250, 0], [150, 70, 1, 9, 3]
    lengths = [s + c for s, c in zip(starts, counts)]
    pool, table = paged_setup(lengths, page_size, Hkv, dh, dtype, seed=31)
    for lane, length in enumerate(lengths):
        fill_cache(pool, table, lane, rand(length, Hkv, dh, seed=300 + lane, dtype=dtype),
                   rand(length, Hkv, dh, seed=320 + lane, dtype=dtype), page_size)
    T = sum(counts)
    q = rand(T, Hq * dh + 16, seed=340, dtype=dtype).to(DEV)[:, :Hq * dh]            # a row stride
    positions = torch.cat([torch.arange(s, s + c) for s, c in zip(starts, counts)]).to(torch.int32)
    lane_of_token = torch.repeat_interleave(torch.arange(len(counts)), torch.tensor(counts)).to(torch.int32)
    cu = [0]
    for count in counts:
        cu.append(cu[-1] + count)
    tiles = [[-1, 0]]                                                       # a row that holds nothing, first
    for lane, count in enumerate(counts):
        tiles += [[lane, row] for row in range(cu[lane], cu[lane + 1], tile)]
    tiles += [[-1, 0], [-1, 0]]
    dev_pool = pool.to(DEV)
    k_cache, v_cache = views(dev_pool, page_size)
    slopes = torch.tensor([0.3 / (head + 1) for head in range(Hq)])
    for window, bias, bound in ((None, None, None), (70, None, 520), (None, slopes, 700), (300, slopes, None)):
        results = []
        for with_tiles in (False, True):
            out = torch.full((T, Hq * dh), float("nan"), dtype=dtype, device=DEV)
            extra = dict(query_tiles=i32(tiles).to(DEV), tile_tokens=tile, cu_seqlens=i32(cu).to(DEV)) if with_tiles else {}
            ops.paged_attention(q, Hq, Hkv, dh, k_cache, v_cache, table.to(DEV), lane_of_token.to(DEV), positions.to(DEV),
                                0.31, window, out, bound, None if bias is None else bias.to(DEV), **extra)
            results.append(out)
        assert not torch.isnan(results[0].float()).any()
        assert torch.equal(results[0], results[1]), (window, bias is not None, (results[0].float() - results[1].float()).abs().max().item())
    want = torch.empty(T, Hq * dh, dtype=dtype)
    ref_ops.paged_attention(q.cpu(), Hq, Hkv, dh, *views(pool, page_size), table, lane_of_token, positions, 0.31, 300,
                            want, slopes=slopes)
    close(results[1], want, dtype, 3.0)


def test_attention_refuses_a_head_size_beyond_its_limit(ops):
    pool = torch.zeros(2, 1, 2, 1, 16 * 320, device=DEV)
    q = torch.zeros(1, 320, device=DEV)
    with pytest.raises(ops.KernelError, match="size not supported"):
        ops.paged_attention(q, 1, 1, 320, *views(pool, 16, 0), i32([[0]]).to(DEV), i32([0]).to(DEV),
                            i32([0]).to(DEV), 1.0, None, torch.empty(1, 320, device=DEV))


# ------------------------------------------------------------------ mamba2
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H, P, N, G, K", [(8, 8, 16, 1, 4), (6, 16, 32, 2, 3), (3, 24, 40, 3, 2), (4, 64, 128, 1, 4),
                                             (2, 40, 256, 2, 4), (5, 7, 9, 1, 1), (1, 8, 512, 1, 4), (2, 16, 64, 1, 4),
                                             (3, 5, 4, 1, 2), (2, 3, 1, 1, 2), (2, 6, 72, 2, 4)])
def test_mamba2_kernels_over_ragged_lanes(ops, dtype, H, P, N, G, K):
    """Lanes of 1, 2 (shorter than the conv tail), 19 and 45 tokens with non-zero conv tails
    and states in shuffled slots; the slot no lane uses must stay as it was."""
    E, GN = H * P, G * N
    C, W = E + 2 * GN, 2 * E + 2 * GN + H
    counts = [1, 2, 19, 45]
    T = sum(counts)
    slots = 6
    slot_ids = i32([4, 0, 5, 2])
    cu = i32([0, 1, 3, 22, 67])
    lane_of_token = torch.repeat_interleave(torch.arange(4), torch.tensor(counts)).to(torch.int32)
    u = rand(T, W, seed=60, dtype=dtype)
    conv_w, conv_b = rand(C, K, seed=61, scale=0.5), rand(C, seed=62, scale=0.1)
    conv_state = rand(slots, max(K - 1, 0), C, seed=63, dtype=dtype)
    ssm_state = rand(slots, H, P, N, seed=64, scale=0.5)
    dt_bias, A, D = rand(H, seed=65) - 2.0, -(rand(H, seed=66).abs() + 0.1), rand(H, seed=67)
    norm_w = rand(E, seed=68) + 1.0

    def run(module, device):
        mv = lambda t: None if t is None else t.to(device)
        uu, cs, ss = mv(u), mv(conv_state.clone()), mv(ssm_state.clone())
        xbc = torch.empty(T, C, dtype=dtype, device=device)
        module.conv1d_silu(uu, E, C, mv(conv_w), mv(conv_b), cs, mv(lane_of_token), mv(cu), mv(slot_ids), xbc)
        module.conv_state_update(uu, E, C, K, cs, mv(cu), mv(slot_ids))
        y = torch.empty(T, E, dtype=torch.float32, device=device)
        module.ssm_scan(xbc, uu[:, E + C:], mv(dt_bias), mv(A), mv(D), ss, mv(cu), mv(slot_ids), G, y)
        outs = []
        for weight in (None, norm_w):
            out = torch.empty(T, E, dtype=dtype, device=device)
            module.gate_norm(y, uu[:, :E], mv(weight), G, 1e-5, out)
            outs.append(out)
        return xbc, cs, ss, y, outs

    want = run(ref_ops, "cpu")
    got = run(ops, DEV)
    close(got[0], want[0], dtype, 4.0)
    close(got[1], want[1], dtype)
    scale = max(1.0, want[3].abs().max().item())
    # the scan's inputs are the GPU conv outputs; in bfloat16 they may differ from the reference's by one rounding
    close(got[2], want[2], dtype, scale)
    close(got[3], want[3], dtype, scale)
    close(got[4][0], want[4][0], dtype, scale)
    close(got[4][1], want[4][1], dtype, 8.0)
    for untouched in (1, 3):
        assert torch.equal(got[1][untouched].cpu(), conv_state[untouched])
        assert torch.equal(got[2][untouched].cpu(), ssm_state[untouched])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("M, C, K, col_offset, ld", [(1, 40, 4, 0, 40), (7, 100, 3, 13, 131), (64, 1792, 4, 1536, 4120),
                                                     (5, 33, 1, 2, 40), (9, 24, 9, 8, 32)])
def test_conv_step_of_single_token_lanes(ops, dtype, M, C, K, col_offset, ld):
    """The in-place conv step against conv1d_silu + conv_state_update of one-token lanes; the slots are a
    permutation with unused ones between, whose tails must stay as they were; so must the other columns."""
    u = rand(M, ld, seed=1, dtype=dtype)
    weight, bias = rand(C, K, seed=2, scale=0.5), rand(C, seed=3)
    slots = 2 * M + 1
    state = rand(slots, max(K - 1, 0), C, seed=4, dtype=dtype)
    slot_ids = i32(torch.randperm(slots, generator=torch.Generator().manual_seed(5))[:M].tolist())
    for with_bias in (True, False):
        want_u, want_state = u.clone(), state.clone()
        ref_ops.conv_step(want_u, col_offset, C, weight, bias if with_bias else None, want_state, slot_ids)
        got_u, got_state, w, b, ids = gpu(u.clone(), state.clone(), weight, bias if with_bias else None, slot_ids)
        ops.conv_step(got_u, col_offset, C, w, b, got_state, ids)
        close(got_u, want_u, dtype, 4.0)
        assert torch.equal(got_state.cpu(), want_state)
        untouched = torch.ones(ld, dtype=torch.bool)
        untouched[col_offset:col_offset + C] = False
        assert torch.equal(got_u.cpu()[:, untouched], u[:, untouched])


@pytest.mark.parametrize("Q", [32, 64, 128, 256])
@pytest.mark.parametrize("H, P, N, G", [(4, 16, 32, 1), (6, 32, 64, 2), (5, 64, 128, 1), (9, 16, 96, 3), (2, 48, 256, 2)])
def test_chunked_scan_matches_the_token_by_token_scan(ops, Q, H, P, N, G):
    """Lanes of 1, 2, 37, 128 and 301 tokens from non-zero states in shuffled slots, whatever the
    chunk size; the decay is strong enough in some heads to forget a chunk and weak in others."""
    E, GN = H * P, G * N
    counts = [1, 2, 37, 128, 301]
    T = sum(counts)
    slot_ids = i32([4, 0, 5, 2, 1])
    cu = i32([0] + torch.tensor(counts).cumsum(0).tolist())
    xbc = rand(T, E + 2 * GN, seed=80, dtype=torch.bfloat16)
    dt = rand(T, H, seed=81, dtype=torch.bfloat16)
    dt_bias = rand(H, seed=82) - 1.0
    A = -torch.exp(torch.linspace(-4.0, 1.5, H))
    D = rand(H, seed=83)
    state = rand(7, H, P, N, seed=84, scale=0.5)
    want_y, want_state = torch.empty(T, E), state.clone()
    ref_ops.ssm_scan(xbc, dt, dt_bias, A, D, want_state, cu, slot_ids, G, want_y)
    assert ops.ssd_supported(Q, P, N, G, E)
    y, got_state = torch.full((T, E), float("nan"), device=DEV), state.to(DEV)
    table = ops.SsdChunks(counts, Q, DEV)
    ops.ssd_prefill(xbc.to(DEV), dt.to(DEV), *gpu(dt_bias, A, D), got_state, table, slot_ids.to(DEV), G, y)
    scale = max(1.0, want_y.abs().max().item())
    close(y, want_y, torch.bfloat16, scale)
    close(got_state, want_state, torch.bfloat16, max(1.0, want_state.abs().max().item()))
    for untouched in (3, 6):
        assert torch.equal(got_state[untouched].cpu(), state[untouched])
    # the gate on the way out: y * SiLU(z), z a column view of a wider matrix
    wide = rand(T, E + 8, seed=85, dtype=torch.bfloat16)
    want_gated = torch.empty(T, E, dtype=torch.bfloat16)
    ref_ops.gate_norm(want_y, wide[:, 8:], None, G, 1e-5, want_gated)
    gated, again = torch.empty(T, E, dtype=torch.bfloat16, device=DEV), state.to(DEV)
    ops.ssd_prefill(xbc.to(DEV), dt.to(DEV), *gpu(dt_bias, A, D), again, table, slot_ids.to(DEV), G, None,
                    z=wide.to(DEV)[:, 8:], gated=gated)
    close(gated, want_gated, torch.bfloat16, max(1.0, want_gated.float().abs().max().item()))
    assert torch.equal(again, got_state)


@pytest.mark.parametrize("K, Q, bias", [(4, 128, True), (3, 32, False), (2, 64, True), (4, 32, True)])
def test_chunked_scan_with_the_conv_inside(ops, K, Q, bias):
    """The conv and the tail update inside the chunked scan's launches against the separate kernels:
    lanes of 1 and 2 tokens (shorter than the taps: part of the old tail stays), lanes that end on a
    chunk's edge and one token after it, a lane of many chunks; shuffled slots; the raw rows are a
    column view of a wider matrix; 192 conv channels = three blocks of 64, the last without x or B."""
    H, P, N, G = 4, 16, 32, 2
    E, GN = H * P, G * N
    C = E + 2 * GN
    counts = [1, 2, Q, Q + 1, 3 * Q + 7, 5]
    T = sum(counts)
    slots = len(counts) + 2
    slot_ids = i32(torch.randperm(slots, generator=torch.Generator().manual_seed(9))[:len(counts)].tolist())
    cu = i32([0] + torch.tensor(counts).cumsum(0).tolist())
    lane_of_token = i32([lane for lane, count in enumerate(counts) for _ in range(count)])
    wide = rand(T, 8 + C + H + 4, seed=90, dtype=torch.bfloat16).to(DEV)
    raw, dt = wide[:, 8:8 + C], wide[:, 8 + C:8 + C + H]
    weight, conv_bias = rand(C, K, seed=91, scale=0.5).to(DEV), (rand(C, seed=92).to(DEV) if bias else None)
    tails = rand(slots, K - 1, C, seed=93, dtype=torch.bfloat16).to(DEV)
    dt_bias, A, D = gpu(rand(H, seed=94) - 1.0, -torch.exp(torch.linspace(-3.0, 1.0, H)), rand(H, seed=95))
    state = rand(slots, H, P, N, seed=96, scale=0.5).to(DEV)
    table = ops.SsdChunks(counts, Q, DEV)
    ids, cu, lane_of_token = gpu(slot_ids, cu, lane_of_token)
    # the separate kernels
    want_xbc, want_tails, want_state = torch.empty(T, C, dtype=torch.bfloat16, device=DEV), tails.clone(), state.clone()
    ops.conv1d_silu(wide, 8, C, weight, conv_bias, want_tails, lane_of_token, cu, ids, want_xbc)
    ops.conv_state_update(wide, 8, C, K, want_tails, cu, ids)
    want_y = torch.empty(T, E, device=DEV)
    ops.ssd_prefill(want_xbc, dt, dt_bias, A, D, want_state, table, ids, G, want_y)
    # the conv inside
    assert ops.ssd_conv_supported(K, C, raw)
    got_xbc, got_tails, got_state = torch.full_like(want_xbc, float("nan")), tails.clone(), state.clone()
    got_y = torch.empty(T, E, device=DEV)
    ops.ssd_prefill(got_xbc, dt, dt_bias, A, D, got_state, table, ids, G, got_y,
                    conv=dict(u=raw, weight=weight, bias=conv_bias, state=got_tails))
    # the same sums in another order of fused multiply-adds: a last bit of bfloat16 may differ here and there
    assert (got_xbc.float() - want_xbc.float()).abs().max().item() <= 2.0 ** -7 * want_xbc.float().abs().max().item()
    assert (got_xbc != want_xbc).float().mean().item() < 1e-3
    assert torch.equal(got_tails, want_tails)
    close(got_y, want_y.cpu(), torch.bfloat16, max(1.0, want_y.abs().max().item()) * 0.1)
    close(got_state, want_state.cpu(), torch.bfloat16, max(1.0, want_state.abs().max().item()) * 0.1)
    # and both against the plain conv
    plain_xbc, plain_tails = torch.empty(T, C, dtype=torch.bfloat16), tails.cpu().clone()
    ref_ops.conv1d_silu(wide.cpu(), 8, C, weight.cpu(), None if conv_bias is None else conv_bias.cpu(), plain_tails,
                        lane_of_token.cpu(), cu.cpu(), slot_ids, plain_xbc)
    close(got_xbc, plain_xbc, torch.bfloat16, 4.0)


def test_chunked_scan_carries_a_far_token_through_many_chunks(ops):
    """One token with a large x and a head that barely decays: 600 tokens later its state is what
    the output consists of; every chunk boundary between must pass it on."""
    H, P, N, G, Q = 4, 16, 32, 1, 32
    E, T = H * P, 640
    xbc = rand(T, E + 2 * N, seed=90, dtype=torch.bfloat16) * 0.05
    xbc[3, :E] = 8.0
    xbc[3, E:E + N] = 1.0
    xbc[T - 1, E + N:] = 1.0
    dt = torch.zeros(T, H, dtype=torch.bfloat16)
    dt_bias, A, D = torch.zeros(H), -torch.tensor([1e-4, 1e-3, 1e-2, 1.0]), torch.zeros(H)
    want_y, want_state = torch.empty(T, E), torch.zeros(1, H, P, N)
    ref_ops.ssm_scan(xbc, dt, dt_bias, A, D, want_state, i32([0, T]), i32([0]), G, want_y)
    assert want_y[T - 1, 0].item() > 50.0          # head 0 still holds the token
    y, state = torch.empty(T, E, device=DEV), torch.zeros(1, H, P, N, device=DEV)
    ops.ssd_prefill(xbc.to(DEV), dt.to(DEV), *gpu(dt_bias, A, D), state, ops.SsdChunks([T], Q, DEV), i32([0]).to(DEV),
                    G, y)
    close(y[T - 1:], want_y[T - 1:], torch.bfloat16, want_y[T - 1].abs().max().item())
    close(state, want_state, torch.bfloat16, want_state.abs().max().item())


def test_chunked_scan_refuses_sizes_it_does_not_take(ops):
    assert not ops.ssd_supported(48, 16, 32, 1, 64)       # chunk not a multiple of 32
    assert not ops.ssd_supported(32, 8, 32, 1, 64)        # head size not a multiple of 16
    assert not ops.ssd_supported(32, 16, 24, 1, 64)       # state size not a multiple of 32
    assert not ops.ssd_supported(512, 16, 32, 1, 64)
    with pytest.raises(ops.KernelError, match="size not supported"):
        ops.ssd_prefill(torch.zeros(4, 16 + 48, device=DEV, dtype=torch.bfloat16),
                        torch.zeros(4, 1, device=DEV, dtype=torch.bfloat16), torch.zeros(1, device=DEV),
                        torch.zeros(1, device=DEV), torch.zeros(1, device=DEV), torch.zeros(1, 1, 16, 24, device=DEV),
                        ops.SsdChunks([4], 32, DEV), i32([0]).to(DEV), 1, torch.zeros(4, 16, device=DEV))


def test_scan_refuses_a_state_size_beyond_its_limit(ops):
    with pytest.raises(ops.KernelError, match="size not supported"):
        ops.ssm_scan(torch.zeros(1, 1 + 2 * 600, device=DEV), torch.zeros(1, 1, device=DEV), torch.zeros(1, device=DEV),
                     torch.zeros(1, device=DEV), torch.zeros(1, device=DEV), torch.zeros(1, 1, 1, 600, device=DEV),
                     i32([0, 1]).to(DEV), i32([0]).to(DEV), 1, torch.zeros(1, 1, device=DEV))


def test_softplus_is_stable_in_the_scan(ops):
    """dt = +-100 (the fixture of crates/macllm-kernels/src/mamba2.rs:561-565)."""
    H, P, N = 2, 4, 8
    xbc = rand(3, H * P + 2 * N, seed=70)
    dt = torch.tensor([[100.0, -100.0], [0.2, -0.7], [-100.0, 100.0]])
    args = [torch.zeros(H), -torch.ones(H) * 0.03, torch.ones(H)]
    state = rand(1, H, P, N, seed=71)
    want_y, want_state = torch.empty(3, H * P), state.clone()
    ref_ops.ssm_scan(xbc, dt, *args, want_state, i32([0, 3]), i32([0]), 1, want_y)
    y, dev_state = torch.empty(3, H * P, device=DEV), state.to(DEV)
    ops.ssm_scan(xbc.to(DEV), dt.to(DEV), *gpu(*args), dev_state, i32([0, 3]).to(DEV), i32([0]).to(DEV), 1, y)
    close(y, want_y, torch.float32, 30.0)
    close(dev_state, want_state, torch.float32, 30.0)


def test_tokens_fed_on_the_device(ops):
    """token_ids[dst] = source[src] for 1, 64 and 150 pairs (more than a launch carries); places not named keep
    their values; an index outside either vector is refused before anything is launched."""
    generator = torch.Generator().manual_seed(5)
    for count in (1, 64, 150):
        token_ids = torch.arange(1000, 1000 + 400, dtype=torch.int32)
        source = torch.randint(0, 30000, (200,), generator=generator, dtype=torch.int32)
        dst = torch.randperm(400, generator=generator)[:count].tolist()
        src = torch.randint(0, 200, (count,), generator=generator).tolist()
        want = token_ids.clone()
        ref_ops.feed_tokens(want, source, dst, src)
        got = token_ids.to(DEV)
        ops.feed_tokens(got, source.to(DEV), dst, src)
        assert torch.equal(got.cpu(), want)
    with pytest.raises(ops.KernelError):
        ops.feed_tokens(got, source.to(DEV), [400], [0])
    with pytest.raises(ops.KernelError):
        ops.feed_tokens(got, source.to(DEV), [0], [200])
    assert torch.equal(got.cpu(), want)


# ------------------------------------------------------------------ sampling
def test_argmax_and_ties(ops):
    logits = rand(5, 1003, seed=80)
    logits[1, 17] = logits[1, 900] = 9.0                         # a tie: the lower index wins
    logits[2, 1002] = 11.0
    out = torch.empty(5, dtype=torch.int32, device=DEV)
    ops.argmax(logits.to(DEV), out)
    assert out.cpu().tolist() == torch.argmax(logits, -1).tolist()
    assert out.cpu()[1] == 17 and out.cpu()[2] == 1002


@pytest.mark.parametrize("V", [3, 130049, 32784, 8191])
def test_argmax_of_rows_at_every_alignment(ops, V):
    """Rows of an odd width start at every alignment of the 16-byte pieces the kernel reads: the best element
    is put, row by row, at the row's first and last elements, around the first aligned piece and far inside;
    a tie between two pieces goes to the lower index."""
    places = sorted({0, 1, 2, 3, 4, 5, V // 2, V - 5, V - 4, V - 3, V - 2, V - 1} & set(range(V)))
    logits = rand(len(places) + 1, V, seed=81)
    for row, place in enumerate(places):
        logits[row, place] = 50.0
    logits[-1, V - 1] = logits[-1, V // 3] = 60.0
    out = torch.empty(len(places) + 1, dtype=torch.int32, device=DEV)
    ops.argmax(logits.to(DEV), out)
    assert out.cpu().tolist() == places + [min(V // 3, V - 1)]


@pytest.mark.parametrize("select", [False, True], ids=["sorted", "selected"])
@pytest.mark.parametrize("V", [320, 1003, 32784])
def test_sampling_matches_the_plain_sampler(ops, V, select):
    """Every row is sorted whole, or (``select``) rows are drawn by selection where that covers
    them: top-k 1, 7, 20, 40 and 1 024; a nucleus that closes within the 1 024 best candidates
    (rows with peaked logits) and one that does not (flat logits: its last token by a select over mass);
    top-k above 1 024 (handed on to the full sort); neither top-k nor top-p; a greedy row."""
    import plain_impl
    settings = [(0.8, 0, 1.0), (1.0, 7, 1.0), (0.9, 0, 0.7), (1.2, 40, 0.85), (0.0, 0, 1.0), (0.7, 20, 0.8),
                (1.0, V + 5, 0.999), (0.5, 1, 0.1), (1.0, 1024, 0.95), (1.1, 1500, 0.9), (0.6, 0, 0.9), (1.0, 0, 0.5)]
    B = len(settings)
    logits = rand(B, V, seed=81, scale=2.5)
    logits[10] *= 4.0                                            # peaked: the nucleus is a handful of tokens
    logits[11] *= 0.02                                           # flat: half the mass is half the vocabulary
    seeds = [3, 99, 2 ** 63 + 5, 42, 0, 7, 11, 13, 17, 19, 23, 29]
    draws = [0, 5, 17, 3, 0, 100, 1, 2, 8, 9, 10, 11]
    padded = 1
    while padded < V:
        padded <<= 1
    for repeat in range(3):
        work = logits.clone().to(DEV)
        out = torch.empty(B, dtype=torch.int32, device=DEV)
        signed = [s - (1 << 64) if s >= (1 << 63) else s for s in seeds]
        ops.sample(work, torch.tensor([s[0] for s in settings]).to(DEV), i32([s[1] for s in settings]).to(DEV),
                   torch.tensor([s[2] for s in settings]).to(DEV), torch.tensor(signed, dtype=torch.int64).to(DEV),
                   i32([d + repeat for d in draws]).to(DEV),
                   torch.empty(B, padded, dtype=torch.int64, device=DEV), out,
                   torch.full((B,), 7, dtype=torch.int32, device=DEV) if select else None)
        want = [plain_impl.sample_token(logits[row], temperature=settings[row][0], top_k=settings[row][1],
                                        top_p=settings[row][2], seed=seeds[row], draw_index=draws[row] + repeat)
                for row in range(B)]
        assert out.cpu().tolist() == want


@pytest.mark.parametrize("V", [5000, 40001])
def test_a_nucleus_wider_than_the_candidates(ops, V):
    """Top-p without top-k over flat rows, where the nucleus is thousands of tokens (more than the 1 024
    candidates that are sorted): nearly equal logits, logits that are all equal (the nucleus is cut among
    ties, by index; more ties than the list of the select holds), two values half and half, an ordinary
    row at a high temperature; several draws each.

    Over thousands of nearly equal masses the order in which float32 sums are taken moves a running sum by
    more than one token's mass (the plain sampler adds one by one, a GPU adds in blocks), so tokens are not
    compared one to one here: the drawn token must be a valid draw of the rule computed in float64: it lies in
    the nucleus (the shortest descending prefix, ties by index, whose mass reaches top_p; one token of slack at
    its end), and u times the kept mass falls into the token's own interval of the running sum in index order,
    give or take V float32 roundings of the total."""
    import numpy as np
    import plain_impl
    settings = [(1.0, 0.5), (1.0, 0.9), (0.7, 0.999), (1.0, 0.25), (1.3, 0.6), (5.0, 0.95), (1.0, 0.0)]
    B = len(settings)
    logits = rand(B, V, seed=83, scale=0.02)
    logits[1] = 0.25                                             # all equal
    logits[3, :V // 2] = 1.0                                     # two values
    logits[3, V // 2:] = 0.0
    logits[5] = rand(V, seed=84, scale=3.0)
    logits[6] = rand(V, seed=85, scale=3.0)                      # top_p 0: the best token alone
    padded = 1
    while padded < V:
        padded <<= 1
    drawn = set()
    for repeat in range(4):
        work = logits.clone().to(DEV)
        out = torch.empty(B, dtype=torch.int32, device=DEV)
        ops.sample(work, torch.tensor([s[0] for s in settings]).to(DEV), i32([0] * B).to(DEV),
                   torch.tensor([s[1] for s in settings]).to(DEV), torch.tensor([31 + row for row in range(B)], dtype=torch.int64).to(DEV),
                   i32([repeat * 7 + row for row in range(B)]).to(DEV),
                   torch.empty(B, padded, dtype=torch.int64, device=DEV), out,
                   torch.full((B,), 7, dtype=torch.int32, device=DEV))
        tokens = out.cpu().tolist()
        for row, (temperature, top_p) in enumerate(settings):
            scaled = (logits[row].numpy() / np.float32(temperature)).astype(np.float64)
            mass = np.exp(scaled - scaled.max())
            mass /= mass.sum()
            order = sorted(range(V), key=lambda index: (-mass[index], index))
            running = np.cumsum(mass[order])
            keep = int(np.searchsorted(running, top_p, side="left")) + 1          # the first prefix that reaches top_p
            token = tokens[row]
            place = order.index(token)
            assert place < min(V, keep + 1), (row, repeat, token, place, keep)
            kept = np.zeros(V)
            kept[order[:keep]] = mass[order[:keep]]
            upto = np.cumsum(kept)
            target = plain_impl.draw_uniform(31 + row, repeat * 7 + row) * upto[-1]
            slack = V * 2.0 ** -23 * upto[-1] + mass[order[min(keep, V - 1)]]
            assert upto[token] - kept[token] - slack <= target <= upto[token] + slack, (row, repeat, token)
            drawn.add((row, token))
    assert tokens[6] == int(torch.argmax(logits[6]))
    assert len(drawn) > 3 * B                                    # the draws differ from one another


def test_penalties_match_the_plain_rule(ops):
    V = 500
    logits = rand(3, V, seed=82)
    histories = [[5, 9, 5, 400, 9, 9], [], [1, 2, 3, 499]]
    prompt_lens = [2, 0, 4]
    flat = [token for history in histories for token in history]
    offsets = [0, 6, 6, 10]
    rep, pres, freq = [1.3, 1.0, 2.0], [0.5, 0.0, 0.0], [0.25, 0.0, 0.3]
    want = logits.clone()
    ref_ops.apply_penalties(want, i32(flat), i32(offsets), i32(prompt_lens), torch.tensor(rep), torch.tensor(pres),
                            torch.tensor(freq), None, None)
    got = logits.clone().to(DEV)
    counts = [torch.zeros(3 * V, dtype=torch.int32, device=DEV) for _ in range(2)]
    ops.apply_penalties(got, i32(flat).to(DEV), i32(offsets).to(DEV), i32(prompt_lens).to(DEV),
                        torch.tensor(rep).to(DEV), torch.tensor(pres).to(DEV), torch.tensor(freq).to(DEV), *counts)
    close(got, want, torch.float32)
    assert not torch.equal(want, logits) and int(counts[0].sum()) == 0 and int(counts[1].sum()) == 0
    # a row's newest token still on the device: it counts as if it closed the row's history
    source, extra_rows = i32([9, 77, 400, 3]), i32([2, -1, 1])
    longer = [histories[0] + [400], histories[1], histories[2] + [77]]
    want = logits.clone()
    ref_ops.apply_penalties(want, i32([token for history in longer for token in history]), i32([0, 7, 7, 12]),
                            i32(prompt_lens), torch.tensor(rep), torch.tensor(pres), torch.tensor(freq), None, None)
    fed = logits.clone()
    ref_ops.apply_penalties(fed, i32(flat), i32(offsets), i32(prompt_lens), torch.tensor(rep), torch.tensor(pres),
                            torch.tensor(freq), None, None, source, extra_rows)
    assert torch.equal(fed, want)
    got = logits.clone().to(DEV)
    ops.apply_penalties(got, i32(flat).to(DEV), i32(offsets).to(DEV), i32(prompt_lens).to(DEV),
                        torch.tensor(rep).to(DEV), torch.tensor(pres).to(DEV), torch.tensor(freq).to(DEV), *counts,
                        source.to(DEV), extra_rows.to(DEV))
    close(got, want, torch.float32)
    assert int(counts[0].sum()) == 0 and int(counts[1].sum()) == 0


def test_allowed_tokens_keep_their_logits_and_the_rest_is_minus_infinity(ops):
    """Rows with a list keep exactly the listed logits (a list may name a token twice, and the last and the first of
    a vocabulary that is no multiple of anything); a row without one is untouched; argmax then takes the best
    allowed token, the lower index on ties."""
    V = 1031
    logits = rand(4, V, seed=91)
    logits[2, 17] = logits[2, 800] = 50.0                       # a tie among the allowed ones
    lists = [[0, 5, 1030, 5], [], [800, 17, 3], [1030]]
    offsets, flat = [0], []
    for allowed in lists:
        flat += allowed
        offsets.append(len(flat))
    want = logits.clone()
    ref_ops.keep_allowed(want, i32(flat), i32(offsets), None)
    got = logits.clone().to(DEV)
    keep = torch.full((4, 2048), 7, dtype=torch.int64, device=DEV)            # the sampler's work area, dirty
    ops.keep_allowed(got, i32(flat).to(DEV), i32(offsets).to(DEV), keep)
    assert torch.equal(got.cpu(), want)
    assert torch.equal(want[1], logits[1]) and int(torch.isfinite(want[0]).sum()) == 3 and int(torch.isfinite(want[3]).sum()) == 1
    out = torch.empty(4, dtype=torch.int32, device=DEV)
    ops.argmax(got, out)
    assert out.cpu().tolist() == [max((0, 5, 1030), key=lambda token: float(logits[0, token])), int(logits[1].argmax()), 17, 1030]
    with pytest.raises(ops.KernelError):
        ops.keep_allowed(got, i32(flat).to(DEV), i32(offsets).to(DEV), torch.empty((4, 500), dtype=torch.float32, device=DEV))


# ------------------------------------------------------------------ decode attention (split over the context)
@pytest.mark.parametrize("Hq, Hkv, dh, page_size, window", [(8, 2, 64, 16, None), (12, 2, 128, 16, None),
                                                              (5, 5, 64, 8, None), (8, 1, 128, 64, None),
                                                              (8, 2, 64, 16, 300), (4, 2, 64, 32, 40)])
def test_decode_attention_over_ragged_contexts(ops, Hq, Hkv, dh, page_size, window):
    """Single decoded tokens of requests with contexts of 1 to 2 500 keys, cut into splits of
    different sizes; NaN in every cell that is not a request's; against the plain reference."""
    dtype = torch.bfloat16
    lengths = [1, 2, 15, 16, 17, 63, 64, 65, 129, 777, 2500, 1024]
    pool, table = paged_setup(lengths, page_size, Hkv, dh, dtype, seed=9)
    for lane, length in enumerate(lengths):
        fill_cache(pool, table, lane, rand(length, Hkv, dh, seed=100 + lane, dtype=dtype),
                   rand(length, Hkv, dh, seed=200 + lane, dtype=dtype), page_size)
    T = len(lengths)
    q = rand(T, Hq * dh, seed=90, dtype=dtype)
    positions = i32([length - 1 for length in lengths])
    lane_of_token = torch.arange(T, dtype=torch.int32)
    want = torch.empty(T, Hq * dh, dtype=dtype)
    ref_ops.paged_attention(q, Hq, Hkv, dh, *views(pool, page_size), table, lane_of_token, positions, 0.11, window, want)
    dev_pool = pool.to(DEV)
    assert ops.decode_attention_supported(dtype, Hq, Hkv, dh, page_size)
    for subset in (list(range(T)), [10], [0, 10, 3]):            # different batch sizes pick different splits
        got = torch.empty(len(subset), Hq * dh, dtype=dtype, device=DEV)
        ops.decode_attention(q[subset].to(DEV), Hq, Hkv, dh, *views(dev_pool, page_size), table.to(DEV),
                             i32(subset).to(DEV), positions[subset].to(DEV), 0.11, window,
                             max(lengths[index] for index in subset), got)
        close(got, want[subset], dtype, 2.0)


def test_decode_attention_finds_one_far_key(ops):
    Hq, Hkv, dh, length, page_size = 8, 2, 64, 2048, 16
    dtype = torch.bfloat16
    pool, table = paged_setup([length], page_size, Hkv, dh, dtype, seed=5)
    values = rand(length, Hkv, dh, seed=54, dtype=dtype)
    direction = torch.zeros(dh)
    direction[9] = 1.0
    q = (direction * 30.0).repeat(Hq)[None].to(dtype).to(DEV)
    for chosen in (0, 15, 16, 255, 256, 257, 1023, 1024, 2046, 2047):
        keys = rand(length, Hkv, dh, seed=55, scale=0.1, dtype=dtype)
        keys[chosen] = (direction * 30.0).to(dtype)
        fill_cache(pool, table, 0, keys, values, page_size)
        out = torch.empty(1, Hq * dh, dtype=dtype, device=DEV)
        ops.decode_attention(q, Hq, Hkv, dh, *views(pool.to(DEV), page_size), table.to(DEV), i32([0]).to(DEV),
                             i32([length - 1]).to(DEV), 1.0 / math.sqrt(dh), None, length, out)
        expected = values[chosen].float()[[0] * 4 + [1] * 4].reshape(-1)
        assert (out.float().cpu()[0] - expected).abs().max() < 1e-2, f"key {chosen} was missed"


# ------------------------------------------------------------------ fused decode kernels
@pytest.mark.parametrize("M, N, K", [(1, 48, 64), (8, 4120, 1024), (5, 100, 96), (16, 250, 1024), (33, 64, 256),
                                     (64, 130, 2048), (48, 4128, 1024), (20, 80, 3072)])
def test_fused_gemm_plain_prologue(ops, M, N, K):
    """Plain and SwiGLU epilogues behind rows given in bfloat16, with one, two and four tiles of 16 output
    features a workgroup (a last workgroup with tiles past the end included)."""
    x = rand(M, K + 8, seed=300, dtype=torch.bfloat16)[:, :K]            # a row stride
    W, b = rand(N, K, seed=301, scale=0.1, dtype=torch.bfloat16), rand(N, seed=302)
    for feature_tiles in (1, 2, 4):
        for out_dtype, scale, bias in ((torch.bfloat16, 1.0, b), (torch.float32, 0.6, None)):
            want = torch.empty(M, N, dtype=out_dtype)
            ref_ops.fused_gemm(W, bias, want, x=x, out_scale=scale)
            got = torch.full((M, N), float("nan"), dtype=out_dtype, device=DEV)
            ops.fused_gemm(W.to(DEV), None if bias is None else bias.to(DEV), got, x=x.to(DEV), out_scale=scale,
                           feature_tiles=feature_tiles)
            close(got, want, out_dtype, 6.0 if out_dtype == torch.bfloat16 else 200.0)
            again = torch.full((M, N), float("nan"), dtype=out_dtype, device=DEV)        # the weight in fragment order
            ops.fused_gemm(W.to(DEV), None if bias is None else bias.to(DEV), again, x=x.to(DEV), out_scale=scale,
                           feature_tiles=feature_tiles, fragments=ops.fragment_order(W.to(DEV)))
            assert torch.equal(again, got)
        if N % 16 == 0:
            want = torch.empty(M, N // 2, dtype=torch.bfloat16)
            ref_ops.fused_gemm(W, b, want, x=x, epilogue=ref_ops.EPI_SWIGLU)
            got = torch.full((M, N // 2), float("nan"), dtype=torch.bfloat16, device=DEV)
            ops.fused_gemm(W.to(DEV), b.to(DEV), got, x=x.to(DEV), epilogue=ops.EPI_SWIGLU, feature_tiles=feature_tiles)
            close(got, want, torch.bfloat16, 16.0)
    assert ops.fused_gemm_supported(False, M, K) and not ops.fused_gemm_supported(False, 65, K)
    assert not ops.fused_gemm_supported(False, M, K + 8)


@pytest.mark.parametrize("M, N, K, deltas", [(1, 64, 64, 0), (8, 160, 1024, 2), (13, 48, 96, 1), (16, 4120, 1024, 2),
                                             (8, 272, 3072, 2), (3, 80, 5120, 1), (5, 64, 3072, 0)])
def test_fused_gemm_norm_prologue_and_epilogues(ops, M, N, K, deltas):
    """Only the step's own rows are staged in LDS: 8 rows of 3,072 and 3 of 5,120 fit where 16 would not."""
    h = rand(M, K, seed=310)
    ds = [rand(M, K, seed=311 + i, dtype=torch.bfloat16) for i in range(deltas)]
    norm_w = rand(K, seed=314, scale=0.1) + 1.0
    W, b = rand(N, K, seed=315, scale=0.1, dtype=torch.bfloat16), rand(N, seed=316)
    assert ops.fused_gemm_supported(True, M, K)
    # plain
    want, want_h = torch.empty(M, N, dtype=torch.bfloat16), torch.empty(M, K)
    ref_ops.fused_gemm(W, b, want, h_in=h, deltas=ds, h_out=want_h, norm_weight=norm_w, eps=3e-6)
    got, got_h = torch.empty(M, N, dtype=torch.bfloat16, device=DEV), torch.full((M, K), float("nan"), device=DEV)
    ops.fused_gemm(W.to(DEV), b.to(DEV), got, h_in=h.to(DEV), deltas=gpu(*ds), h_out=got_h, norm_weight=norm_w.to(DEV),
                   eps=3e-6)
    close(got, want, torch.bfloat16, 8.0)
    close(got_h, want_h, torch.float32)
    again = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device=DEV)           # the weight in fragment order
    ops.fused_gemm(W.to(DEV), b.to(DEV), again, h_in=h.to(DEV), deltas=gpu(*ds), norm_weight=norm_w.to(DEV), eps=3e-6,
                   fragments=ops.fragment_order(W.to(DEV)))
    assert torch.equal(again, got)
    # swiglu (tiles of 8 gate rows + 8 up rows)
    if N % 16 == 0:
        want = torch.empty(M, N // 2, dtype=torch.bfloat16)
        ref_ops.fused_gemm(W, b, want, h_in=h, deltas=ds, norm_weight=norm_w, eps=3e-6, epilogue=ref_ops.EPI_SWIGLU)
        got = torch.empty(M, N // 2, dtype=torch.bfloat16, device=DEV)
        ops.fused_gemm(W.to(DEV), b.to(DEV), got, h_in=h.to(DEV), deltas=gpu(*ds), norm_weight=norm_w.to(DEV),
                       eps=3e-6, epilogue=ops.EPI_SWIGLU)
        close(got, want, torch.bfloat16, 16.0)
    # conv rows in the middle, taps 1..4, shuffled slots (one slot untouched)
    lo, hi = 16, N - 8
    for taps in (4, 3, 1):
        C = hi - lo
        state = rand(M + 2, max(taps - 1, 0), C, seed=320, dtype=torch.bfloat16)
        slot_ids = torch.randperm(M + 2, generator=torch.Generator().manual_seed(taps))[:M].to(torch.int32)
        conv = dict(lo=lo, hi=hi, taps=taps, weight=rand(C, taps, seed=321, scale=0.5), bias=rand(C, seed=322, scale=0.1))
        want_state, got_state = state.clone(), state.clone().to(DEV)
        want = torch.empty(M, N, dtype=torch.bfloat16)
        ref_ops.fused_gemm(W, b, want, h_in=h, deltas=ds, norm_weight=norm_w, eps=3e-6, epilogue=ref_ops.EPI_CONV,
                           conv=dict(conv, state=want_state, slot_ids=slot_ids))
        got = torch.empty(M, N, dtype=torch.bfloat16, device=DEV)
        ops.fused_gemm(W.to(DEV), b.to(DEV), got, h_in=h.to(DEV), deltas=gpu(*ds), norm_weight=norm_w.to(DEV), eps=3e-6,
                       epilogue=ops.EPI_CONV,
                       conv=dict(lo=lo, hi=hi, taps=taps, weight=conv["weight"].to(DEV), bias=conv["bias"].to(DEV),
                                 state=got_state, slot_ids=slot_ids.to(DEV)))
        close(got, want, torch.bfloat16, 8.0)
        close(got_state, want_state, torch.bfloat16, 8.0)
        unused = [slot for slot in range(M + 2) if slot not in slot_ids.tolist()]
        assert torch.equal(got_state[unused].cpu(), state[unused])


@pytest.mark.parametrize("M, N, K, N2", [(8, 1024, 2048, 4120), (1, 72, 64, 48), (13, 1000, 96, 160), (16, 3072, 4608, 272),
                                         (40, 200, 2048, 96), (40, 256, 2048, 96), (24, 96, 64, 80), (64, 1024, 2048, 272),
                                         (48, 1024, 2048, 136), (33, 136, 96, 4120)])
def test_a_product_that_joins_the_residual_stream_and_the_product_behind_the_next_norm(ops, M, N, K, N2):
    """``fused_gemm_residual``: h += x . W^T + b in float32 in place, with the new rows times the next norm's
    weight in bfloat16 and the partial sums of their squares; then ``fused_gemm`` with that row scale against the
    norm written out (the division of the root mean square applied to the rows, then the product), plain, with
    the SwiGLU epilogue and with the conv step; a width that is no multiple of 16, 1 to 64 rows.  Every workgroup
    with all of the step's rows, and the rows dealt out to two and to four workgroups per tile of features (the
    same bits into the stream; nothing written beside the table of partial sums, whose guard rows stay as
    they were)."""
    x = rand(M, K, seed=350, dtype=torch.bfloat16)
    W, b = rand(N, K, seed=351, scale=0.1, dtype=torch.bfloat16), rand(N, seed=352)
    h = rand(M, N, seed=353, scale=2.0)
    next_w = rand(N, seed=354, scale=0.1) + 1.0
    want_h, want_hb, want_ssq = h.clone(), torch.empty(M, N, dtype=torch.bfloat16), ops.residual_workspace(M, N, "cpu")
    ref_ops.fused_gemm_residual(W, b, x, want_h, want_hb, next_w, want_ssq)
    assert torch.allclose(want_h, h + x.float() @ W.float().T + b, atol=1e-4)
    blocks, columns = want_ssq.shape
    first = None
    for fragments in (None, ops.fragment_order(W.to(DEV))):
        for row_tiles in (1, 2, 4):
            got_h, got_hb = h.clone().to(DEV), torch.full((M, N), float("nan"), dtype=torch.bfloat16, device=DEV)
            guarded = torch.full((blocks + 2, columns), float("nan"), device=DEV)       # a row of guards on either side
            got_ssq = guarded[1:-1]
            ops.fused_gemm_residual(W.to(DEV), b.to(DEV), x.to(DEV), got_h, got_hb, next_w.to(DEV), got_ssq, fragments,
                                    row_tiles=row_tiles)
            close(got_h, want_h, torch.float32, max(1.0, want_h.abs().max().item()))
            close(got_hb, want_hb, torch.bfloat16, max(1.0, want_hb.float().abs().max().item()))
            assert torch.allclose(got_ssq[:, :M].cpu(), want_ssq[:, :M], rtol=1e-4, atol=1e-4)
            assert torch.isnan(guarded[0]).all() and torch.isnan(guarded[-1]).all()
            if first is None:
                first = (got_h.clone(), got_hb.clone(), got_ssq[:, :M].clone())
            else:
                assert all(torch.equal(a, b_) for a, b_ in zip(first, (got_h, got_hb, got_ssq[:, :M])))
    got_ssq = got_ssq.contiguous()
    # the product behind the norm: rows = h / rms(h) * w, rounded to bfloat16
    eps = 3e-5
    normed = (want_h / torch.sqrt(want_h.pow(2).mean(-1, keepdim=True) + eps) * next_w)
    W2, b2 = rand(N2, N, seed=355, scale=0.1, dtype=torch.bfloat16), rand(N2, seed=356)
    scale = ops.RowScale(got_ssq, N, eps)
    if N % 32 == 0 and M <= 64:
        want = normed @ W2.float().T + b2
        again = torch.empty(M, N2, dtype=torch.bfloat16)
        ref_ops.fused_gemm(W2, b2, again, x=got_hb.cpu(), row_scale=ops.RowScale(got_ssq.cpu(), N, eps))
        for row_tiles in (1, 2, 4):
            got = torch.full((M + 1, N2), float("nan"), dtype=torch.bfloat16, device=DEV)
            ops.fused_gemm(W2.to(DEV), b2.to(DEV), got[:M], x=got_hb, row_scale=scale, row_tiles=row_tiles)
            assert torch.isnan(got[M].float()).all()
            close(got[:M], want, torch.bfloat16, 3.0 * max(1.0, want.abs().max().item()))
            close(got[:M], again, torch.bfloat16, max(1.0, want.abs().max().item()))
        if N2 % 16 == 0:
            want = torch.empty(M, N2 // 2, dtype=torch.bfloat16)
            ref_ops.fused_gemm(W2, b2, want, x=got_hb.cpu(), row_scale=ops.RowScale(got_ssq.cpu(), N, eps), epilogue=ref_ops.EPI_SWIGLU)
            got = torch.empty(M, N2 // 2, dtype=torch.bfloat16, device=DEV)
            ops.fused_gemm(W2.to(DEV), b2.to(DEV), got, x=got_hb, row_scale=scale, epilogue=ops.EPI_SWIGLU,
                           feature_tiles=2 if M > 16 else 1)
            close(got, want, torch.bfloat16, 16.0)
            for row_tiles in (2, 4):
                got = torch.empty(M, N2 // 2, dtype=torch.bfloat16, device=DEV)
                ops.fused_gemm(W2.to(DEV), b2.to(DEV), got, x=got_hb, row_scale=scale, epilogue=ops.EPI_SWIGLU,
                               row_tiles=row_tiles)
                close(got, want, torch.bfloat16, 16.0)


@pytest.mark.parametrize("M, N, K, S", [(64, 1024, 2048, 8), (33, 100, 2048, 16), (17, 48, 96, 3), (64, 136, 3072, 5),
                                        (5, 64, 64, 1)])
def test_fused_gemm_split_over_k_and_the_norm_that_adds_its_slabs(ops, M, N, K, S):
    """Partial sums over runs of K in float32 slabs (the bias in the first), then the residual add
    of all slabs with the norm, against the plain product and norm."""
    x = rand(M, K + 16, seed=340, dtype=torch.bfloat16)[:, :K]
    W, b = rand(N, K, seed=341, scale=0.1, dtype=torch.bfloat16), rand(N, seed=342)
    want = torch.zeros(S, M, N)
    ref_ops.fused_gemm_split(W, b, x, want)
    for feature_tiles in (4, 2, 1):
        got = torch.full((S, M, N), float("nan"), device=DEV)
        ops.fused_gemm_split(W.to(DEV), b.to(DEV), x.to(DEV), got, feature_tiles=feature_tiles)
        close(got, want, torch.float32, 50.0)
        again = torch.full((S, M, N), float("nan"), device=DEV)
        ops.fused_gemm_split(W.to(DEV), b.to(DEV), x.to(DEV), again, feature_tiles=feature_tiles,
                             fragments=ops.fragment_order(W.to(DEV)))
        assert torch.equal(again, got)
    whole = x.float() @ W.float().T + b
    close(got.sum(0), whole, torch.float32, 200.0)
    if N % 4 == 0:
        h, weight = rand(M, N, seed=343), rand(N, seed=344, scale=0.1) + 1.0
        want_h, want_out = h.clone(), torch.empty(M, N, dtype=torch.bfloat16)
        ref_ops.add_partials_rmsnorm(want_h, want, weight, 3e-6, want_out)
        got_h, got_out = h.clone().to(DEV), torch.empty(M, N, dtype=torch.bfloat16, device=DEV)
        ops.add_partials_rmsnorm(got_h, got, weight.to(DEV), 3e-6, got_out)
        close(got_h, want_h, torch.float32, 50.0)
        close(got_out, want_out, torch.bfloat16, 4.0)
        again = h.clone().to(DEV)
        ops.add_partials_rmsnorm(again, got, weight.to(DEV), 3e-6, None)           # the sum alone
        assert torch.equal(again, got_h)


@pytest.mark.parametrize("M, N, K, S", [(64, 1024, 2048, 8), (33, 100, 2048, 16), (48, 138, 1056, 3), (49, 72, 3072, 5),
                                        (64, 50, 128, 1), (40, 272, 288, 8), (57, 16, 4672, 64), (17, 40, 160, 2), (32, 264, 1024, 4),
                                        (65, 100, 160, 2), (96, 272, 1056, 4), (113, 48, 4672, 16), (128, 1024, 2048, 8),
                                        (1, 72, 160, 3), (8, 1024, 2048, 8), (16, 100, 1056, 4), (5, 40, 128, 1)])
def test_fused_gemm_split_with_the_rows_shared_by_a_workgroups_waves(ops, M, N, K, S):
    """The slabs of the kernel whose waves own feature tiles and share the rows through LDS: widths with a last
    tile of fewer than 16 features and rows that are no multiple of four floats, a K whose last stage is short or
    is moved back over chunks already multiplied, more slabs than stages, slabs without chunks, row-major
    weights and the fragment order, against the plain product per slab and the unshared kernel's slabs; 65 to
    128 rows (6 and 8 tiles of rows, one tile of features a wave), which only this kernel takes."""
    x = rand(M, K + 24, seed=350, dtype=torch.bfloat16)[:, :K]
    W, b = rand(N, K, seed=351, scale=0.1, dtype=torch.bfloat16), rand(N, seed=352)
    want = torch.zeros(S, M, N)
    ref_ops.fused_gemm_split(W, b, x, want)
    other = torch.full((S, M, N), float("nan"), device=DEV)
    if M <= 64:
        ops.fused_gemm_split(W.to(DEV), b.to(DEV), x.to(DEV), other)
    else:
        other = want.to(DEV)
        with pytest.raises((ValueError, RuntimeError)):
            ops.fused_gemm_split(W.to(DEV), b.to(DEV), x.to(DEV), torch.empty((S, M, N), device=DEV), feature_tiles=2,
                                 shared_rows=True)
    for feature_tiles in (1, 2) if M <= 64 else (1,):
        got = torch.full((S, M, N), float("nan"), device=DEV)
        ops.fused_gemm_split(W.to(DEV), b.to(DEV), x.to(DEV), got, feature_tiles=feature_tiles, shared_rows=True)
        close(got, want, torch.float32, 50.0)
        close(got, other.cpu(), torch.float32, 50.0)
        again = torch.full((S, M, N), float("nan"), device=DEV)
        ops.fused_gemm_split(W.to(DEV), None, x.to(DEV), again, feature_tiles=feature_tiles,
                             fragments=ops.fragment_order(W.to(DEV)), shared_rows=True)
        again[0] += b.to(DEV)
        close(again, got.cpu(), torch.float32, 2.0)


@pytest.mark.parametrize("M, N, K, scaled", [(64, 1024, 2048, False), (33, 112, 1056, True), (48, 272, 128, True),
                                             (17, 48, 288, False), (57, 4112, 160, True), (32, 16, 4672, True),
                                             (1, 112, 160, True), (8, 1024, 2048, False), (16, 272, 1056, True)])
def test_fused_gemm_swiglu_with_the_rows_shared_by_a_workgroups_waves(ops, M, N, K, scaled):
    """SiLU(gate) * up from the kernel whose waves own feature tiles and share the rows through LDS, with and
    without the row scale of a norm left to it, one and two tiles a wave, row-major weights and the fragment
    order, a last workgroup with waves that own no tile, an output whose rows are no multiple of four columns
    apart: against the plain product and the skinny kernel's result."""
    x = rand(M, K + 8, seed=360, dtype=torch.bfloat16)[:, :K]
    W, b = rand(N, K, seed=361, scale=0.1, dtype=torch.bfloat16), rand(N, seed=362)
    width, eps = 520, 2e-5
    ssq = rand(width // 16 + 1, 16 * (-(-M // 16)), seed=363).abs() * 3.0 if scaled else None
    want = torch.empty(M, N // 2, dtype=torch.bfloat16)
    ref_ops.fused_gemm(W, b, want, x=x, epilogue=ref_ops.EPI_SWIGLU, row_scale=ops.RowScale(ssq, width, eps) if scaled else None)
    scale = ops.RowScale(ssq.to(DEV), width, eps) if scaled else None
    skinny = torch.empty(M, N // 2, dtype=torch.bfloat16, device=DEV)
    ops.fused_gemm(W.to(DEV), b.to(DEV), skinny, x=x.to(DEV), epilogue=ops.EPI_SWIGLU, row_scale=scale)
    for feature_tiles in (1, 2):
        for fragments in (None, ops.fragment_order(W.to(DEV))):
            for pad in (0, 3):
                got = torch.full((M, N // 2 + pad), float("nan"), dtype=torch.bfloat16, device=DEV)[:, :N // 2]
                ops.fused_gemm(W.to(DEV), b.to(DEV), got, x=x.to(DEV), epilogue=ops.EPI_SWIGLU, row_scale=scale,
                               feature_tiles=feature_tiles, fragments=fragments, shared_rows=True)
                close(got, want, torch.bfloat16, 16.0)
                close(got, skinny.cpu(), torch.bfloat16, max(2.0, want.float().abs().max().item() / 4))   # an ulp of the largest, between two orders of summation
    for rows, k, tiles in ((65, 256, 1), (40, 96, 1), (40, 256, 4)):
        weight = torch.zeros(32, k, dtype=torch.bfloat16, device=DEV)
        out = torch.zeros(rows, 16, dtype=torch.bfloat16, device=DEV)
        with pytest.raises((ValueError, RuntimeError)):
            ops.fused_gemm(weight, None, out, x=torch.zeros(rows, k, dtype=torch.bfloat16, device=DEV),
                           epilogue=ops.EPI_SWIGLU, feature_tiles=tiles, shared_rows=True)


def test_fused_gemm_split_with_the_rows_shared_refuses_other_sizes(ops):
    """More than 128 rows, a K below one stage of 128 columns, four tiles a wave: an error, and nothing
    written."""
    for rows, K, tiles in ((129, 256, 1), (40, 96, 1), (40, 256, 4)):
        W = torch.zeros(48, K, dtype=torch.bfloat16, device=DEV)
        x = torch.zeros(rows, K, dtype=torch.bfloat16, device=DEV)
        partial = torch.full((1, rows, 48), 7.0, device=DEV)
        with pytest.raises((ValueError, RuntimeError)):
            ops.fused_gemm_split(W, None, x, partial, feature_tiles=tiles, shared_rows=True)
        assert bool((partial == 7.0).all())


@pytest.mark.parametrize("M, N, K", [(24, 200, 1024), (64, 136, 1024), (7, 96, 2048), (64, 88, 3072), (40, 64, 64)])
def test_fused_gemm_conv_step_of_wide_batches(ops, M, N, K):
    """The conv epilogue behind the plain prologue: more than one tile of 16 rows, four and eight
    waves (K beyond 1,024), taps the prefetched path holds (2..4) and more than it holds (6); every workgroup
    with all the rows, and the rows dealt out to two or four workgroups per tile of features (each rolls the
    tails of its own rows' slots only)."""
    x = rand(M, K, seed=330, dtype=torch.bfloat16)
    W, b = rand(N, K, seed=331, scale=0.1, dtype=torch.bfloat16), rand(N, seed=332)
    lo, hi = 8, N - 24
    for taps, feature_tiles, row_tiles in ((4, 1, 1), (2, 1, 1), (6, 1, 1), (4, 2, 1), (3, 4, 1), (6, 4, 1), (4, 1, 4), (3, 1, 2),
                                           (6, 1, 4)):
        C = hi - lo
        state = rand(M + 3, taps - 1, C, seed=333, dtype=torch.bfloat16)
        slot_ids = torch.randperm(M + 3, generator=torch.Generator().manual_seed(taps))[:M].to(torch.int32)
        conv = dict(lo=lo, hi=hi, taps=taps, weight=rand(C, taps, seed=334, scale=0.5), bias=rand(C, seed=335, scale=0.1))
        want_state, got_state = state.clone(), state.clone().to(DEV)
        want = torch.empty(M, N, dtype=torch.bfloat16)
        ref_ops.fused_gemm(W, b, want, x=x, epilogue=ref_ops.EPI_CONV, conv=dict(conv, state=want_state, slot_ids=slot_ids))
        got = torch.empty(M, N, dtype=torch.bfloat16, device=DEV)
        ops.fused_gemm(W.to(DEV), b.to(DEV), got, x=x.to(DEV), epilogue=ops.EPI_CONV, feature_tiles=feature_tiles,
                       row_tiles=row_tiles,
                       conv=dict(lo=lo, hi=hi, taps=taps, weight=conv["weight"].to(DEV), bias=conv["bias"].to(DEV),
                                 state=got_state, slot_ids=slot_ids.to(DEV)))
        close(got, want, torch.bfloat16, 8.0)
        close(got_state, want_state, torch.bfloat16, 8.0)
        unused = [slot for slot in range(M + 3) if slot not in slot_ids.tolist()]
        assert torch.equal(got_state[unused].cpu(), state[unused])
    with pytest.raises((ValueError, RuntimeError)):            # rows dealt out: one tile of features a workgroup only
        ops.fused_gemm(W.to(DEV), b.to(DEV), torch.empty(M, N, dtype=torch.bfloat16, device=DEV), x=x.to(DEV),
                       feature_tiles=2, row_tiles=2)


@pytest.mark.parametrize("M, N, K", [(24, 200, 1024), (64, 136, 1056), (17, 96, 128), (49, 90, 3072), (40, 1048, 160),
                                     (1, 96, 160), (7, 200, 1024), (16, 136, 288)])
def test_fused_gemm_conv_step_with_the_rows_shared_by_a_workgroups_waves(ops, M, N, K):
    """The conv epilogue of the kernel whose waves own feature tiles and share the rows through LDS: taps 1 to 6,
    a width that is no multiple of 16 or 4, conv columns that start and end inside a lane's four, with the row
    scale of a norm left to the product and without, padded output rows; and plain rows in bfloat16 (no conv
    column) times a scale.  Against the plain reference, rolled tails included."""
    x = rand(M, K + 8, seed=370, dtype=torch.bfloat16)[:, :K]
    W, b = rand(N, K, seed=371, scale=0.1, dtype=torch.bfloat16), rand(N, seed=372)
    lo, hi = 6, N - 21
    C = hi - lo
    width, eps = 264, 3e-5
    ssq = rand(width // 16, 16 * (-(-M // 16)), seed=373).abs() * 2.0
    for taps, feature_tiles, scaled in ((4, 1, False), (2, 2, True), (6, 1, True), (1, 2, False), (3, 1, True)):
        state = rand(M + 3, taps - 1, C, seed=374, dtype=torch.bfloat16)
        slot_ids = torch.randperm(M + 3, generator=torch.Generator().manual_seed(taps))[:M].to(torch.int32)
        conv = dict(lo=lo, hi=hi, taps=taps, weight=rand(C, taps, seed=375, scale=0.5), bias=rand(C, seed=376, scale=0.1))
        want_state, got_state = state.clone(), state.clone().to(DEV)
        want = torch.empty(M, N, dtype=torch.bfloat16)
        ref_ops.fused_gemm(W, b, want, x=x, epilogue=ref_ops.EPI_CONV, conv=dict(conv, state=want_state, slot_ids=slot_ids),
                           row_scale=ops.RowScale(ssq, width, eps) if scaled else None)
        got = torch.full((M, N + 5), float("nan"), dtype=torch.bfloat16, device=DEV)[:, :N]
        ops.fused_gemm(W.to(DEV), b.to(DEV), got, x=x.to(DEV), epilogue=ops.EPI_CONV, feature_tiles=feature_tiles,
                       shared_rows=True, fragments=ops.fragment_order(W.to(DEV)) if taps % 2 else None,
                       row_scale=ops.RowScale(ssq.to(DEV), width, eps) if scaled else None,
                       conv=dict(lo=lo, hi=hi, taps=taps, weight=conv["weight"].to(DEV), bias=conv["bias"].to(DEV),
                                 state=got_state, slot_ids=slot_ids.to(DEV)))
        close(got, want, torch.bfloat16, 8.0)
        close(got_state, want_state, torch.bfloat16, 8.0)
        unused = [slot for slot in range(M + 3) if slot not in slot_ids.tolist()]
        assert torch.equal(got_state[unused].cpu(), state[unused])
    want = torch.empty(M, N, dtype=torch.bfloat16)
    ref_ops.fused_gemm(W, b, want, x=x, out_scale=0.7)
    for feature_tiles in (1, 2):
        got = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device=DEV)
        ops.fused_gemm(W.to(DEV), b.to(DEV), got, x=x.to(DEV), out_scale=0.7, feature_tiles=feature_tiles, shared_rows=True)
        close(got, want, torch.bfloat16, 8.0)
    with pytest.raises((ValueError, RuntimeError)):                     # float32 rows are the slabs' entry's
        ops.fused_gemm(W.to(DEV), None, torch.empty(M, N, device=DEV), x=x.to(DEV), shared_rows=True)


@pytest.mark.parametrize("Hq, Hkv, dh, H, P, N, G, page_size, window, rotary, gated", [
    (8, 2, 64, 24, 64, 128, 1, 16, None, 64, False), (12, 2, 128, 6, 40, 256, 2, 16, None, 128, True),
    (4, 4, 64, 3, 24, 40, 3, 8, 100, 32, False), (8, 1, 64, 5, 7, 9, 1, 32, None, 0, False)])
def test_mixer_decode_against_the_separate_kernels(ops, Hq, Hkv, dh, H, P, N, G, page_size, window, rotary, gated):
    """Both mixers of a decode step in one launch, for requests with contexts of 1 to 1 500
    tokens; compared with the composition of the plain references, cache and state included.
    Twice in a row on fresh copies of the cache and state."""
    dtype = torch.bfloat16
    lengths = [1, 17, 64, 65, 300, 1500, 2]
    M = len(lengths)
    pool, table = paged_setup(lengths, page_size, Hkv, dh, dtype, seed=11)
    for lane, length in enumerate(lengths):          # everything before the new token is cached already
        fill_cache(pool, table, lane, rand(length, Hkv, dh, seed=400 + lane, dtype=dtype),
                   rand(length, Hkv, dh, seed=500 + lane, dtype=dtype), page_size)
    E, GN = H * P, G * N
    q_col, k_col, v_col = 0, Hq * dh, (Hq + Hkv) * dh
    z_col = (Hq + 2 * Hkv) * dh
    x_col, dt_col = z_col + E, z_col + 2 * E + 2 * GN
    u = rand(M, -(-(dt_col + H) // 8) * 8, seed=410, dtype=dtype)      # rows 16-byte aligned
    positions = i32([length - 1 for length in lengths])
    slot_mapping = i32([int(table[lane, (length - 1) // page_size]) * page_size + (length - 1) % page_size
                        for lane, length in enumerate(lengths)])
    inv_freq = None if rotary == 0 else torch.tensor([1.0 / (1e4 ** (i / rotary)) for i in range(0, rotary, 2)],
                                                      dtype=torch.float64).float()
    slots = M + 1
    slot_ids = torch.randperm(slots, generator=torch.Generator().manual_seed(5))[:M].to(torch.int32)
    state = rand(slots, H, P, N, seed=411, scale=0.5)
    dt_bias, A, D = rand(H, seed=412) - 2.0, -(rand(H, seed=413).abs() + 0.1), rand(H, seed=414)
    common = dict(num_heads=Hq, num_kv_heads=Hkv, head_dim=dh, q_col=q_col, k_col=k_col, v_col=v_col,
                  rotary_dim=rotary, scale=0.11, window=window, max_seq_len=2048, ssm_heads=H, ssm_head_dim=P,
                  state_size=N, num_groups=G, z_col=z_col, x_col=x_col, dt_col=dt_col)
    want_pool, want_state = pool.clone(), state.clone()
    want_out = torch.zeros(M, Hq * dh + E, dtype=dtype)
    want_y = torch.empty(M, E) if gated else None
    ref_ops.mixer_decode(u, inv_freq=inv_freq, k_cache=views(want_pool, page_size)[0], v_cache=views(want_pool, page_size)[1],
                         block_tables=table, positions=positions, slot_mapping=slot_mapping,
                         dt_bias=dt_bias, A=A, D=D, ssm_state=want_state, slot_ids=slot_ids, out=want_out, ssm_y=want_y,
                         **common)
    assert ops.mixer_decode_supported(Hq, Hkv, dh, page_size, N, 2048, window, rotary)
    for repeat in range(2):
        got_pool, got_state = pool.clone().to(DEV), state.clone().to(DEV)
        got_out = torch.zeros(M, Hq * dh + E, dtype=dtype, device=DEV)
        got_y = torch.empty(M, E, device=DEV) if gated else None
        ops.mixer_decode(u.to(DEV), inv_freq=None if inv_freq is None else inv_freq.to(DEV),
                         k_cache=views(got_pool, page_size)[0], v_cache=views(got_pool, page_size)[1],
                         block_tables=table.to(DEV), positions=positions.to(DEV), slot_mapping=slot_mapping.to(DEV),
                         dt_bias=dt_bias.to(DEV), A=A.to(DEV), D=D.to(DEV), ssm_state=got_state,
                         slot_ids=slot_ids.to(DEV), out=got_out, ssm_y=got_y, **common)
        close(got_out[:, :Hq * dh], want_out[:, :Hq * dh], dtype, 2.0)
        scale = max(1.0, want_state.abs().max().item())
        close(got_state, want_state, torch.float32, scale)
        if gated:
            close(got_y, want_y, torch.float32, max(1.0, want_y.abs().max().item()))
        else:
            close(got_out[:, Hq * dh:], want_out[:, Hq * dh:], dtype, max(1.0, want_out.float().abs().max().item()))
        assert torch.equal(torch.isnan(got_pool.float().cpu()), torch.isnan(want_pool.float()))
        close(torch.nan_to_num(got_pool.float()), torch.nan_to_num(want_pool.float()), dtype, 4.0)


@pytest.mark.parametrize("M, Hq, Hkv, dh, H, P, N, G", [(40, 8, 2, 64, 24, 64, 128, 1), (48, 12, 2, 128, 24, 128, 256, 1),
                                                      (64, 4, 2, 64, 12, 32, 64, 3), (30, 4, 2, 64, 20, 24, 128, 2)])
def test_mixer_decode_of_wide_batches(ops, M, Hq, Hkv, dh, H, P, N, G):
    """So many single-token lanes that a state-space workgroup takes several rows per thread group
    (and rows of more than one head where a head has few): the state sizes of the benchmark shapes,
    a head size that is no multiple of a workgroup's rows, groups of heads."""
    dtype = torch.bfloat16
    page_size = 16
    lengths = [1 + (7 * lane) % 45 for lane in range(M)]
    pool, table = paged_setup(lengths, page_size, Hkv, dh, dtype, seed=13)
    for lane, length in enumerate(lengths):
        fill_cache(pool, table, lane, rand(length, Hkv, dh, seed=600 + lane, dtype=dtype),
                   rand(length, Hkv, dh, seed=700 + lane, dtype=dtype), page_size)
    E, GN = H * P, G * N
    q_col, k_col, v_col = 0, Hq * dh, (Hq + Hkv) * dh
    z_col = (Hq + 2 * Hkv) * dh
    x_col, dt_col = z_col + E, z_col + 2 * E + 2 * GN
    u = rand(M, -(-(dt_col + H) // 8) * 8, seed=610, dtype=dtype)
    positions = i32([length - 1 for length in lengths])
    slot_mapping = i32([int(table[lane, (length - 1) // page_size]) * page_size + (length - 1) % page_size
                        for lane, length in enumerate(lengths)])
    inv_freq = torch.tensor([1.0 / (1e4 ** (i / dh)) for i in range(0, dh, 2)], dtype=torch.float64).float()
    slot_ids = torch.randperm(M + 2, generator=torch.Generator().manual_seed(6))[:M].to(torch.int32)
    state = rand(M + 2, H, P, N, seed=611, scale=0.5)
    dt_bias, A, D = rand(H, seed=612) - 2.0, -(rand(H, seed=613).abs() + 0.1), rand(H, seed=614)
    common = dict(num_heads=Hq, num_kv_heads=Hkv, head_dim=dh, q_col=q_col, k_col=k_col, v_col=v_col,
                  rotary_dim=dh, scale=0.11, window=None, max_seq_len=64, ssm_heads=H, ssm_head_dim=P,
                  state_size=N, num_groups=G, z_col=z_col, x_col=x_col, dt_col=dt_col)
    want_pool, want_state = pool.clone(), state.clone()
    want_out = torch.zeros(M, Hq * dh + E, dtype=dtype)
    ref_ops.mixer_decode(u, inv_freq=inv_freq, k_cache=views(want_pool, page_size)[0], v_cache=views(want_pool, page_size)[1],
                         block_tables=table, positions=positions, slot_mapping=slot_mapping, dt_bias=dt_bias, A=A, D=D,
                         ssm_state=want_state, slot_ids=slot_ids, out=want_out, ssm_y=None, **common)
    got_pool, got_state = pool.clone().to(DEV), state.clone().to(DEV)
    got_out = torch.zeros(M, Hq * dh + E, dtype=dtype, device=DEV)
    ops.mixer_decode(u.to(DEV), inv_freq=inv_freq.to(DEV), k_cache=views(got_pool, page_size)[0],
                     v_cache=views(got_pool, page_size)[1], block_tables=table.to(DEV), positions=positions.to(DEV),
                     slot_mapping=slot_mapping.to(DEV), dt_bias=dt_bias.to(DEV), A=A.to(DEV), D=D.to(DEV),
                     ssm_state=got_state, slot_ids=slot_ids.to(DEV), out=got_out, ssm_y=None, **common)
    close(got_out[:, :Hq * dh], want_out[:, :Hq * dh], dtype, 2.0)
    close(got_state, want_state, torch.float32, max(1.0, want_state.abs().max().item()))
    close(got_out[:, Hq * dh:], want_out[:, Hq * dh:], dtype, max(1.0, want_out.float().abs().max().item()))
    unused = [slot for slot in range(M + 2) if slot not in slot_ids.tolist()]
    assert torch.equal(got_state[unused].cpu(), state[unused])


@pytest.mark.parametrize("Hq, Hkv, dh, E, N_out, window, lengths", [
    (8, 2, 64, 1536, 1024, None, [1, 17, 64, 65, 300, 1500, 2, 2060]),
    (4, 2, 64, 96, 200, 40, [1, 17, 64, 65, 300, 1500, 2]),
    (12, 2, 128, 512, 320, None, [700, 3]),
    (4, 4, 64, 64, 48, None, [5000, 9000, 3] + [40 + lane for lane in range(13)]),
])
def test_output_projection_that_merges_the_runs_of_keys(ops, Hq, Hkv, dh, E, N_out, window, lengths):
    """``mixer_decode(merge=False)`` followed by ``fused_gemm_merge`` gives bit for bit what ``mixer_decode``,
    its merge kernel and ``fused_gemm`` give: contexts of one run and of more runs than a merge asks for at
    once, 16 rows, a K beyond 1 024; with a window of one run there is nothing to merge and ``mixer_decode``
    writes the heads itself.  The attended columns of x hold NaN where nobody may read them."""
    dtype = torch.bfloat16
    H, P, N, G, page_size = E // 32, 32, 32, 1, 16
    M = len(lengths)
    pool, table = paged_setup(lengths, page_size, Hkv, dh, dtype, seed=21)
    for lane, length in enumerate(lengths):
        fill_cache(pool, table, lane, rand(length, Hkv, dh, seed=800 + lane, dtype=dtype),
                   rand(length, Hkv, dh, seed=900 + lane, dtype=dtype), page_size)
    q_col, k_col, v_col = 0, Hq * dh, (Hq + Hkv) * dh
    z_col = (Hq + 2 * Hkv) * dh
    x_col, dt_col = z_col + E, z_col + 2 * E + 2 * G * N
    u = rand(M, -(-(dt_col + H) // 8) * 8, seed=810, dtype=dtype).to(DEV)
    positions = i32([length - 1 for length in lengths]).to(DEV)
    slot_mapping = i32([int(table[lane, (length - 1) // page_size]) * page_size + (length - 1) % page_size
                        for lane, length in enumerate(lengths)]).to(DEV)
    inv_freq = torch.tensor([1.0 / (1e4 ** (i / dh)) for i in range(0, dh, 2)], dtype=torch.float64).float().to(DEV)
    state = rand(M, H, P, N, seed=811, scale=0.5)
    vectors = [rand(H, seed=812) - 2.0, -(rand(H, seed=813).abs() + 0.1), rand(H, seed=814)]
    K = Hq * dh + E
    weight, bias = rand(N_out, K, seed=815, scale=0.05, dtype=dtype).to(DEV), rand(N_out, seed=816).to(DEV)

    def run(merge):
        dev_pool = pool.clone().to(DEV)
        mixed = torch.full((M, K), float("nan"), dtype=dtype, device=DEV)
        runs = ops.mixer_decode(u, num_heads=Hq, num_kv_heads=Hkv, head_dim=dh, q_col=q_col, k_col=k_col, v_col=v_col,
                                inv_freq=inv_freq, rotary_dim=dh, k_cache=views(dev_pool, page_size)[0],
                                v_cache=views(dev_pool, page_size)[1], block_tables=table.to(DEV), positions=positions,
                                slot_mapping=slot_mapping, scale=0.13, window=window, max_seq_len=max(lengths) + 5,
                                ssm_heads=H, ssm_head_dim=P, state_size=N, num_groups=G, z_col=z_col, x_col=x_col,
                                dt_col=dt_col, dt_bias=vectors[0].to(DEV), A=vectors[1].to(DEV), D=vectors[2].to(DEV),
                                ssm_state=state.clone().to(DEV), slot_ids=i32(list(range(M))).to(DEV), out=mixed,
                                ssm_y=None, merge=merge)
        return mixed, runs

    mixed, nothing = run(True)
    assert nothing is None and not torch.isnan(mixed.float()).any()
    want = torch.empty(M, N_out, dtype=dtype, device=DEV)
    ops.fused_gemm(weight, bias, want, x=mixed)
    unmerged, runs = run(False)
    if window is not None:           # a window of 40 keys is one run: its workgroup writes the heads itself, nothing is left over
        assert runs is None and torch.equal(unmerged, mixed)
        return
    assert torch.isnan(unmerged[:, :Hq * dh].float()).all() and torch.equal(unmerged[:, Hq * dh:], mixed[:, Hq * dh:])
    assert ops.fused_gemm_merge_supported(M, K, Hq, dh)
    for fragments in (None, ops.fragment_order(weight)):
        got = torch.empty(M, N_out, dtype=dtype, device=DEV)
        ops.fused_gemm_merge(weight, bias, got, unmerged, runs, fragments)
        assert torch.equal(got, want)
    # and the same with the result added to the residual stream: what ``fused_gemm_residual`` gives on the merged rows
    h, next_w = rand(M, N_out, seed=817, scale=2.0).to(DEV), (rand(N_out, seed=818, scale=0.1) + 1.0).to(DEV)
    want_h, want_rows = h.clone(), torch.empty(M, N_out, dtype=dtype, device=DEV)
    want_ssq = ops.residual_workspace(M, N_out, DEV)
    ops.fused_gemm_residual(weight, bias, mixed, want_h, want_rows, next_w, want_ssq)
    got_h, got_rows = h.clone(), torch.empty(M, N_out, dtype=dtype, device=DEV)
    got_ssq = ops.residual_workspace(M, N_out, DEV)
    ops.fused_gemm_merge(weight, bias, None, unmerged, runs, None, residual=(got_h, got_rows, next_w, got_ssq))
    assert torch.equal(got_h, want_h) and torch.equal(got_rows, want_rows)
    assert torch.equal(got_ssq[:, :M], want_ssq[:, :M])
    product = mixed.float().cpu() @ weight.float().cpu().T + bias.cpu()
    close(want, product, dtype, max(1.0, product.abs().max().item()))


def test_mixer_decode_over_a_long_context(ops):
    """Contexts of 5 000 and 9 000 tokens (more runs of keys than the merge takes
    at once) beside a short one; one far key per long request is made to dominate, so a run that
    is dropped or merged with the wrong weight shows."""
    dtype = torch.bfloat16
    Hq, Hkv, dh, H, P, N, G, page_size = 4, 2, 64, 2, 16, 32, 1, 16
    lengths = [5000, 9000, 3]
    M = len(lengths)
    pool, table = paged_setup(lengths, page_size, Hkv, dh, dtype, seed=12)
    E = H * P
    q_col, k_col, v_col = 0, Hq * dh, (Hq + Hkv) * dh
    z_col = (Hq + 2 * Hkv) * dh
    x_col, dt_col = z_col + E, z_col + 2 * E + 2 * G * N
    u = rand(M, -(-(dt_col + H) // 8) * 8, seed=420, dtype=dtype)
    for lane, length in enumerate(lengths):
        keys = rand(length, Hkv, dh, seed=430 + lane, dtype=dtype)
        values = rand(length, Hkv, dh, seed=440 + lane, dtype=dtype)
        if length > 1000:                                    # key 700 looks like the query of head 0 / 2
            for kvh in range(Hkv):
                keys[700, kvh] = u[lane, q_col + kvh * (Hq // Hkv) * dh:q_col + kvh * (Hq // Hkv) * dh + dh] * 3.0
            values[700] = 5.0
        fill_cache(pool, table, lane, keys, values, page_size)
    positions = i32([length - 1 for length in lengths])
    slot_mapping = i32([int(table[lane, (length - 1) // page_size]) * page_size + (length - 1) % page_size
                        for lane, length in enumerate(lengths)])
    slot_ids = i32([2, 0, 1])
    state = rand(M + 1, H, P, N, seed=421, scale=0.5)
    dt_bias, A, D = rand(H, seed=422) - 2.0, -(rand(H, seed=423).abs() + 0.1), rand(H, seed=424)
    common = dict(num_heads=Hq, num_kv_heads=Hkv, head_dim=dh, q_col=q_col, k_col=k_col, v_col=v_col, inv_freq=None,
                  rotary_dim=0, scale=0.125, window=None, max_seq_len=9216, ssm_heads=H, ssm_head_dim=P,
                  state_size=N, num_groups=G, z_col=z_col, x_col=x_col, dt_col=dt_col)
    want_pool, want_state = pool.clone(), state.clone()
    want_out = torch.zeros(M, Hq * dh + E, dtype=dtype)
    ref_ops.mixer_decode(u, k_cache=views(want_pool, page_size)[0], v_cache=views(want_pool, page_size)[1],
                         block_tables=table, positions=positions, slot_mapping=slot_mapping, dt_bias=dt_bias, A=A, D=D,
                         ssm_state=want_state, slot_ids=slot_ids, out=want_out, ssm_y=None, **common)
    assert want_out[0, :dh].float().mean() > 3.0             # the far key does dominate head 0
    got_pool, got_state = pool.clone().to(DEV), state.clone().to(DEV)
    got_out = torch.zeros(M, Hq * dh + E, dtype=dtype, device=DEV)
    ops.mixer_decode(u.to(DEV), k_cache=views(got_pool, page_size)[0], v_cache=views(got_pool, page_size)[1],
                     block_tables=table.to(DEV), positions=positions.to(DEV), slot_mapping=slot_mapping.to(DEV),
                     dt_bias=dt_bias.to(DEV), A=A.to(DEV), D=D.to(DEV), ssm_state=got_state,
                     slot_ids=slot_ids.to(DEV), out=got_out, ssm_y=None, **common)
    close(got_out, want_out, dtype, max(1.0, want_out.float().abs().max().item()))


# ------------------------------------------------------------------ prefill attention on the matrix cores
@pytest.mark.parametrize("Hq, Hkv, dh, page_size, window", [(8, 2, 64, 16, None), (4, 4, 128, 16, None),
                                                              (12, 2, 64, 4, None), (5, 1, 64, 64, None),
                                                              (8, 2, 64, 16, 100), (6, 2, 128, 8, 33)])
def test_prefill_attention_on_the_matrix_cores(ops, Hq, Hkv, dh, page_size, window):
    """A prompt portion that continues a cached prefix, a fresh prompt longer than one tile, a
    two-token portion and single tokens, in one batch; every unwritten cache cell holds NaN."""
    dtype = torch.bfloat16
    starts, counts = [37, 0, 500, 129, 0], [83, 150, 2, 1, 1]
    lengths = [s + c for s, c in zip(starts, counts)]
    pool, table = paged_setup(lengths, page_size, Hkv, dh, dtype, seed=21)
    T = sum(counts)
    keys, values = {}, {}
    for lane, length in enumerate(lengths):          # the whole context, the step's own tokens included
        keys[lane] = rand(length, Hkv, dh, seed=600 + lane, dtype=dtype)
        values[lane] = rand(length, Hkv, dh, seed=700 + lane, dtype=dtype)
        fill_cache(pool, table, lane, keys[lane], values[lane], page_size)
    q = rand(T, Hq * dh + 16, seed=610, dtype=dtype)
    positions = torch.cat([torch.arange(s, s + c) for s, c in zip(starts, counts)]).to(torch.int32)
    lane_of_token = torch.repeat_interleave(torch.arange(len(counts)), torch.tensor(counts)).to(torch.int32)
    cu = torch.zeros(len(counts) + 1, dtype=torch.int32)
    cu[1:] = torch.cumsum(torch.tensor(counts), 0)
    tiles = i32([(lane, row) for lane in range(len(counts)) for row in range(int(cu[lane]), int(cu[lane + 1]), 64)])
    want = torch.empty(T, Hq * dh, dtype=dtype)
    ref_ops.paged_attention(q, Hq, Hkv, dh, *views(pool, page_size), table, lane_of_token, positions, 0.21, window, want)
    assert ops.prefill_attention_supported(dtype, Hq, Hkv, dh, page_size)
    for bound in (0, 600, 4096):                 # of the longest context: it picks how many heads share a key fragment
        got = torch.full((T, Hq * dh), float("nan"), dtype=dtype, device=DEV)
        ops.prefill_attention(q.to(DEV), Hq, Hkv, dh, *views(pool.to(DEV), page_size), table.to(DEV), tiles.to(DEV),
                              cu.to(DEV), i32(starts).to(DEV), 0.21, window, got, bound)
        close(got, want, dtype, 2.0)


@pytest.mark.parametrize("Hq, Hkv, dh", [(8, 2, 64), (12, 2, 64), (3, 1, 64), (4, 2, 128)])
def test_prefill_attention_many_short_portions(ops, Hq, Hkv, dh):
    """130 requests with portions of one to three tokens after prefixes of different lengths: a grid large
    enough for the widest sets of query heads that share a key fragment (few tiles take narrower sets)."""
    dtype, page_size = torch.bfloat16, 16
    generator = torch.Generator().manual_seed(77)
    counts = torch.randint(1, 4, (130,), generator=generator).tolist()
    starts = torch.randint(0, 90, (130,), generator=generator).tolist()
    lengths = [s + c for s, c in zip(starts, counts)]
    pool, table = paged_setup(lengths, page_size, Hkv, dh, dtype, seed=22)
    for lane, length in enumerate(lengths):
        fill_cache(pool, table, lane, rand(length, Hkv, dh, seed=800 + lane, dtype=dtype),
                   rand(length, Hkv, dh, seed=1000 + lane, dtype=dtype), page_size)
    T = sum(counts)
    q = rand(T, Hq * dh, seed=611, dtype=dtype)
    positions = torch.cat([torch.arange(s, s + c) for s, c in zip(starts, counts)]).to(torch.int32)
    lane_of_token = torch.repeat_interleave(torch.arange(len(counts)), torch.tensor(counts)).to(torch.int32)
    cu = torch.zeros(len(counts) + 1, dtype=torch.int32)
    cu[1:] = torch.cumsum(torch.tensor(counts), 0)
    tiles = i32([(lane, int(cu[lane])) for lane in range(len(counts))])
    want = torch.empty(T, Hq * dh, dtype=dtype)
    ref_ops.paged_attention(q, Hq, Hkv, dh, *views(pool, page_size), table, lane_of_token, positions, 0.17, None, want)
    got = torch.full((T, Hq * dh), float("nan"), dtype=dtype, device=DEV)
    ops.prefill_attention(q.to(DEV), Hq, Hkv, dh, *views(pool.to(DEV), page_size), table.to(DEV), tiles.to(DEV),
                          cu.to(DEV), i32(starts).to(DEV), 0.17, None, got)
    close(got, want, dtype, 2.0)


def test_prefill_attention_finds_far_keys_and_edges(ops):
    """Queries at the end of a 700-token prompt; one chosen key takes all the weight."""
    Hq, Hkv, dh, length, page_size = 4, 2, 64, 700, 16
    dtype = torch.bfloat16
    pool, table = paged_setup([length], page_size, Hkv, dh, dtype, seed=6)
    values = rand(length, Hkv, dh, seed=56, dtype=dtype)
    direction = torch.zeros(dh)
    direction[3] = 1.0
    T = 20
    q = (direction * 30.0).repeat(Hq)[None].repeat(T, 1).to(dtype).to(DEV)
    tiles = i32([(0, 0)])
    for chosen in (0, 1, 15, 16, 31, 32, 33, 511, 512, 679, 680, 698):
        keys = rand(length, Hkv, dh, seed=57, scale=0.1, dtype=dtype)
        keys[chosen] = (direction * 30.0).to(dtype)
        fill_cache(pool, table, 0, keys, values, page_size)
        out = torch.empty(T, Hq * dh, dtype=dtype, device=DEV)
        ops.prefill_attention(q, Hq, Hkv, dh, *views(pool.to(DEV), page_size), table.to(DEV), tiles.to(DEV),
                              i32([0, T]).to(DEV), i32([length - T]).to(DEV), 1.0 / math.sqrt(dh), None, out)
        expected = values[chosen].float()[[0, 0, 1, 1]].reshape(-1)
        for row in range(T):
            position = length - T + row
            hit = (out.float().cpu()[row] - expected).abs().max() < 1e-2
            assert hit == (chosen <= position), f"key {chosen}, query at {position}"
