"""The entry point that allocates nothing (``mi_decode_attention_static``), called through ctypes as a
caller without an allocator would: its output against that of ``mi_decode_attention`` (whose partial results
go to a workspace the caller allocates) on two calls in a row, the second with a smaller input, and its
refusal of a step whose partial results do not fit the static array."""
import ctypes

import pytest
import torch

from test_gpu_kernels import DEV, fill_cache, i32, paged_setup, rand, views

pytestmark = pytest.mark.gpu


def _splits(T, Hkv, page_size, span):
    """The split of the context that ``ops.decode_attention`` chooses."""
    split_keys = 64
    while split_keys < 512 and span * T * Hkv > 1024 * split_keys:
        split_keys *= 2
    split_keys = max(split_keys, page_size)
    return split_keys, max(1, -(-span // split_keys))


def test_decode_attention_from_the_static_array_matches_the_one_with_a_workspace():
    from macllm_infer_amd.kernels import build, ops
    ops.require_gpu(DEV)
    library = build.load_module("attention")
    static = library.mi_decode_attention_static
    c_int, c_long, c_float, c_ptr = ctypes.c_int, ctypes.c_long, ctypes.c_float, ctypes.c_void_p
    static.argtypes = [c_ptr, c_long, c_int, c_int, c_int, c_int, c_ptr, c_ptr, c_long, c_int, c_ptr, c_int, c_ptr,
                       c_ptr, c_float, c_int, c_int, c_int, c_ptr, c_long, c_ptr]
    static.restype = c_int
    library.mi_static_scratch_bytes.restype = c_long
    capacity = library.mi_static_scratch_bytes()
    assert capacity == 8 << 20

    Hq, Hkv, dh, page_size = 8, 2, 64, 16
    dtype = torch.bfloat16
    lengths = [1, 17, 64, 65, 129, 777, 2500, 1024]
    pool, table = paged_setup(lengths, page_size, Hkv, dh, dtype, seed=9)
    for lane, length in enumerate(lengths):
        fill_cache(pool, table, lane, rand(length, Hkv, dh, seed=100 + lane, dtype=dtype),
                   rand(length, Hkv, dh, seed=200 + lane, dtype=dtype), page_size)
    q = rand(len(lengths), Hq * dh, seed=90, dtype=dtype)
    positions = i32([length - 1 for length in lengths])
    dev_pool, dev_table = pool.to(DEV), table.to(DEV)
    k_cache, v_cache = views(dev_pool, page_size)
    stream = torch.cuda.current_stream().cuda_stream

    def both(subset, first_call=False):
        T = len(subset)
        queries, lanes, places = q[subset].to(DEV), i32(subset).to(DEV), positions[subset].to(DEV)
        longest = max(lengths[index] for index in subset)
        want = torch.empty(T, Hq * dh, dtype=dtype, device=DEV)
        ops.decode_attention(queries, Hq, Hkv, dh, k_cache, v_cache, dev_table, lanes, places, 0.11, None, longest, want)
        got = torch.full((T, Hq * dh), float("nan"), dtype=dtype, device=DEV)
        split_keys, splits = _splits(T, Hkv, page_size, longest)
        torch.cuda.synchronize()
        # the device's own count of free bytes (torch's counters see only torch's allocator: a hipMalloc inside
        # the library would pass them); the first call on a device may load the code object and resolve the symbol
        before, free_before = torch.cuda.memory_allocated(), torch.cuda.mem_get_info()[0]
        code = static(queries.data_ptr(), queries.stride(0), T, Hq, Hkv, dh, k_cache.data_ptr(), v_cache.data_ptr(),
                      k_cache.stride(0), page_size, dev_table.data_ptr(), dev_table.shape[1], lanes.data_ptr(),
                      places.data_ptr(), 0.11, 0, split_keys, splits, got.data_ptr(), got.stride(0), stream)
        assert code == 0, f"mi_decode_attention_static returned {code}"
        torch.cuda.synchronize()
        assert torch.cuda.memory_allocated() == before
        if not first_call:
            assert torch.cuda.mem_get_info()[0] == free_before, "the device's free memory changed across the call"
        assert torch.equal(got, want), f"subset {subset}: {(got.float() - want.float()).abs().max().item()}"

    both(list(range(len(lengths))), first_call=True)     # the first call on this device asks for the array's address
    both([6, 2])                             # a smaller step right behind it, in the same array
    both([0])
    both(list(range(len(lengths))))

    # partial results beyond the array: refused, nothing launched, the output untouched
    T = len(lengths)
    queries, lanes, places = q.to(DEV), torch.arange(T, dtype=torch.int32, device=DEV), positions.to(DEV)
    untouched = torch.full((T, Hq * dh), 3.0, dtype=dtype, device=DEV)
    too_many = capacity // 4 // (T * Hq * (dh + 2)) + 1
    code = static(queries.data_ptr(), queries.stride(0), T, Hq, Hkv, dh, k_cache.data_ptr(), v_cache.data_ptr(),
                  k_cache.stride(0), page_size, dev_table.data_ptr(), dev_table.shape[1], lanes.data_ptr(),
                  places.data_ptr(), 0.11, 0, 64, too_many, untouched.data_ptr(), untouched.stride(0), stream)
    torch.cuda.synchronize()
    assert code == -2 and bool((untouched == 3.0).all())
