"""The entry point that allocates nothing: decode attention whose partial results
go to a fixed device array of the library (yalm_attn_decode_static), called through
ctypes and compared with yalm_attn_decode, which takes its workspace from the
caller, and with the plain implementation's attention of one query (these two entry
points read pages kept in rows, which no other caller does).  Two calls in a row on
the same array, the second with a smaller input: what the first call left behind must
not reach the second one's result.  The second call is also watched for device memory
taken or given back, by the driver's own count of free memory."""
import ctypes

import pytest
import torch

from test_gpu_kernels import DEV, close, i32, one_query_reference, paged_case, rnd

pytestmark = pytest.mark.gpu

STATIC_BYTES = 8 << 20
ERR_SCRATCH = 1003


def _both(lib, q, kp, vp, bt, ring, slots, lens, n_heads, n_kv, hd, window, splits, dtype, simple, watch=False):
    """(result with a workspace of the caller's, result with the library's fixed array).  watch: the
    driver's free device memory must be the same before and after the call (a hipMalloc or hipFree
    inside the library would move it; torch's own counters cannot see one)."""
    from yalm_amd.ops import kernels
    B = q.shape[0]
    code = kernels.dtype_code(dtype)
    n_pages = kp.shape[0]
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    sl, ln = i32(slots), i32(lens)
    want = torch.full((B, n_heads * hd), 3.0, dtype=dtype, device=DEV)
    partial = torch.full((kernels.attn_decode_workspace_floats(B, n_heads, hd, splits),), float("nan"), device=DEV)
    rc = lib.yalm_attn_decode(q.data_ptr(), kp.data_ptr(), vp.data_ptr(), bt.data_ptr(), bt.shape[1], ring,
                              sl.data_ptr(), ln.data_ptr(), want.data_ptr(), partial.data_ptr(), B, n_heads, n_kv, hd,
                              window, splits, n_pages, code, int(simple), stream)
    assert rc == 0
    got = torch.full((B, n_heads * hd), 5.0, dtype=dtype, device=DEV)
    torch.cuda.synchronize()
    before = torch.cuda.mem_get_info()[0]
    rc = lib.yalm_attn_decode_static(q.data_ptr(), kp.data_ptr(), vp.data_ptr(), bt.data_ptr(), bt.shape[1], ring,
                                     sl.data_ptr(), ln.data_ptr(), got.data_ptr(), B, n_heads, n_kv, hd, window,
                                     splits, n_pages, code, int(simple), stream)
    assert rc == 0, lib.yalm_error_string(rc)
    torch.cuda.synchronize()
    if watch:        # no torch allocation lies between the two readings
        after = torch.cuda.mem_get_info()[0]
        assert after == before, "free device memory moved by %d bytes across the call" % (after - before)
    return want.cpu(), got.cpu()


def _against_plain(got, q, keys, vals, n_heads, hd, window, dtype, what):
    for b in range(len(keys)):
        want = one_query_reference(q[b].double().reshape(n_heads, hd), keys[b], vals[b], window).reshape(-1)
        close(got[b], want, dtype, "%s, row %d" % (what, b))


@pytest.mark.parametrize("simple", [False, True])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("hd", [128, 64])
def test_static_scratch_decode_attention_twice(hd, dtype, simple):
    from yalm_amd.ops import library
    lib = library.lib()
    n_heads, n_kv = 8, 2
    # first call: four sequences (one row of padding), seven splits
    lens = [1000, 3, 517, 64]
    kp, vp, bt, slots, ring, keys, vals = paged_case(lens, n_kv, hd, 0, dtype, 41, stored=False)
    q = rnd((len(lens) + 1, n_heads * hd), 42, dtype).to(DEV)
    want, got = _both(lib, q, kp.to(DEV), vp.to(DEV), bt.to(DEV), ring, slots + [-1], lens + [0], n_heads, n_kv, hd, 0,
                      7, dtype, simple)
    assert torch.isfinite(want.float()).all() and torch.equal(want, got)
    assert (got[-1] == 0).all()
    _against_plain(got, q.cpu(), keys, vals, n_heads, hd, 0, dtype, "first call")
    # second call, smaller in every size: the array still holds the first call's partial results
    lens2 = [130, 70]
    kp2, vp2, bt2, slots2, ring2, keys2, vals2 = paged_case(lens2, n_kv, hd, 100, dtype, 43, stored=False)
    q2 = rnd((2, n_heads * hd), 44, dtype).to(DEV)
    want2, got2 = _both(lib, q2, kp2.to(DEV), vp2.to(DEV), bt2.to(DEV), ring2, slots2, lens2, n_heads, n_kv, hd, 100,
                        2, dtype, simple, watch=True)
    assert torch.isfinite(want2.float()).all() and torch.equal(want2, got2)
    _against_plain(got2, q2.cpu(), keys2, vals2, n_heads, hd, 100, dtype, "second call")


def test_static_scratch_refuses_sizes_beyond_its_array():
    from yalm_amd.ops import kernels, library
    lib = library.lib()
    B, n_heads, hd, splits = 64, 32, 128, 16
    assert kernels.attn_decode_workspace_floats(B, n_heads, hd, splits) * 4 > STATIC_BYTES
    dummy = torch.zeros(8, device=DEV)
    p = dummy.data_ptr()
    rc = lib.yalm_attn_decode_static(p, p, p, p, 1, 1, p, p, p, B, n_heads, 8, hd, 0, splits, 1, 1, 0,
                                     ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    assert rc == ERR_SCRATCH
    assert b"scratch" in lib.yalm_error_string(rc)
