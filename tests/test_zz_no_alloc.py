"""GPU: the allocation-free hash-encoding backward (``nf_hash_encode_bwd_static``) against ``nf_hash_encode_bwd``.

Both are called through the C ABI on the same inputs; the static-scratch variant must give the same table gradient
(bit for bit where a bin is one accumulation task; float atomics meet in another order where a bin is split or the
bit-plane variant runs, hence rtol 1e-3 with a floor of 1e-3 of the level's RMS, the hash backward's tolerance).  Calls
follow each other on one GPU with shrinking inputs, so stale scratch contents of a larger call would show.
"""
import ctypes

import pytest
import torch

from oracle import hash_encoding as O

pytestmark = pytest.mark.gpu
DEV = "cuda"
T, L, F, D, LO, HI = 2**19, 16, 2, 3, 16, 7006


def _call(lib, L_, static, x, do, E, geom, pi, flags=0):
    de = torch.zeros(E, F, dtype=torch.float32, device=DEV)
    stream = L_.current_stream(x.device)
    if static:
        torch.cuda.synchronize()
        free_before = torch.cuda.mem_get_info()[0]
        rc = lib.nf_hash_encode_bwd_static(x.data_ptr(), L_.dtype_code(x.dtype), x.stride(0), x.stride(1), do.data_ptr(), L_.dtype_code(do.dtype),
                                           do.stride(0), de.data_ptr(), x.shape[0], geom, pi.data_ptr(), 1.0, flags, stream)
        torch.cuda.synchronize()
        # after the first call on a device (which may load the code object and resolve the array's address) the entry
        # point leaves the device's free memory exactly as it found it
        if _call.warm:
            assert torch.cuda.mem_get_info()[0] == free_before, "the allocation-free entry point changed the free device memory"
        _call.warm = True
    else:
        n = lib.nf_hash_encode_bwd_workspace_bytes(x.shape[0], geom, L_.dtype_code(do.dtype), flags)
        ws = torch.empty(max(n, 16), dtype=torch.uint8, device=DEV)
        rc = lib.nf_hash_encode_bwd(x.data_ptr(), L_.dtype_code(x.dtype), x.stride(0), x.stride(1), do.data_ptr(), L_.dtype_code(do.dtype),
                                    do.stride(0), de.data_ptr(), x.shape[0], geom, pi.data_ptr(), 1.0, ws.data_ptr(), n, flags, stream)
    torch.cuda.synchronize()
    return rc, de


_call.warm = False


def test_static_scratch_backward_matches_the_workspace_backward():
    from triton_helpers_amd import _lib as L_
    from triton_helpers_amd.layers.hash_encoding.helpers import level_geometry

    lib = L_.load()
    limit = lib.nf_hash_encode_bwd_static_bytes()
    assert limit == 128 * 2**20
    geom = level_geometry(T, L, D, F, LO, HI)
    offs = O.level_row_offsets(L, T, D, LO, HI)
    E = offs[-1]
    pi = torch.tensor(O.PRIMES, dtype=torch.int64, device=DEV)
    g = torch.Generator().manual_seed(7)
    # 2^20 points: the records do not fit, the bit-planes do; 80000: records; 33000: records, smaller than the call before
    for n, dtype in ((2**20, torch.float16), (80000, torch.float16), (33000, torch.float16), (60000, torch.float32), (40000, torch.bfloat16), (1000, torch.float16)):
        x = torch.rand(n, D, generator=g).to(DEV)
        do = torch.randn(n, L * F, generator=g).to(dtype).to(DEV)
        need = lib.nf_hash_encode_bwd_workspace_bytes(n, geom, L_.dtype_code(dtype), 0)
        planes = need > limit
        rc, got = _call(lib, L_, True, x, do, E, geom, pi)
        assert rc == 0, lib.nf_last_error()
        rc, want = _call(lib, L_, False, x, do, E, geom, pi, flags=L_.NF_HASH_FORCE_PLANES if planes else 0)
        assert rc == 0, lib.nf_last_error()
        for l in range(L):
            a, b = got[offs[l]:offs[l + 1]], want[offs[l]:offs[l + 1]]
            rms = float(b.pow(2).mean().sqrt())
            assert float(((a - b).abs() - 1e-3 * b.abs()).max()) <= 1e-3 * rms, (n, dtype, l)
        if n == 80000:  # and against the oracle once
            ref = O.encode_backward(x.cpu(), do.cpu(), E, F, None, T, L, LO, HI)
            torch.testing.assert_close(got.cpu(), ref, rtol=1e-3, atol=1e-4)
    # beyond the scratch: refused before anything is launched, with the sizes in the message
    n = 2**21
    x = torch.rand(n, D, generator=g).to(DEV)
    do = torch.randn(n, L * F, generator=g).half().to(DEV)
    rc, de = _call(lib, L_, True, x, do, E, geom, pi)
    assert rc == L_.NF_EINVAL and b"static scratch holds 134217728" in lib.nf_last_error()
    assert not bool(de.any())
    # float32 gradients have no bit-plane variant: refused as soon as the records do not fit
    rc, de = _call(lib, L_, True, x[: 2**18], do[: 2**18].float(), E, geom, pi)
    assert rc == L_.NF_EINVAL and not bool(de.any())
