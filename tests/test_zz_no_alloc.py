"""The allocation-free weight-gradient entry point (jf_igemm_block_fp_noalloc) against jf_igemm_block_fp.

Bar: bit-exact (same kernels, same K-split plan, same arithmetic; only the home of the fp32 partial sums differs).
Two calls in a row share the GPU's built-in scratch buffer, the second with a smaller problem, so stale partial sums of
the first call lie next to (and beyond) the ones the second call writes.
"""
import ctypes as C

import numpy as np
import pytest
import torch

from helpers import QB, rand_codes, rand_scales

pytestmark = pytest.mark.gpu


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def _problem(seed, M, N, K):
    rng = np.random.default_rng(seed)
    A = rand_codes(rng, (M, K))
    B = rand_codes(rng, (K, N))
    sa = rand_scales(rng, (K // QB, M // QB), f16=False)
    sb = rand_scales(rng, (K // QB, N // QB), f16=False)
    return A, B, sa, sb


def _both(jf, A, B, sa, sb, a_km, splitk, out_dtype):
    """(result of the existing entry point, result of the allocation-free one) through the C ABI."""
    M, K = A.shape
    N = B.shape[1]
    dA = dev(A.T) if a_km else dev(A)
    dB, dsa, dsb = dev(B), dev(sa), dev(sb)
    a_layout = jf.A_KM if a_km else jf.A_MK
    want = jf.igemm_block_fp(dA, dB, dsa, dsb, jf.B_KN, out_dtype, a_layout=a_layout, splitk=splitk)
    out = torch.full((M, N), float("nan"), dtype=out_dtype, device="cuda")
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated()
    free_before = torch.cuda.mem_get_info()[0]                 # the device's own count: sees a hipMalloc inside the library too
    L = jf.lib()
    print(f"noalloc M={M} N={N} K={K} a_km={a_km} splitk={splitk} {out_dtype}", flush=True)
    rc = L.jf_igemm_block_fp_noalloc(dA.data_ptr(), dB.data_ptr(), dsa.data_ptr(), dsb.data_ptr(), out.data_ptr(), M, N, K,
                                     a_layout, jf.B_KN, jf.SCALE_F32, jf.SCALES_KMAJOR, jf.SCALES_KMAJOR,
                                     jf._FP_CODE[out_dtype], splitk, C.c_void_p(torch.cuda.current_stream().cuda_stream))
    assert rc == 0, L.jf_error_string(rc)
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() == before
    assert torch.cuda.mem_get_info()[0] >= free_before, "device memory was allocated during the call"
    return want, out


def _same_bits(a, b):
    return torch.equal(a.view(torch.int16 if a.element_size() == 2 else torch.int32),
                       b.view(torch.int16 if b.element_size() == 2 else torch.int32))


def test_two_calls_in_a_row_second_smaller(jf, oracle):
    # GPT-2 small attention projection weight gradient: 768 x 768 outputs over 12288 tokens, 14 parts = 33 MB of partials
    big = _problem(1, 768, 768, 12288)
    parts, per = jf.splitk_plan(768, 768, 12288, 0)
    assert parts > 1 and parts * 768 * 768 * 4 <= jf.NOALLOC_SCRATCH_BYTES
    want, got = _both(jf, *big, a_km=True, splitk=0, out_dtype=torch.float32)
    assert _same_bits(want, got)
    # a smaller problem right behind it, in the same buffer: 4 parts of 256 x 384
    small = _problem(2, 256, 384, 2048)
    assert jf.splitk_plan(256, 384, 2048, 4)[0] == 4
    want, got = _both(jf, *small, a_km=False, splitk=4, out_dtype=torch.float32)
    assert _same_bits(want, got)
    A, B, sa, sb = small
    p, k = jf.splitk_plan(256, 384, 2048, 4)
    ref = oracle.igemm_block_f32_splitk(A, B, sa, sb, 1, p, k)
    assert np.array_equal(got.cpu().numpy().view(np.uint32), ref.view(np.uint32))
    # and the half-precision output, with the big problem's leftovers still in the buffer
    want, got = _both(jf, *small, a_km=True, splitk=0, out_dtype=torch.float16)
    assert _same_bits(want, got)


def test_one_chain_needs_no_scratch_and_oversize_is_refused(jf):
    A, B, sa, sb = _problem(3, 160, 96, 1056)
    want, got = _both(jf, A, B, sa, sb, a_km=False, splitk=1, out_dtype=torch.float32)
    assert _same_bits(want, got)
    # 16 parts of 1600 x 1600 fp32 = 164 MB: more than the built-in buffer
    M = N = 1600
    K = 16 * 16 * QB
    dA = torch.zeros((M, K), dtype=torch.int8, device="cuda")
    dB = torch.zeros((K, N), dtype=torch.int8, device="cuda")
    s1 = torch.ones((K // QB, M // QB), device="cuda")
    out = torch.empty((M, N), device="cuda")
    assert jf.splitk_plan(M, N, K, 16)[0] * M * N * 4 > jf.NOALLOC_SCRATCH_BYTES
    with pytest.raises(RuntimeError, match="scratch"):
        jf.igemm_block_fp_noalloc(dA, dB, s1, s1, out, splitk=16)
