"""The allocation-free decode entry point (vqa_decode_static_bf16) against vqa_decode_bf16: same kernels, the scratch
in the library's static device array instead of a caller workspace.  Two calls in a row, the second on a smaller
input, each compared bit for bit with the workspace entry point and, within tolerance, with the CPU oracle."""
import math

import pytest
import torch

import oracle
from tests.util import assert_close_16, assert_close_lse
from vqtree_amd import _lib
from vqtree_amd.synthetic import decode_case

pytestmark = pytest.mark.gpu


def _call(lib, name, case, N, workspace):
    B, H, _, D = case.q.shape
    M, K = case.codes.shape[3], case.codebooks.shape[2]
    q, cb = case.q, case.codebooks
    codes, v = case.codes[:, :, :N].contiguous(), case.v[:, :, :N].contiguous()
    out = torch.empty((B, H, 1, D), dtype=q.dtype, device=q.device)
    lse = torch.empty((B, H, 1), dtype=torch.float32, device=q.device)
    strides = _lib.strides_array(q.stride(0), q.stride(1), codes.stride(0), codes.stride(1), cb.stride(0), cb.stride(1),
                                 cb.stride(2), v.stride(0), v.stride(1), v.stride(2), out.stride(0), out.stride(1))
    scale = 1.0 / math.sqrt(D)
    stream = _lib.current_stream(q.device)
    head = (q.data_ptr(), codes.data_ptr(), cb.data_ptr(), v.data_ptr(), out.data_ptr(), lse.data_ptr())
    tail = (B, H, N, D, M, K, strides, scale, 0, stream)
    if workspace is None:
        rc = getattr(lib, name)(*head, *tail)
    else:
        rc = getattr(lib, name)(*head, workspace.data_ptr(), workspace.numel(), *tail)
    _lib.check(rc)
    torch.cuda.synchronize()
    want, want_lse = oracle.attn_vq_decode(q, codes, cb, v, scale)
    return out, lse, want, want_lse


def test_static_scratch_decode_matches_workspace_decode_twice(lib):
    case = decode_case(3, 8, 5000, 128, 4, device="cuda:0", seed=11)
    for N in (5000, 1300):  # the second call is smaller: stale scratch of the first must not leak into it
        print(f"no-alloc decode: B3 H8 N{N} D128 M4", flush=True)
        ws = torch.empty(lib.vqa_decode_workspace_bytes(3, 8, N, 128, 4, 256, 0), dtype=torch.uint8, device="cuda:0")
        ref_out, ref_lse, want, want_lse = _call(lib, "vqa_decode_bf16", case, N, ws)
        out, lse, _, _ = _call(lib, "vqa_decode_static_bf16", case, N, None)
        assert torch.equal(out, ref_out) and torch.equal(lse, ref_lse)
        assert_close_16(out, want, f"static-scratch decode N={N}")
        assert_close_lse(lse, want_lse)


def test_static_scratch_decode_refuses_oversized_problem(lib):
    # 16 x 32 x 64 splits x (128 + 2) floats of split states alone exceed the 8 MiB array: refused on the host
    strides = _lib.strides_array(*([0] * 12))
    # (NULL tensors: were the size check ever moved behind the others, the call would still stop at the pointer
    # check and launch nothing)
    rc = lib.vqa_decode_static_bf16(None, None, None, None, None, None, 16, 32, 1 << 20, 128, 4, 256, strides, 1.0, 64,
                                    None)
    assert rc == -9
    assert b"static" in lib.vqa_strerror(rc)
