"""CPU-side checks of the C-ABI library: it loads, exports every symbol include/vqattn.h declares, and its
host-only entry points (no kernel launch) behave."""
import os
import re

import pytest

from vqtree_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "vqattn.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(vqa_[a-z0-9_]+)\s*\(", text)))


def test_header_symbols_are_exported_and_bound(lib):
    declared = _declared_symbols()
    assert declared, "no declarations parsed"
    for name in declared:
        assert hasattr(lib, name), f"{name} declared in include/vqattn.h but not exported"
        assert name in _lib.SIGNATURES, f"{name} has no ctypes signature in vqtree_amd/_lib.py"
    assert sorted(_lib.SIGNATURES) == declared


def test_version_and_error_strings(lib):
    assert lib.vqa_version() >= 100
    assert lib.vqa_strerror(0) == b"ok"
    seen = set()
    for code in range(-9, 0):
        msg = lib.vqa_strerror(code)
        assert msg and msg != b"unknown vqa status" and msg not in seen
        seen.add(msg)
    assert lib.vqa_strerror(-99) == b"unknown vqa status"


def test_decode_host_side_queries(lib):
    # 512 (b,h) units fill the chip with one split each (the streaming kernel then stores the result itself, no merge
    # launch); fewer units are split for about a thousand workgroups of at least 4096 keys each
    assert lib.vqa_decode_default_splits(16, 32, 32768) == 1
    assert lib.vqa_decode_default_splits(8, 32, 32768) == 4
    assert lib.vqa_decode_default_splits(4, 32, 65536) == 8
    # few (batch, head) units: shorter splits so every compute unit still gets a workgroup
    assert lib.vqa_decode_default_splits(1, 8, 32768) == 32
    assert lib.vqa_decode_default_splits(1, 1, 10) == 1
    small = lib.vqa_decode_workspace_bytes(1, 1, 64, 128, 4, 256, 1)
    big = lib.vqa_decode_workspace_bytes(16, 32, 32768, 128, 4, 256, 8)
    assert 0 < small < big
    # LUT (B*H*M*256 fp32) + partial states (B*H*S*(D+2) fp32), each 256-byte aligned
    assert big >= 512 * 4 * 256 * 4 + 512 * 8 * 130 * 4


def test_decode_rejects_bad_arguments_before_any_launch(lib):
    strides = _lib.strides_array(*([0] * 12))
    args = dict(B=1, H=1, N=8, D=128, M=4, K=256)

    def call(q=1, codes=1, cb=1, v=1, out=1, ws=256, ws_bytes=1 << 20, **kw):
        a = dict(args, **kw)
        return lib.vqa_decode_bf16(q, codes, cb, v, out, None, ws, ws_bytes, a["B"], a["H"], a["N"], a["D"], a["M"],
                                   a["K"], strides, 1.0, 1, None)

    assert call(q=None) == -1                      # VQA_ERR_NULL_POINTER
    assert call(q=16, cb=16, v=16, N=0) == -2      # VQA_ERR_BAD_SHAPE
    assert call(q=16, cb=16, v=16, D=96) == -3     # VQA_ERR_UNSUPPORTED_HEAD_DIM
    assert call(q=16, cb=16, v=16, M=3) == -4      # VQA_ERR_UNSUPPORTED_CODEBOOK
    assert call(q=16, cb=16, v=16, K=257) == -4
    assert call(q=18, cb=16, v=16) == -5           # VQA_ERR_MISALIGNED
    assert call(q=16, cb=16, v=16, codes=4, ws_bytes=8) == -6  # VQA_ERR_WORKSPACE_TOO_SMALL


def test_row_strides_beyond_the_32_bit_lane_offsets_are_rejected(lib):
    """64 rows x stride x 2 bytes must fit the 32-bit per-lane offsets of the streaming / tile-copy loops; larger (or
    negative) row strides are refused on the host, before any launch."""
    big = 1 << 24
    s = [0] * 12
    s[9] = big  # v row stride of the coded decode
    rc = lib.vqa_decode_bf16(16, 16, 16, 16, 16, None, 256, 1 << 30, 1, 1, 8, 128, 4, 256, _lib.strides_array(*s), 1.0,
                             1, None)
    assert rc == -7
    s = [0] * 10
    s[4] = big  # k row stride of the exact decode
    rc = lib.vqa_decode_exact_bf16(16, 16, 16, 16, None, 256, 1 << 30, 1, 1, 8, 128, _lib.strides_array(*s), 1.0, 1,
                                   None)
    assert rc == -7
    s = [128] * 18
    s[8] = -128  # negative k1 row stride of the window kernel
    rc = lib.vqa_local_attn_bf16(16, 16, 16, 16, 16, 16, None, 1, 1, 8, 128, _lib.strides_array(*s), 4, 0, 1.0, None)
    assert rc == -7
    s[8] = big
    rc = lib.vqa_local_attn_bf16(16, 16, 16, 16, 16, 16, None, 1, 1, 8, 128, _lib.strides_array(*s), 4, 0, 1.0, None)
    assert rc == -7
    s = [128] * 23
    s[10] = big  # v row stride of the prefill: refused before the reconstruction kernel is enqueued
    rc = lib.vqa_prefill_bf16(16, 16, 16, 16, None, None, None, 16, None, 256, 1 << 30, 1, 1, 8, 128, 4, 256,
                              _lib.strides_array(*s), 0, 0, 1, 1.0, None)
    assert rc == -7


def test_count_state_and_schedule_entry_points_reject_bad_arguments_before_any_launch(lib):
    six = _lib.strides_array(*([128] * 6))
    add = lib.vqa_count_state_add_bf16
    assert add(None, 16, 16, 16, 1, 1, 8, 128, 512, six, None) == -1        # ids missing
    assert add(16, 16, 16, 16, 1, 1, 8, 48, 512, six, None) == -3          # head dim
    assert add(16, 16, 16, 16, 0, 1, 8, 128, 512, six, None) == -2         # batch
    assert add(16, 16, 16, 16, 1, 1, 0, 128, 512, six, None) == 0          # nothing to add: no launch, ok
    dec = lib.vqa_count_decode_bf16
    assert dec(16, 16, 16, 16, None, None, 1, 1, 512, 128, six, 1.0, None) == -1   # out missing
    assert dec(16, 16, 16, 16, 16, None, 1, 1, 8193, 128, six, 1.0, None) == -2    # more codewords than the state holds
    assert dec(16, 16, 16, 16, 16, None, 1, 1, 512, 96, six, 1.0, None) == -3
    assert dec(16, 24, 16, 16, 16, None, 1, 1, 512, 128, six, 1.0, None) == -5     # codebook not 16-byte aligned
    # the pipelined schedule is refused where it does not apply: window not a multiple of 128 / exact boundary rule
    s23 = _lib.strides_array(*([128] * 23))
    rc = lib.vqa_prefill_pipelined_bf16(16, 16, 16, 16, 16, 16, None, 256, 1 << 30, 1, 1, 256, 128, 4, 256, s23, 100, 1,
                                        1.0, None)
    assert rc == -7
    # the tiled entry point validates like vqa_prefill_*: unsupported head dim, too small a workspace
    rc = lib.vqa_prefill_tiled_bf16(16, 16, 16, 16, None, None, None, 16, None, 256, 1 << 30, 1, 1, 8, 96, 4, 256, s23,
                                    0, 0, 1, 1.0, None)
    assert rc == -3
    rc = lib.vqa_prefill_tiled_bf16(16, 16, 16, 16, None, None, None, 16, None, 256, 8, 1, 1, 8, 128, 4, 256, s23, 0, 0,
                                    1, 1.0, None)
    assert rc == -6
    # integer-count entry points share the count kernel's checks
    s17 = _lib.strides_array(*([128] * 17))
    assert lib.vqa_vqcount_fwd_icnt_bf16(16, 16, None, 16, 16, 16, None, 1, 1, 512, 128, 128, s17, 128, 1.0, None) == -1
    assert lib.vqa_vqcount_merge_icnt_bf16(16, 16, 16, 16, 16, 16, None, 1, 1, 512, 128, 128, s17, 128, 1.0, None) == -1


def test_roped_decode_rejects_bad_arguments_before_any_launch(lib):
    strides = _lib.strides_array(*([0] * 12))

    def call(cos=16, sin=16, q=16, D=128):
        return lib.vqa_decode_roped_bf16(q, cos, sin, 16, 16, 16, 16, None, 256, 1 << 20, 1, 1, 8, D, 4, 256, strides,
                                         1.0, 1, None, None)

    assert call(cos=None) == -1 and call(sin=None) == -1 and call(q=None) == -1  # VQA_ERR_NULL_POINTER
    assert call(cos=18) == -5                                                  # VQA_ERR_MISALIGNED
    assert call(D=96) == -3                                                    # VQA_ERR_UNSUPPORTED_HEAD_DIM


def test_static_scratch_decode_refuses_oversized_problem_on_the_host(lib):
    strides = _lib.strides_array(*([0] * 12))
    # (NULL tensors: were the size check ever moved behind the others, the call would still stop at the pointer
    # check and launch nothing)
    rc = lib.vqa_decode_static_bf16(None, None, None, None, None, None, 16, 32, 1 << 20, 128, 4, 256, strides, 1.0, 64,
                                    None)
    assert rc == -9 and b"static" in lib.vqa_strerror(rc)


def test_generation_step_is_recognised_after_any_prefill():
    """A cache that has recorded a prefill classifies the next seqlen_q == 1 call as a generation step whatever the
    codebook size (it must not restart as a one-token prefill); without a GPU that step fails loudly in the HIP
    layer -- there is no CPU fallback."""
    import torch

    from vqtree_amd.ops import attn_vq as A

    H, C, D, N = 2, 512, 64, 700
    cache = A.VectorQuantizedReRoPECache(256, torch.zeros(H, C, D, dtype=torch.bfloat16))
    assert cache.get_seq_length() == 0
    cache.seq_lengths.append(N)
    cache.decode_state.append(None)
    assert cache.get_seq_length() == N
    one = torch.zeros(1, H, 1, D, dtype=torch.bfloat16)
    with pytest.raises(Exception) as e:
        A.dispatch_attn(one, one, one, torch.tensor([[N]]), cache)
    assert cache.get_seq_length() == N  # nothing was recorded as a fresh prefill
    assert not isinstance(e.value, AssertionError)
    with pytest.raises(AssertionError):
        A.dispatch_attn(one, one, one, torch.tensor([[N]]), A.VectorQuantizedReRoPECache(256, cache.codebook, sphere=True))


def test_ops_refuse_cpu_tensors():
    import torch

    from vqtree_amd.ops.attn_vq import attn_vq_decode

    q = torch.zeros(1, 1, 1, 128, dtype=torch.bfloat16)
    with pytest.raises(_lib.VqaError):
        attn_vq_decode(q, torch.zeros(1, 1, 8, 4, dtype=torch.uint8), torch.zeros(1, 4, 256, 128, dtype=torch.bfloat16),
                       torch.zeros(1, 1, 8, 128, dtype=torch.bfloat16))


def test_encoder_preprocessing_rope_reject_bad_arguments_before_any_launch(lib):
    s12, s18, s8 = (_lib.strides_array(*([8] * n)) for n in (12, 18, 8))
    enc = lambda x=16, cb=16, codes=16, ids=None, N=8, D=128, M=4, K=256, mode=1: lib.vqa_encode_keys_bf16(
        x, cb, codes, ids, 1, 1, N, D, M, K, s12, mode, 0, None)
    assert enc(x=None) == -1 and enc(codes=None, ids=None) == -1   # VQA_ERR_NULL_POINTER
    assert enc(N=0) == -2 and enc(K=250) == -2                      # VQA_ERR_BAD_SHAPE (K must be a multiple of 32)
    assert enc(D=96) == -3 and enc(D=32) == -3                      # VQA_ERR_UNSUPPORTED_HEAD_DIM
    assert enc(K=512) == -7 and enc(mode=2) == -7                   # uint8 codes need K <= 256; unknown mode
    assert enc(x=18) == -5                                          # VQA_ERR_MISALIGNED

    need = lib.vqa_preprocess_workspace_bytes(2, 4, 1000, 512)
    # histograms [B*H, ceil(N/128), C] + start [B*H, C] + order [B*H, N], int32 each
    assert need >= 8 * 8 * 512 * 4 + 8 * 512 * 4 + 8 * 1000 * 4 and need % 256 == 0
    assert lib.vqa_preprocess_workspace_bytes(0, 4, 1000, 512) == 0
    pre = lambda ids=16, v=16, vvq=16, vi=16, ws=256, ws_bytes=1 << 30, N=1000, D=128, C=512: lib.vqa_preprocess_bf16(
        ids, v, None, None, vvq, vi, ws, ws_bytes, 2, 4, N, D, C, s18, None)
    assert pre(ids=None) == -1 and pre(vi=None) == -1
    assert pre(C=8193) == -2 and pre(N=0) == -2
    assert pre(D=130) == -3 and pre(D=7) == -3
    assert pre(ws_bytes=need - 1) == -6                             # VQA_ERR_WORKSPACE_TOO_SMALL
    assert pre(ws=128) == -5

    rope = lambda x=16, pos=16, cos=16, sin=16, out=16, out2=None, D=128, n_pos=64, fixed=0: lib.vqa_rope_bf16(
        x, pos, cos, sin, out, out2, 1, 1, 8, D, n_pos, 128, s8, fixed, None)
    assert rope(x=None) == -1 and rope(cos=None) == -1
    assert rope(D=24) == -3
    assert rope(pos=None, fixed=64) == -7 and rope(pos=None, fixed=-1) == -7   # fixed position outside the tables
    assert rope(out=20) == -5
    assert rope(pos=None, out2=16) == -7 and rope(out2=16, fixed=99) == -7      # second output: per-row form only

    s17 = _lib.strides_array(*([8] * 17))
    merge = lambda lse=16, out=16: lib.vqa_vqcount_merge_bf16(16, 16, 16, 16, 16, out, lse, 1, 1, 256, 128, 128, s17,
                                                              64, 1.0, None)
    assert merge(lse=None) == -1 and merge(out=None) == -1          # the state to merge into is required


def test_exact_decode_rejects_bad_arguments_before_any_launch(lib):
    s10 = _lib.strides_array(*([8] * 10))
    need = lib.vqa_decode_exact_workspace_bytes(2, 4, 5000, 128, 4)
    assert need >= 8 * 4 * 130 * 4 and need % 256 == 0 and lib.vqa_decode_exact_workspace_bytes(2, 4, 0, 128, 4) == 0
    call = lambda q=16, k=16, v=16, out=16, ws=256, ws_bytes=1 << 20, N=5000, D=128: lib.vqa_decode_exact_bf16(
        q, k, v, out, None, ws, ws_bytes, 2, 4, N, D, s10, 1.0, 4, None)
    assert call(k=None) == -1 and call(ws=None) == -1
    assert call(N=0) == -2
    assert call(D=96) == -3
    assert call(v=24) == -5 and call(ws=64) == -5
    assert call(ws_bytes=need - 1) == -6


def test_windowed_decode_rejects_bad_arguments_before_any_launch(lib):
    s17 = _lib.strides_array(*([8] * 17))
    need = lib.vqa_decode_windowed_workspace_bytes(2, 4, 5000, 512, 128, 4)
    assert need > lib.vqa_decode_workspace_bytes(2, 4, 5000 - 512, 128, 4, 256, 0) and need % 256 == 0
    assert lib.vqa_decode_windowed_workspace_bytes(2, 4, 100, 200, 128, 4) == 0  # window longer than the cache
    call = lambda qf=16, qw=16, codes=16, cb=16, v=16, kw=16, out=16, ws=256, ws_bytes=1 << 24, N=5000, W=512, D=128, M=4: \
        lib.vqa_decode_windowed_bf16(qf, qw, codes, cb, v, kw, out, None, ws, ws_bytes, 2, 4, N, W, D, M, 256, s17, 1.0,
                                     None)
    assert call(qw=None) == -1 and call(kw=None) == -1 and call(codes=None) == -1
    assert call(W=0) == -2 and call(W=6000) == -2
    assert call(D=96) == -3 and call(M=3) == -4
    assert call(kw=24) == -5
    assert call(ws_bytes=need - 1) == -6
