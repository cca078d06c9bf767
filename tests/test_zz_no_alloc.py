"""The decode attention entry point that allocates nothing (`illm_attn_decode_bf16_static`, for
callers that cannot allocate device memory): called through ctypes, it must give bit for bit what
`illm_attn_decode_bf16` gives with a workspace of the caller's, on two calls in a row that share
the library's scratch array, the second with a smaller input; and it must refuse what does not
fit the array."""
import ctypes
import math

import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
PAGE = 64


def _case(B, nh, nkv, hd, lens, seed):
    g = torch.Generator().manual_seed(seed)
    per_seq = max((n + PAGE - 1) // PAGE for n in lens)
    n_pages = B * per_seq + 1
    perm = torch.randperm(n_pages, generator=g)[: B * per_seq].reshape(B, per_seq).to(torch.int32)
    kc = torch.randn(n_pages, nkv, PAGE, hd, generator=g).to(torch.bfloat16)
    vc = torch.randn(n_pages, nkv, PAGE, hd, generator=g).to(torch.bfloat16)
    qkv = torch.randn(B, (nh + 2 * nkv) * hd, generator=g).to(torch.bfloat16)
    slots = torch.arange(B, dtype=torch.int32)
    return [t.to(DEV) for t in (qkv, kc, vc, perm, slots, torch.tensor(lens, dtype=torch.int32))]


def _both(lib, B, nh, nkv, hd, lens, nsplit, waves, seed):
    qkv, kc, vc, pt, slots, seq_len = _case(B, nh, nkv, hd, lens, seed)
    p = lambda t: ctypes.c_void_p(t.data_ptr())
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    scale = ctypes.c_float(1.0 / math.sqrt(hd))
    want = torch.zeros((B, nh * hd), dtype=torch.bfloat16, device=DEV)
    partial = torch.full((B, nh, nsplit, hd + 2), float("nan"), dtype=torch.float32, device=DEV)
    rc = lib.illm_attn_decode_bf16(p(qkv), p(want), p(kc), p(vc), p(pt), pt.shape[1], PAGE, 0,
                                   p(slots), p(seq_len), p(partial), nsplit, waves, B, nh, nkv, hd,
                                   scale, 0, stream)
    assert rc == 0
    got = torch.zeros_like(want)
    torch.cuda.synchronize()
    # free memory as the driver counts it: torch's own counters would not see a hipMalloc
    before = torch.cuda.mem_get_info(DEV)[0]
    rc = lib.illm_attn_decode_bf16_static(p(qkv), p(got), p(kc), p(vc), p(pt), pt.shape[1], PAGE, 0,
                                          p(slots), p(seq_len), nsplit, waves, B, nh, nkv, hd,
                                          scale, 0, stream)
    assert rc == 0
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info(DEV)[0] == before
    assert torch.isfinite(got.float()).all()
    assert torch.equal(got, want), (B, nh, nkv, hd, nsplit)
    return got


def test_two_calls_in_a_row_share_the_scratch_array():
    from inferllm_amd.kernels import build
    lib = build.library()
    # grouped heads on the matrix cores, 4 splits: 3 x 32 x 4 x 130 floats of scratch
    _both(lib, 3, 32, 8, 128, [650, 90, 3000], 4, 4, seed=1)
    # a smaller input right after it: what the first call left beyond it must not be read
    _both(lib, 1, 4, 4, 64, [200], 2, 2, seed=2)
    # one query head per kv head, many splits, and the first shape again
    _both(lib, 2, 8, 8, 128, [4000, 70], 16, 8, seed=3)
    _both(lib, 3, 32, 8, 128, [650, 90, 3000], 4, 4, seed=1)
    # a single range per sequence uses no scratch at all
    _both(lib, 2, 8, 2, 32, [100, 63], 1, 1, seed=4)


def test_the_entry_point_can_be_captured_into_a_graph():
    """An allocation (or any other call that a capture forbids) inside the entry point would end
    the capture with an error; the replays, with eager work between them, must give what the
    eager call gave."""
    from inferllm_amd.kernels import build
    lib = build.library()
    B, nh, nkv, hd, nsplit, waves = 2, 16, 4, 128, 4, 4
    want = _both(lib, B, nh, nkv, hd, [900, 130], nsplit, waves, seed=6)   # the device's first call is eager
    qkv, kc, vc, pt, slots, seq_len = _case(B, nh, nkv, hd, [900, 130], seed=6)
    p = lambda t: ctypes.c_void_p(t.data_ptr())
    got = torch.zeros_like(want)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        rc = lib.illm_attn_decode_bf16_static(
            p(qkv), p(got), p(kc), p(vc), p(pt), pt.shape[1], PAGE, 0, p(slots), p(seq_len), nsplit,
            waves, B, nh, nkv, hd, ctypes.c_float(1.0 / math.sqrt(hd)), 0,
            ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    assert rc == 0
    for _ in range(3):
        got.fill_(0)
        _both(lib, 1, 4, 4, 64, [200], 2, 2, seed=2)        # eager work that uses the array between replays
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(got, want)


def test_what_does_not_fit_the_array_is_refused():
    from inferllm_amd.kernels import build
    lib = build.library()
    B, nh, nkv, hd, nsplit = 64, 64, 8, 128, 16          # 64 * 64 * 16 * 130 * 4 bytes = 34 MB
    qkv, kc, vc, pt, slots, seq_len = _case(B, nh, nkv, hd, [70] * B, seed=5)
    out = torch.full((B, nh * hd), 7.0, dtype=torch.bfloat16, device=DEV)
    p = lambda t: ctypes.c_void_p(t.data_ptr())
    rc = lib.illm_attn_decode_bf16_static(p(qkv), p(out), p(kc), p(vc), p(pt), pt.shape[1], PAGE, 0,
                                          p(slots), p(seq_len), nsplit, 4, B, nh, nkv, hd,
                                          ctypes.c_float(0.1), 0,
                                          ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    torch.cuda.synchronize()
    assert rc == 3                                       # ILLM_ERR_SCRATCH, nothing launched
    assert bool((out == 7.0).all())
