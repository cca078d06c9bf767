"""Each HIP kernel alone against its plain torch contract (tests/kernel_refs.py),
at sizes other than the engine's tiny models: widths and vocabularies that are no
power of two, head sizes in steps of 16 (and 24), odd head and group counts.
Shapes include those of the reference's own op tests (test/GPU/test_opr.cpp:9-119)."""
import math

import pytest
import torch

import kernel_refs as R

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
DTYPES = [torch.float32, torch.bfloat16]


def ops():
    from inferllm_amd.kernels import ops as o
    return o


def tol(dtype):
    return (2e-5, 2e-5) if dtype == torch.float32 else (2e-2, 2e-2)


def close(got, want, dtype, scale=1.0):
    a, r = tol(dtype)
    assert got.shape == want.shape
    torch.testing.assert_close(got.double().cpu(), want.double().cpu(), atol=a * scale, rtol=r)


def rnd(*shape, dtype=torch.float32, seed=0, std=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g) * std).to(dtype)


def test_every_entry_point_is_declared_and_a_wrong_call_raises():
    """The loader gives each function of api.h its argument types: a call with too few arguments
    or with a float where a size is meant raises instead of launching on garbage."""
    import ctypes
    lib = ops()._lib()
    assert lib.illm_version.argtypes == [] and lib.illm_embed.argtypes[-1] is ctypes.c_void_p
    with pytest.raises(TypeError):
        lib.illm_silu_mul(None, None, 0, 4)
    with pytest.raises(ctypes.ArgumentError):
        lib.illm_silu_mul(None, None, 0, 4.5, 8, None)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("V,E,ids", [(10, 128, [1, 9, 3, 3]), (411, 80, [0, 410, 7]), (1000, 4100, [999])])
def test_embed(dtype, V, E, ids):
    table = rnd(V, E, dtype=dtype)
    t = torch.tensor(ids, dtype=torch.int32)
    got = ops().embed(t.to(DEV), table.to(DEV))
    assert torch.equal(got.cpu(), R.embed(t, table))       # rows are copied bit for bit


@pytest.mark.parametrize("out_dtype", DTYPES)
@pytest.mark.parametrize("w_dtype", DTYPES)
@pytest.mark.parametrize("T,E,eps", [(4, 4096, 1e-5), (3, 80, 1e-6), (1, 1001, 3e-2), (70, 96, 1e-5), (2, 6000, 1e-5), (2, 9000, 1e-5), (5, 1536, 1e-6)])
def test_add_rmsnorm(out_dtype, w_dtype, T, E, eps):
    x = rnd(T, E, seed=1) * 0.05            # small rows: eps matters
    w = (1 + rnd(E, seed=2) * 0.1).to(w_dtype)
    for delta_dtype in (None, torch.float32, torch.bfloat16):
        delta = None if delta_dtype is None else rnd(T, E, seed=3, std=0.05).to(delta_dtype)
        xr, xg = x.clone(), x.clone().to(DEV)
        want = R.add_rmsnorm(xr, delta, w, eps, out_dtype)
        got = ops().add_rmsnorm(xg, None if delta is None else delta.to(DEV), w.to(DEV), eps, out_dtype)
        close(got, want, out_dtype)
        close(xg, xr, torch.float32)          # the sum is written back
        if T > 2:
            idx = torch.tensor([T - 1, 0], dtype=torch.int32)
            xr2, xg2 = x.clone(), x.clone().to(DEV)
            want = R.add_rmsnorm(xr2, delta, w, eps, out_dtype, idx)
            got = ops().add_rmsnorm(xg2, None if delta is None else delta.to(DEV), w.to(DEV), eps,
                                    out_dtype, idx.to(DEV))
            close(got, want, out_dtype)
            assert torch.equal(xg2.cpu(), x)   # gathered rows leave x alone


@pytest.mark.parametrize("out_dtype", DTYPES)
@pytest.mark.parametrize("S,T,E", [(1, 3, 80), (3, 20, 96), (8, 64, 4096), (5, 17, 6000), (2, 3, 8196), (13, 4, 1536)])
def test_add_rmsnorm_adds_planes(out_dtype, S, T, E):
    """delta as the planes of a product whose K was split: their sum is added, in float32."""
    x = rnd(T, E, seed=1)
    w = (1 + rnd(E, seed=2) * 0.1).to(torch.bfloat16)
    planes = rnd(S, T, E, seed=3) * torch.linspace(0.5, 2.0, S)[:, None, None]
    xr, xg = x.clone(), x.clone().to(DEV)
    want = R.add_rmsnorm(xr, planes, w, 1e-5, out_dtype)
    got = ops().add_rmsnorm(xg, planes.to(DEV), w.to(DEV), 1e-5, out_dtype)
    close(got, want, out_dtype)
    close(xg, xr, torch.float32, scale=4.0)
    idx = torch.tensor([T - 1, 0, T // 2], dtype=torch.int32)
    xg2 = x.clone().to(DEV)
    got = ops().add_rmsnorm(xg2, planes.to(DEV), w.to(DEV), 1e-5, out_dtype, idx.to(DEV))
    close(got, R.add_rmsnorm(x.clone(), planes, w, 1e-5, out_dtype, idx), out_dtype)
    assert torch.equal(xg2.cpu(), x)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("T,F", [(4, 10), (5, 130), (3, 11008), (1, 173), (70, 64), (2, 2056)])
def test_silu_mul(dtype, T, F):
    gu = rnd(T, 2 * F, dtype=dtype, std=3.0)
    gu[0, 0] = 0.0; gu[0, 1] = -60.0; gu[0, 2] = 40.0
    close(ops().silu_mul(gu.to(DEV)), R.silu_mul(gu), dtype, scale=10)


def make_cache(n_pages, nkv, page, hd, dtype):
    return (torch.full((n_pages, nkv, page, hd), float("nan"), dtype=dtype),
            torch.full((n_pages, nkv, page, hd), float("nan"), dtype=dtype))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("nh,nkv,hd,rot,pairing", [(4, 2, 24, 24, 0), (3, 3, 16, 16, 1), (8, 1, 128, 128, 0),
                                                    (5, 5, 48, 32, 0), (2, 1, 256, 256, 1), (32, 8, 64, 64, 0), (3, 1, 48, 48, 0), (2, 2, 32, 16, 0)])
def test_rope_store(dtype, nh, nkv, hd, rot, pairing):
    from inferllm_amd.parts.position import rotary_table
    page, max_pos = 8, 64
    table = rotary_table(12345.0, rot, max_pos, "cpu")
    lens = [13, 1, 20]
    slots = [2, 0, 3]
    pos = [p for n in lens for p in range(n)]
    slot = [s for n, s in zip(lens, slots) for _ in range(n)]
    T = len(pos)
    qkv = rnd(T, (nh + 2 * nkv) * hd, dtype=dtype, seed=5)
    pt = torch.full((5, 4), 11, dtype=torch.int32)
    pt[2, :2] = torch.tensor([7, 3]); pt[0, :1] = 9; pt[3, :3] = torch.tensor([0, 5, 1])
    slot_len = torch.tensor([1, 0, 13, 20, 0], dtype=torch.int32)
    kc, vc = make_cache(12, nkv, page, hd, dtype)
    rp, rs = torch.tensor(pos, dtype=torch.int32), torch.tensor(slot, dtype=torch.int32)
    q_ref, kc_ref, vc_ref = qkv.clone(), kc.clone(), vc.clone()
    R.rope_store(q_ref, table, rot, pairing, rp, rs, slot_len, kc_ref, vc_ref, pt, page, 0, nh, nkv, hd)
    q_g, kc_g, vc_g = qkv.to(DEV), kc.to(DEV), vc.to(DEV)
    ops().rope_store(q_g, table.to(DEV), rot, pairing, rp.to(DEV), rs.to(DEV), slot_len.to(DEV),
                     kc_g, vc_g, pt.to(DEV), page, 0, nh, nkv, hd)
    close(q_g, q_ref, dtype, scale=4)
    for got, want in ((kc_g, kc_ref), (vc_g, vc_ref)):
        got, want = got.cpu(), want
        assert torch.equal(torch.isnan(got), torch.isnan(want))      # exactly the same rows are written
        close(torch.nan_to_num(got), torch.nan_to_num(want), dtype, scale=4)
    # position 0 leaves the row as it is
    first = [0, 13, 14]
    assert torch.equal(q_g.cpu()[first], qkv[first])


@pytest.mark.parametrize("dtype", DTYPES)
def test_rope_store_window_ring(dtype):
    """A ring of pages: rows that a later row of the same step overwrites are skipped."""
    nh, nkv, hd, page, ring = 2, 2, 16, 4, 3
    n = 23
    qkv = rnd(n, (nh + 2 * nkv) * hd, dtype=dtype, seed=9)
    pt = torch.tensor([[4, 2, 6]], dtype=torch.int32)
    slot_len = torch.tensor([n], dtype=torch.int32)
    rp = torch.arange(n, dtype=torch.int32); rs = torch.zeros(n, dtype=torch.int32)
    kc, vc = make_cache(8, nkv, page, hd, dtype)
    kr, vr = kc.clone(), vc.clone()
    R.rope_store(qkv.clone(), None, 0, 0, rp, rs, slot_len, kr, vr, pt, page, ring, nh, nkv, hd)
    kg, vg = kc.to(DEV), vc.to(DEV)
    ops().rope_store(qkv.to(DEV), None, 0, 0, rp.to(DEV), rs.to(DEV), slot_len.to(DEV), kg, vg,
                     pt.to(DEV), page, ring, nh, nkv, hd)
    assert torch.equal(torch.nan_to_num(kg.cpu()), torch.nan_to_num(kr))
    assert torch.equal(torch.nan_to_num(vg.cpu()), torch.nan_to_num(vr))
    # the last ring*page - (page - 1 - (n-1) % page) positions are there, e.g. position n-1
    view = qkv.view(n, nh + 2 * nkv, hd)
    assert torch.equal(kg.cpu()[int(pt[0, ((n - 1) // page) % ring]), :, (n - 1) % page], view[n - 1, nh:nh + nkv])


@pytest.mark.parametrize("xd,wd,yd", [(torch.float32,) * 3, (torch.bfloat16,) * 3,
                                      (torch.bfloat16, torch.bfloat16, torch.float32),
                                      (torch.bfloat16, torch.float32, torch.bfloat16)])
@pytest.mark.parametrize("M,N,K", [(1, 2, 128), (4, 128, 128), (70, 411, 80), (65, 64, 1001), (3, 1000, 172)])
def test_gemm_generic(xd, wd, yd, M, N, K):
    x, w = rnd(M, K, dtype=xd, seed=1), rnd(N, K, dtype=wd, seed=2)
    got = ops().gemm_generic(x.to(DEV), w.to(DEV), yd)
    close(got, R.linear(x, w, yd), yd, scale=math.sqrt(K))


def test_gemm_generic_row_bits_do_not_depend_on_batch():
    x, w = rnd(70, 300, seed=1), rnd(130, 300, seed=2)
    whole = ops().gemm_generic(x.to(DEV), w.to(DEV), torch.float32).cpu()
    for r in (0, 17, 69):
        alone = ops().gemm_generic(x[r:r + 1].to(DEV), w.to(DEV), torch.float32).cpu()
        assert torch.equal(alone[0], whole[r])


def test_gemm_identity_and_linearity():
    x = rnd(5, 96, seed=3)
    eye = torch.eye(96)
    assert torch.equal(ops().gemm_generic(x.to(DEV), eye.to(DEV), torch.float32).cpu(), x)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("nh,nkv,hd,lens,window", [
    (4, 4, 16, [7], 0), (4, 2, 24, [5, 11, 2], 0), (16, 16, 8, [2], 0), (32, 2, 128, [5, 70], 0),
    (3, 1, 48, [33, 64, 1, 100], 0), (2, 2, 256, [40], 0), (4, 2, 32, [90, 17], 13), (5, 5, 16, [130], 64)])
def test_attn_prefill(dtype, nh, nkv, hd, lens, window):
    T = sum(lens)
    qkv = rnd(T, (nh + 2 * nkv) * hd, dtype=dtype, seed=7)
    cu = torch.tensor([0] + list(torch.tensor(lens).cumsum(0)), dtype=torch.int32)
    scale = 1.0 / math.sqrt(hd)
    got = ops().attn_prefill(qkv.to(DEV), cu.to(DEV), len(lens), max(lens), nh, nkv, hd, scale, window)
    want = R.attn_prefill(qkv, cu, len(lens), max(lens), nh, nkv, hd, scale, window)
    close(got, want, dtype, scale=2)


@pytest.mark.parametrize("nh,nkv,hd,lens,window", [
    (4, 4, 128, [300, 129, 128, 1], 0), (8, 1, 64, [257, 64], 0), (3, 3, 96, [200], 0), (6, 2, 32, [127, 130], 0),
    (2, 1, 160, [70], 0), (4, 2, 128, [400], 100), (2, 2, 64, [333, 5], 64), (5, 5, 224, [66], 0), (2, 2, 192, [129], 7),
    # head sizes that are no multiple of 32: the last block of dims is half used
    (4, 2, 80, [300, 129, 1], 0), (3, 1, 16, [200, 65], 0), (2, 2, 48, [333], 40), (6, 3, 112, [257], 0),
    (2, 1, 144, [130], 0), (1, 1, 240, [70, 3], 0), (2, 2, 176, [129], 9), (2, 1, 208, [64], 0),
    # more blocks than the chip holds at once (heaviest first, not paired), and a long sequence
    (32, 8, 128, [600, 130, 577, 64], 0), (2, 1, 128, [2500, 40], 0)])
def test_attn_prefill_mfma(nh, nkv, hd, lens, window):
    """The matrix-core kernels over several blocks of 128 query rows and tiles of 64 keys: the one
    with one LDS buffer, the one with two (head sizes up to 128), and the library's own choice."""
    dtype = torch.bfloat16
    T = sum(lens)
    qkv = rnd(T, (nh + 2 * nkv) * hd, dtype=dtype, seed=17)
    cu = torch.tensor([0] + list(torch.tensor(lens).cumsum(0)), dtype=torch.int32)
    scale = 1.0 / math.sqrt(hd)
    want = R.attn_prefill(qkv, cu, len(lens), max(lens), nh, nkv, hd, scale, window)
    lib = ops()._lib()
    try:
        for which in (0, 2, 1):
            lib.illm_set_prefill_two_buffers(which)
            got = ops().attn_prefill(qkv.to(DEV), cu.to(DEV), len(lens), max(lens), nh, nkv, hd, scale, window)
            close(got, want, dtype, scale=2)
    finally:
        lib.illm_set_prefill_two_buffers(1)


@pytest.mark.parametrize("nh,nkv,hd,lens,window", [
    (4, 4, 128, [300, 129, 128, 1], 0), (8, 1, 64, [257, 64], 0), (3, 3, 96, [200], 0), (6, 2, 32, [127, 130], 0),
    (4, 2, 128, [400], 100), (2, 2, 64, [333, 5], 64), (2, 1, 32, [300], 7), (3, 1, 96, [31, 32, 33, 161], 33),
    (32, 8, 128, [600, 130, 577, 64], 0), (2, 1, 128, [1500, 40], 0)])
def test_attn_prefill_f32_matrix_cores(nh, nkv, hd, lens, window):
    """Float32 prompts with head sizes 32 to 128: the kernel on the matrix cores' float32
    instruction (blocks of 128 query rows, tiles of 32 keys) and the multiply-add kernel, both
    within the float32 budget of the plain implementation."""
    T = sum(lens)
    qkv = rnd(T, (nh + 2 * nkv) * hd, seed=19)
    cu = torch.tensor([0] + list(torch.tensor(lens).cumsum(0)), dtype=torch.int32)
    scale = 1.0 / math.sqrt(hd)
    want = R.attn_prefill(qkv, cu, len(lens), max(lens), nh, nkv, hd, scale, window)
    lib = ops()._lib()
    try:
        for on in (1, 0):
            lib.illm_set_attn_f32_mfma(on)
            got = ops().attn_prefill(qkv.to(DEV), cu.to(DEV), len(lens), max(lens), nh, nkv, hd, scale, window)
            close(got, want, torch.float32, scale=2)
    finally:
        lib.illm_set_attn_f32_mfma(1)


def test_attn_prefill_f32_finds_one_far_key():
    """One early key is made to stand out for a late query of another block and wave: the
    output is that key's value; a query before the key does not see it."""
    nh, nkv, hd, n = 2, 1, 128, 700
    qkv = rnd(n, (nh + 2 * nkv) * hd, seed=3)
    view = qkv.view(n, nh + 2 * nkv, hd)
    view[37, nh] = view[650, 1] * 30
    cu = torch.tensor([0, n], dtype=torch.int32)
    got = ops().attn_prefill(qkv.to(DEV), cu.to(DEV), 1, n, nh, nkv, hd, 1.0, 0).cpu().view(n, nh, hd)
    torch.testing.assert_close(got[650, 1], view[37, nh + nkv], atol=1e-4, rtol=1e-4)
    assert not torch.allclose(got[30, 1], view[37, nh + nkv], atol=0.1)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("nh,nkv,hd,starts,rows,page", [
    (4, 2, 32, [0, 70, 5], [40, 30, 1], 64), (8, 8, 128, [200, 0], [130, 64], 64), (3, 1, 48, [17, 64], [9, 200], 64),
    (6, 2, 24, [3], [5], 16), (2, 2, 256, [63], [66], 64), (32, 8, 128, [1000, 37, 0], [300, 27, 129], 64),
    (5, 5, 96, [130, 0], [131, 300], 32), (4, 1, 64, [31], [290], 16),
    (4, 2, 80, [70, 0], [200, 130], 64), (2, 1, 16, [5], [300], 64), (3, 3, 112, [129], [64], 128), (2, 1, 240, [64], [70], 64)])
def test_attn_prefill_paged(dtype, nh, nkv, hd, starts, rows, page):
    """A step's rows that go on from tokens the cache holds (a prompt cut into steps): attention
    over the paged cache at absolute positions, several sequences with different starts (0
    among them: a sequence that begins while others go on).  Stale rows of the pages are NaN."""
    lens = [s + r for s, r in zip(starts, rows)]
    pt, kc, vc, slots, _ = paged_case(dtype, nkv, hd, lens, page)
    for b, sl in enumerate(slots.tolist()):                    # rows beyond a sequence's end: NaN
        lp, r = divmod(lens[b], page)
        if r:
            kc[int(pt[sl, lp]), :, r:] = float("nan"); vc[int(pt[sl, lp]), :, r:] = float("nan")
    kc[-1] = float("nan"); vc[-1] = float("nan")
    T = sum(rows)
    qkv = rnd(T, (nh + 2 * nkv) * hd, dtype=dtype, seed=11)
    qkv[:, nh * hd:] = float("nan")                            # k and v come from the cache alone
    cu = torch.tensor([0] + list(torch.tensor(rows).cumsum(0)), dtype=torch.int32)
    st = torch.tensor(starts, dtype=torch.int32)
    scale = 1.0 / math.sqrt(hd)
    want = R.attn_prefill_paged(qkv, cu, slots, st, kc, vc, pt, page, 0, len(rows), max(rows), nh, nkv, hd,
                                scale, 0)
    lib = ops()._lib()
    try:
        # the library's own choice, and for bfloat16 the kernel with two LDS buffers forced
        # (head sizes 32 to 128 in steps of 32; the others do not have it)
        for which in ((1, 2) if dtype == torch.bfloat16 else (1,)):
            lib.illm_set_prefill_two_buffers(which)
            got = ops().attn_prefill_paged(qkv.to(DEV), cu.to(DEV), slots.to(DEV), st.to(DEV), kc.to(DEV),
                                           vc.to(DEV), pt.to(DEV), page, 0, len(rows), max(rows), nh, nkv, hd,
                                           scale, 0)
            assert torch.isfinite(got.float()).all()
            close(got, want, dtype, scale=2)
    finally:
        lib.illm_set_prefill_two_buffers(1)


def test_attn_prefill_paged_long_steps_with_a_window_ring():
    """Steps of 1,100 rows that go on from 1,500 and from 0 tokens (the kernel with two LDS buffers
    is the library's choice from 1,024 rows on): all keys, and a window of 500 keys over a ring of
    26 pages, which the longer sequence's 2,600 positions wrap round."""
    dtype, nh, nkv, hd, page = torch.bfloat16, 4, 2, 128, 64
    starts, rows = [1500, 0], [1100, 1030]
    lens = [s + r for s, r in zip(starts, rows)]
    qkv = rnd(sum(rows), (nh + 2 * nkv) * hd, dtype=dtype, seed=13)
    qkv[:, nh * hd:] = float("nan")
    cu = torch.tensor([0] + list(torch.tensor(rows).cumsum(0)), dtype=torch.int32)
    st = torch.tensor(starts, dtype=torch.int32)
    scale = 1.0 / math.sqrt(hd)
    for window, ring in ((0, 0), (500, 26)):
        pt, kc, vc, slots, _ = paged_case(dtype, nkv, hd, lens, page, ring=ring)
        got = ops().attn_prefill_paged(qkv.to(DEV), cu.to(DEV), slots.to(DEV), st.to(DEV), kc.to(DEV), vc.to(DEV),
                                       pt.to(DEV), page, ring, len(rows), max(rows), nh, nkv, hd, scale, window)
        want = R.attn_prefill_paged(qkv, cu, slots, st, kc, vc, pt, page, ring, len(rows), max(rows),
                                    nh, nkv, hd, scale, window)
        close(got, want, dtype, scale=2)


def test_attn_prefill_finds_one_far_key():
    """One early key is made to stand out for a late query: the output is that key's value."""
    nh, nkv, hd, n = 2, 1, 128, 700
    dtype = torch.bfloat16
    qkv = rnd(n, (nh + 2 * nkv) * hd, dtype=dtype, seed=3)
    view = qkv.view(n, nh + 2 * nkv, hd)
    view[37, nh] = view[650, 1].float().mul(30).to(dtype)          # key 37 matches query row 650, head 1
    cu = torch.tensor([0, n], dtype=torch.int32)
    got = ops().attn_prefill(qkv.to(DEV), cu.to(DEV), 1, n, nh, nkv, hd, 1.0, 0).cpu().view(n, nh, hd)
    close(got[650, 1], view[37, nh + nkv], dtype)
    assert not torch.allclose(got[30, 1].float(), view[37, nh + nkv].float(), atol=0.1)   # hidden from row 30


def paged_case(dtype, nkv, hd, lens, page, ring=0, seed=3):
    """Random cache contents laid out through a shuffled page table."""
    B = len(lens)
    per_seq = max((n + page - 1) // page for n in lens) if not ring else ring
    n_pages = B * per_seq + 3
    g = torch.Generator().manual_seed(seed)
    perm = torch.randperm(n_pages - 1, generator=g)[: B * per_seq].reshape(B, per_seq)
    pt = torch.full((B + 2, per_seq), n_pages - 1, dtype=torch.int32)
    slots = list(range(B, 0, -1))                    # slot numbers differ from batch order
    for b, s in enumerate(slots):
        pt[s] = perm[b].to(torch.int32)
    kc, vc = rnd(n_pages, nkv, page, hd, dtype=dtype, seed=seed + 1), rnd(n_pages, nkv, page, hd, dtype=dtype, seed=seed + 2)
    return pt, kc, vc, torch.tensor(slots, dtype=torch.int32), torch.tensor(lens, dtype=torch.int32)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("nh,nkv,hd,lens,window,nsplit", [
    (4, 4, 16, [7], 0, 1), (4, 2, 24, [5, 11, 2], 0, 2), (32, 2, 128, [300, 70], 0, 3),
    (3, 1, 48, [33, 64, 1, 600], 0, 4), (2, 2, 256, [257], 0, 2), (4, 2, 32, [90, 17, 700], 13, 2),
    (5, 5, 16, [130, 520], 64, 5)])
def test_attn_decode(dtype, nh, nkv, hd, lens, window, nsplit):
    page = 16
    ring = 0
    if window:
        ring = (window + page - 2) // page + 1
    pt, kc, vc, slots, seq_len = paged_case(dtype, nkv, hd, lens, page, ring)
    B = len(lens)
    qkv = rnd(B, (nh + 2 * nkv) * hd, dtype=dtype, seed=11)
    scale = 1.0 / math.sqrt(hd)
    got = ops().attn_decode(qkv.to(DEV), kc.to(DEV), vc.to(DEV), pt.to(DEV), page, ring, slots.to(DEV),
                            seq_len.to(DEV), nh, nkv, hd, scale, window, nsplit)
    want = R.attn_decode(qkv, kc, vc, pt, page, ring, slots, seq_len, nh, nkv, hd, scale, window, nsplit)
    close(got, want, dtype, scale=2)


@pytest.mark.parametrize("nh,nkv,hd,lens,window,nsplit", [
    (32, 32, 128, [600, 1, 64, 65], 0, 1), (32, 8, 128, [300, 70], 0, 3), (4, 4, 16, [7, 200], 0, 2),
    (8, 1, 64, [1000], 0, 32), (6, 2, 24, [5, 11, 130], 0, 2), (16, 1, 256, [257, 31], 0, 2),
    (5, 5, 96, [130, 520], 70, 5), (12, 4, 32, [90, 17, 700], 13, 2), (3, 3, 8, [129], 0, 1),
    (20, 2, 48, [333], 0, 4), (64, 8, 128, [1000, 63], 0, 5), (32, 8, 64, [129], 0, 1), (6, 3, 96, [70, 700], 0, 3),
    (34, 2, 32, [200], 0, 2), (8, 2, 160, [90, 300], 50, 2), (10, 5, 224, [65], 0, 1),
    # long contexts, the most splits, both kernels (plain and grouped heads)
    (8, 8, 128, [8192, 16001], 0, 16), (16, 2, 128, [12000, 5], 0, 16)])
def test_attn_decode_bf16_pages_of_64(nh, nkv, hd, lens, window, nsplit):
    """The fast bfloat16 kernel (pages of 64 rows, as the engine's cache has them); stale rows
    of the pages are NaN and must not leak into the result."""
    dtype, page = torch.bfloat16, 64
    ring = (window + page - 2) // page + 1 if window else 0
    pt, kc, vc, slots, seq_len = paged_case(dtype, nkv, hd, lens, page, ring)
    for b, s in enumerate(slots.tolist()):
        n = lens[b]
        if not ring:
            lp, r = divmod(n, page)
            if r:
                kc[int(pt[s, lp]), :, r:] = float("nan"); vc[int(pt[s, lp]), :, r:] = float("nan")
    kc[-1] = float("nan"); vc[-1] = float("nan")
    B = len(lens)
    qkv = rnd(B, (nh + 2 * nkv) * hd, dtype=dtype, seed=11)
    scale = 1.0 / math.sqrt(hd)
    want = R.attn_decode(qkv, kc, vc, pt, page, ring, slots, seq_len, nh, nkv, hd, scale, window, nsplit)
    for waves in (1, 2, 3, 8):                  # waves of a block that share a key range
        got = ops().attn_decode(qkv.to(DEV), kc.to(DEV), vc.to(DEV), pt.to(DEV), page, ring, slots.to(DEV),
                                seq_len.to(DEV), nh, nkv, hd, scale, window, nsplit, waves)
        close(got, want, dtype, scale=2)


@pytest.mark.parametrize("nh,nkv,hd,lens,window,nsplit", [(32, 8, 128, [650, 90, 3000], 0, 4), (12, 4, 32, [90, 17, 700], 13, 2),
                                                          (64, 8, 128, [1000, 63], 0, 5), (34, 2, 64, [200, 129], 0, 1)])
def test_both_grouped_head_decode_kernels_agree(nh, nkv, hd, lens, window, nsplit):
    """Grouped heads up to head size 128 run with both products on the matrix cores; the kernel
    with P.V on the vector units (which larger head sizes still use) must give the same."""
    o = ops()
    dtype, page = torch.bfloat16, 64
    ring = (window + page - 2) // page + 1 if window else 0
    pt, kc, vc, slots, seq_len = paged_case(dtype, nkv, hd, lens, page, ring)
    qkv = rnd(len(lens), (nh + 2 * nkv) * hd, dtype=dtype, seed=11)
    args = (qkv.to(DEV), kc.to(DEV), vc.to(DEV), pt.to(DEV), page, ring, slots.to(DEV), seq_len.to(DEV),
            nh, nkv, hd, 1.0 / math.sqrt(hd), window, nsplit, 4)
    new = o.attn_decode(*args)
    try:
        o._lib().illm_set_gqa_pv_on_matrix_cores(0)
        old = o.attn_decode(*args)
    finally:
        o._lib().illm_set_gqa_pv_on_matrix_cores(1)
    want = R.attn_decode(qkv, kc, vc, pt, page, ring, slots, seq_len, nh, nkv, hd, 1.0 / math.sqrt(hd), window, nsplit)
    close(new, want, dtype, scale=2)
    close(old, want, dtype, scale=2)
    close(new, old.float(), dtype, scale=2)


def test_linear_add_over_a_short_k_in_one_piece_a_wave():
    """K up to 4096 with at most 512 tiles runs with 8 waves that each take their share of K at
    once; the looping variant sums in another order and must agree to rounding."""
    o = ops()
    for M, N, K in ((8, 4096, 4096), (16, 2048, 1024), (3, 520, 4096), (1, 8192, 2048)):
        x, w = rnd(M, K, dtype=torch.bfloat16, seed=1), rnd(N, K, dtype=torch.bfloat16, seed=2)
        nw = (1 + rnd(N, seed=4) * 0.3).to(torch.bfloat16)
        into = rnd(M, N, seed=3) * 10
        wc = _plain_copy(w.to(DEV))
        outs = []
        for on in (1, 0):
            try:
                o._lib().illm_set_skinny_one_shot(on)
                dev = into.clone().to(DEV)
                rows = o.linear_add(x.to(DEV), wc, dev, (nw.to(DEV), 1e-5))
            finally:
                o._lib().illm_set_skinny_one_shot(1)
            outs.append((dev, rows))
        want = into.double() + R.linear(x, w, torch.float64)
        for dev, rows in outs:
            torch.testing.assert_close(dev.double().cpu(), want, atol=2e-4 * math.sqrt(K), rtol=1e-5)
            close(rows.xb, want * nw.double(), torch.bfloat16, scale=float(want.abs().max()))
            torch.testing.assert_close(rows.ssq.double().sum(1).cpu(), (want ** 2).sum(1), rtol=1e-5, atol=1e-6)


@pytest.mark.parametrize("ydt", DTYPES)
@pytest.mark.parametrize("M,N,K", [(1, 2, 128), (4, 128, 128), (8, 4096, 4096), (1, 32000, 4096), (16, 411, 80),
                                   (17, 100, 1000), (33, 64, 1008), (48, 31, 8), (64, 4096, 11008), (7, 12288, 4096),
                                   (64, 33, 40)])
def test_gemm_skinny(ydt, M, N, K):
    x, w = rnd(M, K, dtype=torch.bfloat16, seed=1), rnd(N, K, dtype=torch.bfloat16, seed=2)
    got = ops().gemm_skinny_bf16(x.to(DEV), w.to(DEV), ydt)
    close(got, R.linear(x, w, ydt), ydt, scale=math.sqrt(K))
    if ydt == torch.float32:       # float32 out keeps the accumulator: far tighter than bfloat16
        torch.testing.assert_close(got.double().cpu(), R.linear(x, w, torch.float64), atol=2e-4 * math.sqrt(K), rtol=1e-4)


@pytest.mark.parametrize("M,F,K", [(1, 11008, 4096), (8, 172, 64), (16, 200, 80), (3, 33, 1000), (40, 50, 64)])
def test_gate_up_silu(M, F, K):
    x = rnd(M, K, dtype=torch.bfloat16, seed=1)
    w = rnd(2 * F, K, dtype=torch.bfloat16, seed=2, std=0.2)
    got = ops().gate_up_silu(x.to(DEV), w.to(DEV))
    g, u = R.linear(x, w[:F], torch.float64), R.linear(x, w[F:], torch.float64)
    want = g / (1 + torch.exp(-g)) * u
    close(got, want, torch.bfloat16, scale=max(1.0, float(want.abs().max())))
    swapped = u / (1 + torch.exp(-u)) * g
    assert not torch.allclose(got.double().cpu(), swapped, atol=0.1 * float(want.abs().max()))


@pytest.mark.parametrize("ydt", DTYPES)
@pytest.mark.parametrize("M,N,K", [(1, 4096, 4096), (8, 100, 136), (16, 33, 1000), (5, 320, 96), (3, 7, 4), (9, 11008, 4096),
                                   (17, 100, 136), (64, 320, 96), (100, 33, 1000), (128, 4096, 512)])
def test_gemv_rows_f32(ydt, M, N, K):
    """The 32-bit path's product of few rows: float32 sums, W read once for every 16 rows; a
    row's result is the same bits whatever rows stand beside it."""
    x, w = rnd(M, K, seed=1), rnd(N, K, seed=2)
    assert ops().gemv_rows_f32_fits(x.to(DEV), w.to(DEV))
    got = ops().gemv_rows_f32(x.to(DEV), w.to(DEV), ydt)
    want = R.linear(x, w, torch.float64)
    if ydt == torch.float32:
        torch.testing.assert_close(got.double().cpu(), want, atol=2e-6 * math.sqrt(K) * 4, rtol=1e-5)
    else:
        close(got, want, ydt, scale=math.sqrt(K))
    if ydt == torch.float32 and M > 1:
        alone = ops().gemv_rows_f32(x[M - 1:].contiguous().to(DEV), w.to(DEV), ydt)
        assert torch.equal(alone[0], got[M - 1])
    if K % 32 or M < ops().ROWS_F32_MFMA_FROM:
        assert torch.equal(ops().linear(x.to(DEV), w.to(DEV), ydt), got)
    assert not ops().gemv_rows_f32_fits(rnd(129, K).to(DEV), w.to(DEV))
    assert not ops().gemv_rows_f32_fits(x.to(DEV).to(torch.bfloat16), w.to(DEV))


@pytest.mark.parametrize("ydt", DTYPES)
@pytest.mark.parametrize("M,N,K", [(1, 4096, 4096), (8, 100, 160), (16, 33, 992), (5, 320, 96), (3, 7, 32), (9, 11008, 4096),
                                   (17, 100, 256), (64, 320, 96), (100, 33, 1024), (128, 4096, 512), (70, 16400, 64),
                                   (33, 22016, 4096)])
def test_gemm_rows_f32_mfma(ydt, M, N, K):
    """The 32-bit path's product of up to 128 rows on the matrix cores' float32 instruction:
    float32 accuracy, edges, one and two tiles of W a block with the same bits, and a row's result
    the same bits whatever rows stand beside it."""
    x, w = rnd(M, K, seed=1), rnd(N, K, seed=2)
    assert ops().gemm_rows_f32_mfma_fits(x.to(DEV), w.to(DEV))
    got = ops().gemm_rows_f32_mfma(x.to(DEV), w.to(DEV), ydt)
    if M >= ops().ROWS_F32_MFMA_FROM:
        assert torch.equal(ops().linear(x.to(DEV), w.to(DEV), ydt), got)
    want = R.linear(x, w, torch.float64)
    if ydt == torch.float32:
        torch.testing.assert_close(got.double().cpu(), want, atol=2e-6 * math.sqrt(K) * 4, rtol=1e-5)
    else:
        close(got, want, ydt, scale=math.sqrt(K))
    lib = ops()._lib()
    try:
        for tiles in (1, 2):
            lib.illm_set_rows_f32_tiles(tiles)
            assert torch.equal(ops().gemm_rows_f32_mfma(x.to(DEV), w.to(DEV), ydt), got)
    finally:
        lib.illm_set_rows_f32_tiles(0)
    if M > 1:
        alone = ops().gemm_rows_f32_mfma(x[M - 1:].contiguous().to(DEV), w.to(DEV), ydt)
        assert torch.equal(alone[0], got[M - 1])
    assert not ops().gemm_rows_f32_mfma_fits(rnd(129, K).to(DEV), w.to(DEV))
    assert not ops().gemm_rows_f32_mfma_fits(rnd(M, K + 16).to(DEV), rnd(N, K + 16).to(DEV))


@pytest.mark.parametrize("ydt", DTYPES)
@pytest.mark.parametrize("M,N,K", [(129, 128, 16), (130, 33, 48), (200, 411, 80), (257, 129, 1008), (1, 5, 32),
                                   (300, 1000, 4096), (2048, 130, 512)])
def test_gemm_f32_mfma(ydt, M, N, K):
    """The 32-bit path's product of many rows, on the matrix cores' float32 instruction: float32
    accuracy (a product with operands rounded to a shorter type would miss this budget by two
    orders), edges that are no multiple of the tile, and a row's result the same bits wherever
    it stands in the batch."""
    x, w = rnd(M, K, seed=1), rnd(N, K, seed=2)
    assert ops().gemm_f32_mfma_fits(x.to(DEV), w.to(DEV))
    got = ops().gemm_f32_mfma(x.to(DEV), w.to(DEV), ydt)
    want = R.linear(x, w, torch.float64)
    if ydt == torch.float32:
        torch.testing.assert_close(got.double().cpu(), want, atol=2e-6 * math.sqrt(K) * 4, rtol=1e-5)
    else:
        close(got, want, ydt, scale=math.sqrt(K))
    if ydt == torch.float32 and M > 2:
        part = ops().gemm_f32_mfma(x[M // 2 + 1:].contiguous().to(DEV), w.to(DEV), ydt)
        assert torch.equal(part, got[M // 2 + 1:])
    if M > 128:
        assert torch.equal(ops().linear(x.to(DEV), w.to(DEV), ydt), got)
    assert not ops().gemm_f32_mfma_fits(rnd(M, K + 8).to(DEV), rnd(N, K + 8).to(DEV))
    assert not ops().gemm_f32_mfma_fits(x.to(DEV).to(torch.bfloat16), w.to(DEV))


def _decode_copy(w, mode="plain", **geometry):
    o = ops()
    return o.Weight(w, o.tile_weight(w, o.tile_rows(w.shape[0], mode, **geometry)), mode)


def test_tile_rows_cover_every_row_once():
    o = ops()
    for rows, N in ((o.tile_rows(100), 100), (o.tile_rows(2 * 44, "gate_up"), 88),
                    (o.tile_rows((6 + 2 * 3) * 48, "qkv", nh=6, nkv=3, hd=48), 12 * 48)):
        assert rows.shape[1] == 16
        kept = rows[rows >= 0]
        assert sorted(kept.tolist()) == list(range(N))
    g = o.tile_rows(2 * 44, "gate_up")
    assert g[5, :8].tolist() == [40, 41, 42, 43, -1, -1, -1, -1] and g[5, 8:12].tolist() == [84, 85, 86, 87]
    q = o.tile_rows((2 + 2) * 32, "qkv", nh=2, nkv=1, hd=32)
    assert q[1].tolist() == list(range(8, 16)) + list(range(24, 32))          # a row and its partner hd/2 on
    assert q[-1].tolist() == list(range(3 * 32 + 16, 4 * 32))                  # v: 16 rows in a run


@pytest.mark.parametrize("M,N,K", [(1, 4096, 4096), (8, 100, 160), (16, 33, 992), (5, 320, 96), (9, 4096, 11008),
                                   (8, 16400, 64)])      # 1025 tiles: two a block, the last block has one
def test_products_from_the_decode_copy_equal_those_from_the_matrix(M, N, K, monkeypatch):
    """The copy laid out for the few-rows kernels holds the same numbers in another order: with
    K cut over the same number of waves the products are the same sums in the same order, bit
    for bit."""
    o = ops()
    for knob in ("PLAIN_WAVES", "GATE_UP_WAVES", "QKV_ROPE_WAVES"):
        monkeypatch.setattr(o, knob, 3)
    x, w = rnd(M, K, dtype=torch.bfloat16, seed=1).to(DEV), rnd(N, K, dtype=torch.bfloat16, seed=2).to(DEV)
    wc = _decode_copy(w)
    assert wc.tiled.shape == ((N + 15) // 16, K // 32, 16, 32)
    for ydt in DTYPES:
        assert torch.equal(o.linear(x, wc, ydt), o.linear(x, w, ydt))
    into_a, into_b = rnd(M, N, seed=3).to(DEV), rnd(M, N, seed=3).to(DEV)
    nw = (1 + rnd(N, seed=4) * 0.3).to(torch.bfloat16).to(DEV)
    ra, rb = o.linear_add(x, wc, into_a, (nw, 1e-5)), o.linear_add(x, w, into_b, (nw, 1e-5))
    assert torch.equal(into_a, into_b)
    if ra is not None:
        assert torch.equal(ra.xb, rb.xb) and torch.equal(ra.ssq, rb.ssq)
        w2 = rnd(48, N, dtype=torch.bfloat16, seed=5).to(DEV)
        if N % 32 == 0:
            assert torch.equal(o.linear(ra, _decode_copy(w2)), o.linear(rb, w2))
    if K % 64 == 0:                                        # gate|up: N rows as two halves
        for F in (56, 8200):                               # 8200: 1025 tiles, two a block
            wg = rnd(2 * F, K, dtype=torch.bfloat16, seed=6, std=0.2).to(DEV)
            assert torch.equal(o.gate_up_silu(x, _decode_copy(wg, "gate_up")), o.gate_up_silu(x, wg))
    xl = rnd(17, K, dtype=torch.bfloat16, seed=7).to(DEV)     # more rows: the matrix itself is read
    assert torch.equal(o.linear(xl, wc), o.linear(xl, w))
    # a copy that follows another kernel's tiles is never read by the plain product
    if N % 2 == 0 and K % 64 == 0:
        other = _decode_copy(w, "gate_up")
        assert not torch.equal(other.tiled.view(-1)[: 16 * K], wc.tiled.view(-1)[: 16 * K]) or N <= 16
        assert torch.equal(o.linear(x, other), o.linear(x, w))


def test_products_of_many_rows_follow_the_plan_and_stay_right(monkeypatch):
    """A product of many rows runs whole or cut along its output columns as the plan's table
    says; a plan that measures times the candidates once per shape; whatever plan is taken,
    every element is the plain product."""
    o = ops()
    from inferllm_amd.kernels.plan import Plan
    M, N, K = 1100, 9000, 64
    x, w = rnd(M, K, dtype=torch.bfloat16, seed=1), rnd(N, K, dtype=torch.bfloat16, seed=2)
    fixed = Plan()
    monkeypatch.setattr(o, "_plan", fixed)
    whole = o.linear(x.to(DEV), w.to(DEV))
    assert not fixed.cuts                                  # no table entry: whole, nothing timed
    assert torch.equal(whole, torch.matmul(x.to(DEV), w.to(DEV).t()))
    fixed.cuts[(-(-M // 256), N, K)] = (4096,)
    cut = o.linear(x.to(DEV), w.to(DEV))
    close(cut, R.linear(x, w), torch.bfloat16, scale=math.sqrt(K))
    assert torch.equal(cut[:, :4096], torch.matmul(x.to(DEV), w.to(DEV)[:4096].t()))
    plan = Plan(measure=True)
    monkeypatch.setattr(o, "_plan", plan)
    got = o.linear(x.to(DEV), w.to(DEV))
    key = (-(-M // 256), N, K)
    assert key in plan.cuts and len(plan.cuts) == 1
    close(got, R.linear(x, w), torch.bfloat16, scale=math.sqrt(K))
    for cand in o._split_candidates(N):                    # every candidate gives the product
        assert all(0 < c < N for c in cand)
        close(o._run_plan(x.to(DEV), w.to(DEV), cand), R.linear(x, w), torch.bfloat16, scale=math.sqrt(K))
    big = rnd(2048, K, dtype=torch.bfloat16, seed=3)       # many rows: also as two halves
    cands = o._split_candidates(N, 2048)
    assert ("rows", 2) in cands and ("rows", 2) not in o._split_candidates(N, 1100)
    close(o._run_plan(big.to(DEV), w.to(DEV), ("rows", 2)), R.linear(big, w), torch.bfloat16, scale=math.sqrt(K))
    plan.cuts[(8, N, K)] = ("rows", 2)                     # ragged rows of that class run whole
    close(o.linear(big[:1900].to(DEV), w.to(DEV)), R.linear(big[:1900], w), torch.bfloat16, scale=math.sqrt(K))
    del plan.cuts[(8, N, K)]
    o.linear(x.to(DEV), w.to(DEV))
    assert len(plan.cuts) == 1                             # measured once
    o.linear(x[:1000].to(DEV), w.to(DEV))                  # fewer rows than planning is for
    assert len(plan.cuts) == 1
    # 65 to 255 rows: whole against filled up to 256 rows, once per shape and 32 rows
    few = x[:100].to(DEV)
    close(o.linear(few, w.to(DEV)), R.linear(x[:100], w), torch.bfloat16, scale=math.sqrt(K))
    assert plan.cuts.get(("pad", 4, N, K)) in ((), ("pad", 256)) and len(plan.cuts) == 2
    close(o._run_plan(few, w.to(DEV), ("pad", 256)), R.linear(x[:100], w), torch.bfloat16, scale=math.sqrt(K))
    into = torch.empty(100, N, dtype=torch.bfloat16, device=DEV)
    assert o._run_plan(few, w.to(DEV), ("pad", 256), into) is into
    close(into, R.linear(x[:100], w), torch.bfloat16, scale=math.sqrt(K))
    o.linear(x[:64].to(DEV), w.to(DEV))
    o.linear(x[:256].to(DEV), w.to(DEV))
    assert len(plan.cuts) == 2
    assert Plan.from_dict(plan.to_dict()) == plan


def _prepared_rows(M, K, nw_dtype, eps, seed=5):
    """Residual rows with unequal scales and a norm weight far from 1, as `linear_add(norm=)`
    leaves them (made here by adding a product of zeros), and their plain norm."""
    x = rnd(M, K, seed=seed) * torch.linspace(0.02, 3.0, M)[:, None]
    nw = (1 + rnd(K, seed=seed + 1) * 0.3).to(nw_dtype)
    want = R.add_rmsnorm(x.clone(), None, nw, eps, torch.bfloat16)
    zeros = torch.zeros(M, 8, dtype=torch.bfloat16, device=DEV)
    rows = ops().linear_add(zeros, torch.zeros(K, 8, dtype=torch.bfloat16, device=DEV),
                            x.clone().to(DEV), (nw.to(DEV), eps))
    assert rows is not None and torch.equal(rows.x.cpu(), x)
    return rows, want


@pytest.mark.parametrize("nw_dtype", DTYPES)
@pytest.mark.parametrize("ydt", DTYPES)
@pytest.mark.parametrize("M,N,K,eps", [(1, 4096, 4096, 1e-5), (8, 100, 136, 1e-6), (16, 33, 1000, 1e-2), (5, 320, 96, 1e-5)])
def test_gemm_skinny_takes_the_norm(nw_dtype, ydt, M, N, K, eps):
    """The product of rows whose norm was prepared against norm, then product."""
    rows, h = _prepared_rows(M, K, nw_dtype, eps)
    w = rnd(N, K, dtype=torch.bfloat16, seed=2)
    got = ops().linear(rows, w.to(DEV), ydt)
    # the kernel rounds x * weight to bfloat16 and scales the sums, the reference rounds the
    # normed rows: the operands differ by bfloat16 roundings whatever the output's dtype
    close(got, R.linear(h, w, ydt), torch.bfloat16, scale=math.sqrt(K))
    close(rows.rows(), h, torch.bfloat16)                  # and can still be had normalised


@pytest.mark.parametrize("M,F,K", [(1, 11008, 4096), (8, 172, 64), (16, 203, 80), (3, 33, 1000)])
def test_gate_up_silu_takes_the_norm(M, F, K):
    rows, h = _prepared_rows(M, K, torch.bfloat16, 1e-5)
    w = rnd(2 * F, K, dtype=torch.bfloat16, seed=2, std=0.2)
    got = ops().gate_up_silu(rows, w.to(DEV))
    g, u = R.linear(h, w[:F], torch.float64), R.linear(h, w[F:], torch.float64)
    want = g / (1 + torch.exp(-g)) * u
    close(got, want, torch.bfloat16, scale=max(1.0, float(want.abs().max())))
    if K % 64 == 0:
        # the same through the kernel that shares X through LDS, where the plan sends few rows to it
        o = ops()
        plan = o.current_plan()
        try:
            plan.rows_from[("gate_up", 2 * F, K)] = 1
            again = o.gate_up_silu(rows, _decode_copy(w.to(DEV), "gate_up"))
        finally:
            del plan.rows_from[("gate_up", 2 * F, K)]
        close(again, want, torch.bfloat16, scale=max(1.0, float(want.abs().max())))


@pytest.mark.parametrize("nw_dtype", [None] + DTYPES)
@pytest.mark.parametrize("M,N,K", [(1, 4096, 4096), (8, 4096, 11008), (16, 104, 136), (7, 33, 1000)])
def test_linear_add(M, N, K, nw_dtype):
    """into += x . w^T in float32, nothing but the sum is rounded; with a norm's weight also
    bfloat16(into * weight) and the rows' sums of squares in parts."""
    x, w = rnd(M, K, dtype=torch.bfloat16, seed=1), rnd(N, K, dtype=torch.bfloat16, seed=2)
    into = rnd(M, N, seed=3) * 10
    dev = into.clone().to(DEV)
    assert ops().linear_add_fits(x.to(DEV), w.to(DEV), dev)
    nw = None if nw_dtype is None else (1 + rnd(N, seed=4) * 0.3).to(nw_dtype)
    rows = ops().linear_add(x.to(DEV), w.to(DEV), dev, None if nw is None else (nw.to(DEV), 1e-5))
    want = into.double() + R.linear(x, w, torch.float64)
    torch.testing.assert_close(dev.double().cpu(), want, atol=2e-4 * math.sqrt(K), rtol=1e-5)
    if nw is None or N % 8:
        assert rows is None
    else:
        assert rows.x is dev and rows.ssq.shape == (M, (N + 15) // 16)
        close(rows.xb, want * nw.double(), torch.bfloat16, scale=float(want.abs().max()))
        torch.testing.assert_close(rows.ssq.double().sum(1).cpu(), (want ** 2).sum(1), rtol=1e-5, atol=1e-6)
    assert not ops().linear_add_fits(x.to(DEV), w.to(DEV), dev.to(torch.bfloat16))
    assert not ops().linear_add_fits(rnd(17, K, dtype=torch.bfloat16).to(DEV), w.to(DEV), torch.zeros(17, N, device=DEV))


def _plain_copy(w):
    o = ops()
    return o.Weight(w, o.tile_weight(w, o.tile_rows(w.shape[0], "plain")), "plain")


# rows in every count of 16-row tiles; N with a last tile of 4 rows, with fewer tiles than
# a block's waves, with tiles beyond a multiple of 4; K of one piece, of a partial last piece
@pytest.mark.parametrize("tiles_per_wave", [0, 1, 2])
@pytest.mark.parametrize("M,N,K,splits", [(17, 40, 96, 0), (33, 100, 224, 0), (64, 4096, 11008, 0),
                                          (50, 84, 1184, 5), (48, 20, 64, 1), (31, 72, 352, 3),
                                          (64, 36, 2048, 16), (20, 8192, 16384, 0),
                                          (1, 40, 96, 0), (7, 100, 224, 2), (16, 4096, 11008, 0),
                                          (65, 40, 96, 0), (100, 84, 1184, 4), (128, 4096, 11008, 0),
                                          (81, 36, 2048, 16), (97, 132, 352, 3), (113, 4096, 4096, 0), (128, 8192, 8192, 0)])
def test_linear_planes(M, N, K, splits, tiles_per_wave):
    """The product for up to 128 rows, K cut into ranges: the planes add up to x . w^T, and what
    `add_rmsnorm` makes of them is the residual add and norm of the product.  Beyond 64 rows one
    launch and two of 64 rows give the same bits."""
    o = ops()
    if N >= 8192 and tiles_per_wave:
        return                   # the large case is there for the library's own choice of tiles
    x, w = rnd(M, K, dtype=torch.bfloat16, seed=1), rnd(N, K, dtype=torch.bfloat16, seed=2)
    wc = _plain_copy(w.to(DEV))
    assert o.linear_planes_fits(x.to(DEV), wc)
    o._lib().illm_set_mid_tiles_per_wave(tiles_per_wave)
    try:
        planes = o.linear_planes(x.to(DEV), wc, splits)
    finally:
        o._lib().illm_set_mid_tiles_per_wave(0)
    assert planes.dtype == torch.float32 and planes.shape[1:] == (M, N)
    assert splits == 0 or planes.shape[0] == splits
    if M > 64:
        o._lib().illm_set_mid_tiles_per_wave(tiles_per_wave)
        o._lib().illm_set_mid_rows_a_launch(64)
        try:
            assert torch.equal(o.linear_planes(x.to(DEV), wc, splits), planes)
        finally:
            o._lib().illm_set_mid_tiles_per_wave(0)
            o._lib().illm_set_mid_rows_a_launch(128)
    want = R.linear(x, w, torch.float64)
    torch.testing.assert_close(planes.double().sum(0).cpu(), want, atol=2e-4 * math.sqrt(K), rtol=1e-5)
    into = rnd(M, N, seed=3) * 10
    nw = (1 + rnd(N, seed=4) * 0.3).to(torch.bfloat16)
    dev = into.clone().to(DEV)
    got = o.add_rmsnorm(dev, planes, nw.to(DEV), 1e-5, torch.bfloat16)
    ref_x = into.clone()
    close(got, R.add_rmsnorm(ref_x, want.float(), nw, 1e-5, torch.bfloat16), torch.bfloat16, scale=4.0)
    torch.testing.assert_close(dev.cpu(), ref_x, atol=2e-4 * math.sqrt(K), rtol=1e-5)


def test_linear_planes_refuses_what_it_does_not_take():
    o = ops()
    w = rnd(64, 256, dtype=torch.bfloat16).to(DEV)
    x = rnd(20, 256, dtype=torch.bfloat16).to(DEV)
    assert o.linear_planes_fits(x, _plain_copy(w))
    assert not o.linear_planes_fits(x, w)                                  # no decode copy
    assert o.linear_planes_fits(x[:16], _plain_copy(w)) and o.linear_planes_pays(x, _plain_copy(w))
    assert not o.linear_planes_fits(rnd(129, 256, dtype=torch.bfloat16).to(DEV), _plain_copy(w))
    assert not o.linear_planes_fits(x.float(), _plain_copy(w))
    wide = rnd(256, 256, dtype=torch.bfloat16).to(DEV)                      # K < 2 N: not up to 16 rows
    assert not o.linear_planes_fits(x[:16], _plain_copy(wide)) and o.linear_planes_fits(x, _plain_copy(wide))
    many = rnd(100, 256, dtype=torch.bfloat16).to(DEV)                      # from 17 rows K = N is taken
    assert o.linear_planes_fits(many, _plain_copy(wide)) and o.linear_planes_pays(many, _plain_copy(wide))
    assert not o.linear_planes_fits(many, _plain_copy(rnd(512, 256, dtype=torch.bfloat16).to(DEV)))
    gate_up = o.Weight(w, o.tile_weight(w, o.tile_rows(64, "gate_up")), "gate_up")
    assert not o.linear_planes_fits(x, gate_up)                            # another kernel's tile order
    with pytest.raises(Exception):
        o.linear_planes(x, w)
    y = torch.empty(2, 20, 64, device=DEV)
    assert o._lib().illm_gemm_mid_bf16(o._p(x), o._p(_plain_copy(w).tiled), o._p(y), 0, 20, 64, 250, 2, None) != 0
    assert o._lib().illm_gemm_mid_bf16(o._p(x), o._p(_plain_copy(w).tiled), o._p(y), 0, 129, 64, 256, 2, None) != 0
    assert o._lib().illm_gemm_mid_bf16(o._p(x), o._p(_plain_copy(w).tiled), o._p(y), 0, 20, 64, 256, 3, None) != 0


@pytest.mark.parametrize("dtype", DTYPES)
def test_attn_decode_finds_one_far_key(dtype):
    """One key among hundreds is made to stand out: the output must be its value."""
    nh, nkv, hd, page, n = 4, 2, 32, 16, 777
    pt, kc, vc, slots, seq_len = paged_case(dtype, nkv, hd, [n], page)
    qkv = rnd(1, (nh + 2 * nkv) * hd, dtype=dtype, seed=1)
    target = 5
    pg, r = R.cache_offsets(pt, int(slots[0]), target, page, 0)
    q = qkv.view(1, nh + 2 * nkv, hd)
    for kvh in range(nkv):
        kc[pg, kvh, r] = q[0, kvh * (nh // nkv)].float().mul(40).to(dtype)   # huge score for head kvh*per
    got = ops().attn_decode(qkv.to(DEV), kc.to(DEV), vc.to(DEV), pt.to(DEV), page, 0, slots.to(DEV),
                            seq_len.to(DEV), nh, nkv, hd, 1.0, 0, 4).cpu().view(nh, hd)
    for kvh in range(nkv):
        close(got[kvh * (nh // nkv)], vc[pg, kvh, r], dtype)


@pytest.mark.parametrize("B,V", [(1, 256), (3, 320), (2, 32000), (64, 411), (1, 128256), (5, 128256), (64, 32000),
                                 (9, 4099)])
def test_argmax(B, V):
    logits = rnd(B, V, seed=4)
    logits[0, V - 1] = 50.0
    if B > 1:
        logits[1, 3] = 60.0; logits[1, 200] = 60.0           # a tie: the lower id wins
    got = ops().argmax(logits.to(DEV)).cpu()
    assert got.tolist() == R.argmax(logits).tolist()
    assert got[0] == V - 1 and (B == 1 or got[1] == 3)
    # ties across the parts a long row is cut into, a NaN above everything, a row of NaN alone
    logits[0, V - 1] = 0.0
    logits[0, 5] = 70.0; logits[0, V - 2] = 70.0; logits[0, V // 2] = float("nan")
    if B > 2:
        logits[2] = float("nan")
    got = ops().argmax(logits.to(DEV)).cpu()
    assert got[0] == 5 and (B <= 2 or got[2] == 0)
    assert got.tolist()[3:] == R.argmax(logits).tolist()[3:]


def interval_ok(logits_row, token, u, temperature, top_k, top_p, penalty, last):
    """The drawn token's interval of the id-ordered CDF over the kept ids contains u (with slack)."""
    ids, p = R.kept_distribution(logits_row, temperature, top_k, top_p, penalty, last)
    pairs = sorted(zip(ids, p.tolist()))
    cum = 0.0
    for i, pi in pairs:
        if i == token:
            return cum - 1e-4 <= u <= cum + pi + 1e-4
        cum += pi
    return False


def test_the_uniform_numbers_of_the_tests_and_of_the_host_side_agree():
    """The tests state the sampler's hash themselves (kernel_refs.uniform), pinned by the
    published first outputs of splitmix64; the host side's `uniform`, which the generation loop
    would use, must be the same function."""
    from inferllm_amd.sampling.params import request_seed, uniform
    assert [R.mix64(i * 0x9E3779B97F4A7C15) for i in (1, 2, 3)] == \
        [0xE220A8397B1DCDAF, 0x6E789E6AA1B965F4, 0x06C45D188009454F]
    for seed in (0, 3, 2**63 + 5, (1 << 64) - 1):
        for c in (0, 1, 77):
            assert uniform(seed, c) == R.uniform(seed, c)
            assert 0.0 <= R.uniform(seed, c) < 1.0
    assert len({R.uniform(request_seed(9, i), c) for i in range(4) for c in range(64)}) > 250


@pytest.mark.parametrize("V,temperature,top_k,top_p,penalty", [
    (256, 0.8, 0, 1.0, 1.0), (320, 0.8, 40, 0.95, 1.1), (411, 0.1, 40, 0.95, 1.3), (1000, 1.5, 5, 1.0, 1.0),
    (32000, 1.0, 0, 0.9, 1.0), (300, 0.7, 1, 1.0, 1.0), (128256, 0.9, 50, 0.8, 1.2),
    (2000, 0.9, 1024, 0.7, 1.1), (2000, 0.9, 1025, 0.7, 1.0), (50, 1.0, 49, 0.5, 1.0), (32000, 0.1, 40, 0.95, 1.1),
    # rows too long for a thread's registers: top_p alone, with a large top_k, temperature alone
    (128256, 0.9, 0, 0.8, 1.2), (40000, 1.0, 2000, 0.6, 1.0), (33000, 0.7, 0, 0.999, 1.0), (50000, 1.3, 0, 1.0, 1.0),
    # long rows with a small top_k are cut into parts that blocks of their own take: a length that
    # no part divides, the largest top_k of that way and the first beyond it
    (70001, 0.1, 40, 0.95, 1.1), (65536, 1.0, 64, 0.5, 1.0), (65536, 1.0, 65, 0.5, 1.3), (200003, 0.8, 3, 1.0, 1.3),
    # long rows without top_k: several blocks a row and a kernel a pass
    (70001, 0.7, 0, 0.9, 1.0), (131072, 1.0, 0, 1.0, 1.1), (200003, 0.5, 0, 0.5, 1.3), (65536, 2.0, 0, 0.999, 1.0),
    (65537, 0.3, 0, 0.05, 1.0), (16384, 0.9, 0, 0.7, 1.2), (16387, 1.1, 0, 1.0, 1.0)])
def test_sample_draws_from_the_reference_distribution(V, temperature, top_k, top_p, penalty):
    uniform = R.uniform                                      # the tests' own statement of the hash
    B = 6
    logits = rnd(B, V, seed=8, std=2.0)
    logits[2] = 0.0                                            # all equal: ties everywhere
    last = torch.full((B, 8), -1, dtype=torch.int32)
    last[:, :4] = torch.tensor([1, 5, V - 1, 5], dtype=torch.int32)     # an id twice: penalised once
    seeds = torch.tensor([3, 99, 12345, -7, 2**62, 0], dtype=torch.int64)
    counters = torch.tensor([0, 1, 2, 3, 4, 5], dtype=torch.int32)
    got = ops().sample(logits.to(DEV), temperature, top_k, top_p, penalty,
                       last.to(DEV) if penalty != 1.0 else None, seeds.to(DEV), counters.to(DEV)).cpu().tolist()
    for b in range(B):
        u = uniform(int(seeds[b]) & ((1 << 64) - 1), int(counters[b]))
        assert interval_ok(logits[b], got[b], u, temperature, top_k, top_p, penalty,
                           last[b] if penalty != 1.0 else None), (b, got[b], u)
    if top_k == 1:
        assert got == torch.argmax(logits, -1).tolist() or penalty != 1.0


def test_sample_of_a_long_row_in_parts_keeps_what_one_block_would():
    """A long row with a small top_k is the work of several blocks, each with a stretch of the ids.
    Equal scores at the k-th place go to the lower ids, wherever the stretches' edges lie: of 90 equal
    scores spread over the whole row, the 40 with the lowest ids are kept, and every draw is one of them."""
    V, B, top_k = 131072, 64, 40
    logits = rnd(B, V, seed=21, std=1.0).clamp_(max=3.0)
    high = torch.arange(90) * 1451 + 7                        # up to id 129,146: in every stretch
    logits[:, high] = 9.0
    logits[1, high[:5]] = 12.0                                # row 1: five above, then 35 of the 85 equal ones
    seeds = torch.arange(B, dtype=torch.int64) * 104729 + 3
    counters = torch.arange(B, dtype=torch.int32)
    got = ops().sample(logits.to(DEV), 1.0, top_k, 1.0, 1.0, None, seeds.to(DEV), counters.to(DEV)).cpu()
    kept = set(high[:top_k].tolist())
    assert all(int(t) in kept for t in got), [int(t) for t in got if int(t) not in kept]
    assert len({int(t) for t in got}) > 20                    # and not always the same few
    for b in range(B):
        u = R.uniform(int(seeds[b]), int(counters[b]))
        assert interval_ok(logits[b], int(got[b]), u, 1.0, top_k, 1.0, 1.0, None), (b, int(got[b]), u)


@pytest.mark.parametrize("top_p", [1.0, 0.9, 0.3])
def test_sample_of_a_long_row_does_not_depend_on_its_company(top_p):
    """Rows of 16,384 ids and more without top_k are cut into more or fewer parts depending on how
    many rows there are; the masses are added as integers, so a row draws the same id alone and
    among 69 others, draw after draw."""
    V = 100003
    rows = rnd(70, V, seed=33, std=3.0)
    seeds = torch.arange(70, dtype=torch.int64) * 7919 + 5
    last = torch.randint(0, V, (70, 16), generator=torch.Generator().manual_seed(2), dtype=torch.int32)
    for counter in (0, 1, 2):
        counters = torch.full((70,), counter, dtype=torch.int32)
        together = ops().sample(rows.to(DEV), 0.8, 0, top_p, 1.2, last.to(DEV), seeds.to(DEV), counters.to(DEV)).cpu()
        for b in (0, 13, 69):
            alone = ops().sample(rows[b:b + 1].to(DEV), 0.8, 0, top_p, 1.2, last[b:b + 1].to(DEV),
                                 seeds[b:b + 1].to(DEV), counters[b:b + 1].to(DEV)).cpu()
            assert int(alone[0]) == int(together[b]), (b, counter)
        few = ops().sample(rows[:9].to(DEV), 0.8, 0, top_p, 1.2, last[:9].to(DEV), seeds[:9].to(DEV),
                           counters[:9].to(DEV)).cpu()
        assert few.tolist() == together[:9].tolist()


def test_sample_frequencies_match_probabilities():
    V, n = 7, 4000
    row = torch.tensor([2.0, 1.0, 0.5, 0.0, -1.0, 1.5, -3.0])
    logits = row.repeat(n, 1)
    seeds = torch.arange(n, dtype=torch.int64) * 7919 + 1
    counters = torch.zeros(n, dtype=torch.int32)
    got = ops().sample(logits.to(DEV), 0.9, 0, 1.0, 1.0, None, seeds.to(DEV), counters.to(DEV)).cpu()
    freq = torch.bincount(got.long(), minlength=V).double() / n
    p = torch.softmax(row.double() / 0.9, 0)
    chi2 = float((n * (freq - p) ** 2 / p).sum())
    assert chi2 < 30.0, (chi2, freq, p)           # 6 degrees of freedom: far beyond any honest draw


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("hd", [32, 24])
def test_window_edge_prefill_and_decode(dtype, hd):
    """A key that stands out sits exactly at the window's edge: the query `window - 1` places
    after it still sees it, the next query does not (prefill), and likewise for a single new
    token over the cache (decode)."""
    nh, nkv, n, window, edge = 2, 2, 150, 40, 70
    qkv = rnd(n, (nh + 2 * nkv) * hd, dtype=dtype, seed=5, std=0.3)
    view = qkv.view(n, nh + 2 * nkv, hd)
    probe = rnd(hd, seed=6).to(dtype)
    view[:, 0] = probe                                   # every query of head 0 looks for the probe
    view[edge, nh] = probe.float().mul(25).to(dtype)     # and key `edge` answers it loudly
    view[edge, nh + nkv] = 7.0                           # its value is unmistakable
    cu = torch.tensor([0, n], dtype=torch.int32)
    out = ops().attn_prefill(qkv.to(DEV), cu.to(DEV), 1, n, nh, nkv, hd, 1.0, window).cpu().view(n, nh, hd).float()
    last_seeing = edge + window - 1
    assert float(out[last_seeing, 0].mean()) > 6.5       # still inside the window
    assert float(out[last_seeing + 1, 0].mean()) < 3.0   # one step further: gone
    assert float(out[edge - 1, 0].mean()) < 3.0          # and the future is hidden
    want = R.attn_prefill(qkv, cu, 1, n, nh, nkv, hd, 1.0, window)
    close(out.reshape(n, -1), want, dtype, scale=8)
    # decode: cache holds keys 0..L-1 (the last one is the new token's)
    page = 64
    ring = (window + page - 2) // page + 1
    for L, sees in ((edge + window, True), (edge + window + 1, False)):
        pt = torch.tensor([[3, 1, 0][:ring] + [2] * max(0, ring - 3)], dtype=torch.int32)[:, :ring]
        kc = torch.full((4, nkv, page, hd), float("nan"), dtype=dtype); vc = kc.clone()
        for pos in range(max(0, L - ring * page), L):    # what a ring keeps
            pg = int(pt[0, (pos // page) % ring])
            if pos // page + ring > (L - 1) // page:
                kc[pg, :, pos % page] = view[pos, nh:nh + nkv]; vc[pg, :, pos % page] = view[pos, nh + nkv:]
        q = view[L - 1:L].reshape(1, -1).contiguous()
        got = ops().attn_decode(q.to(DEV), kc.to(DEV), vc.to(DEV), pt.to(DEV), page, ring,
                                torch.zeros(1, dtype=torch.int32, device=DEV),
                                torch.tensor([L], dtype=torch.int32, device=DEV), nh, nkv, hd, 1.0, window, 2)
        mean = float(got.cpu().view(nh, hd)[0].float().mean())
        assert (mean > 6.5) == sees, (L, mean)
        close(got.cpu().view(nh, hd), out[L - 1], dtype, scale=8)


_QKV_SHAPES = [(1, 32, 32, 128, 4096), (8, 4, 2, 32, 64), (16, 6, 3, 64, 200), (3, 8, 1, 96, 72),
               (5, 3, 3, 48, 136), (2, 2, 1, 16, 40), (5, 3, 3, 48, 160), (7, 2, 2, 16, 96),
               (13, 3, 3, 48, 192), (16, 8, 2, 128, 1024)]


# with the decode copy only where one can be made (K a multiple of 32)
@pytest.mark.parametrize("M,nh,nkv,hd,K,copy", [s + (c,) for s in _QKV_SHAPES for c in (False, True)
                                                if not (c and s[4] % 32)])
@pytest.mark.parametrize("normed", [False, True])
@pytest.mark.parametrize("shared_x", [False, True])
def test_qkv_rope_store_equals_the_three_steps(M, nh, nkv, hd, K, normed, copy, shared_x, monkeypatch):
    """The fused decode kernel against (norm,) product, then rotation and cache store.
    `shared_x`: the plan sends these few rows to the kernel that shares X through LDS
    (csrc/gemm_rows.hip), which needs the decode copy and K a multiple of 64."""
    from inferllm_amd.parts.position import rotary_table
    if shared_x:
        if not copy or K % 64:
            pytest.skip("the shared-X kernel needs the decode copy and K % 64 == 0")
        monkeypatch.setitem(ops().current_plan().rows_from, ("qkv", (nh + 2 * nkv) * hd, K), 1)
    dtype, page = torch.bfloat16, 64
    table = rotary_table(777.0, hd, 300, "cpu")
    x = rnd(M, K, dtype=dtype, seed=1)
    x_dev = x.to(DEV)
    if normed:
        x_dev, x = _prepared_rows(M, K, torch.bfloat16, 1e-5)
    w = rnd((nh + 2 * nkv) * hd, K, dtype=dtype, seed=2, std=0.1)
    pos = torch.tensor([(37 * i + 5) % 290 for i in range(M)], dtype=torch.int32)
    slot = torch.randperm(M + 2, generator=torch.Generator().manual_seed(9))[:M].to(torch.int32)
    assert len(set(slot.tolist())) == M
    g = torch.Generator().manual_seed(4)
    pt = torch.randperm((M + 2) * 5, generator=g).reshape(M + 2, 5).to(torch.int32)
    kc, vc = make_cache((M + 2) * 5, nkv, page, hd, dtype)
    # reference: float64 product, rounded to bfloat16 once (as the fused kernel rounds once)
    qkv_ref = R.linear(x, w, torch.float64)
    kr, vr = kc.clone().double(), vc.clone().double()
    R.rope_store(qkv_ref, table, hd, 0, pos, slot, None, kr, vr, pt, page, 0, nh, nkv, hd)
    w_dev = _decode_copy(w.to(DEV), "qkv", nh=nh, nkv=nkv, hd=hd) if copy else w.to(DEV)
    got = ops().qkv_rope_store(x_dev, w_dev, table.to(DEV), pos.to(DEV), slot.to(DEV), kc_g := kc.to(DEV),
                               vc_g := vc.to(DEV), pt.to(DEV), page, 0, nh, nkv, hd).cpu()
    sc = math.sqrt(K) * 0.1
    close(got[:, :nh * hd], qkv_ref[:, :nh * hd], dtype, scale=sc)
    for gotc, wantc in ((kc_g.cpu(), kr), (vc_g.cpu(), vr)):
        assert torch.equal(torch.isnan(gotc), torch.isnan(wantc))        # the same rows, nothing else
        close(torch.nan_to_num(gotc), torch.nan_to_num(wantc), dtype, scale=sc)


# ---------------------------------------------------------------- products of 9 to 128 rows
# (tiles a block, parts of K)
_ROWS_SHAPES = [(None, None), (2, 1), (2, 4), (3, 2), (3, 4), (4, 1), (4, 2), (5, 2), (6, 1), (7, 1), (8, 2)]


@pytest.fixture
def rows_shape():
    """Forces the block shape of the rows kernels and gives the library's own choice back after."""
    lib = ops()._lib()
    yield lambda tb, kp: lib.illm_set_rows_shape(tb or 0, kp or 0)
    lib.illm_set_rows_shape(0, 0)


@pytest.mark.parametrize("tb,kp", _ROWS_SHAPES)
@pytest.mark.parametrize("M,N,K", [(17, 40, 128), (33, 100, 192), (64, 12288, 4096), (9, 320, 64), (1, 64, 64),
                                   (65, 411, 320), (128, 1000, 1088), (48, 32000, 256), (100, 8, 4096)])
def test_linear_rows(M, N, K, tb, kp, rows_shape):
    """The product with X shared through LDS and K cut inside the block, in every block shape,
    float32 and bfloat16 results; row counts around the tile and launch edges (16, 64)."""
    o = ops()
    rows_shape(tb, kp)
    x, w = rnd(M, K, dtype=torch.bfloat16, seed=1), rnd(N, K, dtype=torch.bfloat16, seed=2, std=0.2)
    wc = _decode_copy(w.to(DEV))
    want = R.linear(x, w, torch.float64)
    for ydt in DTYPES:
        got = o.linear_rows(x.to(DEV), wc, ydt)
        assert got.dtype == ydt
        close(got, want, ydt, scale=0.2 * math.sqrt(K))
    # a row's result does not depend on the other rows of the step: the same bits (beyond 64 rows
    # a block has half as many parts of K at most, so a forced number of parts may hold for the
    # row alone and not for the step: another order of summation)
    if not (M > 64 and kp is not None and kp > (1 if tb >= 4 else 2)):
        alone = o.linear_rows(x[M - 1:].to(DEV), wc, torch.float32)
        among = o.linear_rows(x.to(DEV), wc, torch.float32)[M - 1]
        assert torch.equal(alone[0], among)


def test_linear_rows_takes_the_norm_and_refuses_what_it_does_not_take(rows_shape):
    o = ops()
    M, N, K = 12, 200, 4096
    x_dev, x = _prepared_rows(M, K, torch.bfloat16, 1e-5)
    w = rnd(N, K, dtype=torch.bfloat16, seed=2, std=0.2)
    wc = _decode_copy(w.to(DEV))
    for tb, kp, ps in ((None, None, None), (2, 4, 2), (4, 1, 4)):
        rows_shape(tb, kp)
        close(o.linear_rows(x_dev, wc, torch.float32), R.linear(x, w, torch.float64), torch.bfloat16,
              scale=0.2 * math.sqrt(K))
    assert not o.rows_fits(rnd(129, K, dtype=torch.bfloat16).to(DEV), wc, "plain")
    assert not o.rows_fits(rnd(20, K, dtype=torch.bfloat16).to(DEV), wc, "gate_up")     # another kernel's tiles
    assert not o.rows_fits(rnd(20, K, dtype=torch.bfloat16).to(DEV), w.to(DEV), "plain")  # no copy
    assert not o.rows_fits(rnd(20, K).to(DEV), wc, "plain")                             # float32 rows
    w96 = _decode_copy(rnd(N, 96, dtype=torch.bfloat16, seed=3).to(DEV))
    assert not o.rows_fits(rnd(20, 96, dtype=torch.bfloat16).to(DEV), w96, "plain")     # K must be a multiple of 64
    with pytest.raises(o.KernelError):
        o.linear_rows(rnd(20, K).to(DEV), wc, torch.float32)


@pytest.mark.parametrize("tb,kp", _ROWS_SHAPES)
@pytest.mark.parametrize("M,F,K", [(17, 172, 64), (64, 11008, 4096), (40, 50, 192), (64, 203, 320), (33, 8, 1024),
                                   (65, 50, 192), (100, 172, 128), (128, 2056, 512), (113, 203, 320)])
def test_gate_up_silu_of_many_rows(M, F, K, tb, kp, rows_shape):
    """17 to 128 rows: the product and the SiLU-multiply in one kernel, from the gate|up tiles."""
    o = ops()
    rows_shape(tb, kp)
    x = rnd(M, K, dtype=torch.bfloat16, seed=1)
    w = rnd(2 * F, K, dtype=torch.bfloat16, seed=2, std=0.2)
    got = o.gate_up_silu(x.to(DEV), _decode_copy(w.to(DEV), "gate_up"))
    g, u = R.linear(x, w[:F], torch.float64), R.linear(x, w[F:], torch.float64)
    want = g / (1 + torch.exp(-g)) * u
    top = max(1.0, float(want.abs().max()))
    close(got, want, torch.bfloat16, scale=top)
    swapped = u / (1 + torch.exp(-u)) * g
    assert not torch.allclose(got.double().cpu(), swapped, atol=0.1 * top)
    # the product alone keeps float32 sums where the unfused path rounds gate and up to bfloat16
    # first: the fused result is the closer one
    loose = o.gate_up_silu(x.to(DEV), w.to(DEV))            # no copy: vendor GEMM, then SiLU-multiply
    close(loose, want, torch.bfloat16, scale=top)
    assert float((got.double().cpu() - want).abs().mean()) <= float((loose.double().cpu() - want).abs().mean()) * 1.05


@pytest.mark.parametrize("tb,kp", _ROWS_SHAPES)
@pytest.mark.parametrize("M,nh,nkv,hd,K", [(17, 4, 2, 32, 64), (64, 32, 32, 128, 4096), (40, 6, 3, 64, 256),
                                           (64, 8, 1, 96, 128), (33, 3, 3, 48, 192), (50, 2, 1, 16, 1024),
                                           (65, 4, 2, 32, 64), (96, 6, 3, 64, 256), (128, 48, 8, 128, 256),
                                           (113, 40, 40, 128, 128)])
def test_qkv_rope_store_of_many_rows(M, nh, nkv, hd, K, tb, kp, rows_shape):
    """17 to 128 sequences decoding together (96 for matrices of fewer than 8192 rows): the q|k|v
    product, the rotation and the cache store in one kernel against the three steps."""
    from inferllm_amd.parts.position import rotary_table
    o = ops()
    rows_shape(tb, kp)
    dtype, page = torch.bfloat16, 64
    table = rotary_table(777.0, hd, 300, "cpu")
    x = rnd(M, K, dtype=dtype, seed=1)
    w = rnd((nh + 2 * nkv) * hd, K, dtype=dtype, seed=2, std=0.1)
    pos = torch.tensor([(37 * i + 5) % 290 for i in range(M)], dtype=torch.int32)
    slot = torch.randperm(M + 2, generator=torch.Generator().manual_seed(9))[:M].to(torch.int32)
    g = torch.Generator().manual_seed(4)
    pt = torch.randperm((M + 2) * 5, generator=g).reshape(M + 2, 5).to(torch.int32)
    kc, vc = make_cache((M + 2) * 5, nkv, page, hd, dtype)
    qkv_ref = R.linear(x, w, torch.float64)
    kr, vr = kc.clone().double(), vc.clone().double()
    R.rope_store(qkv_ref, table, hd, 0, pos, slot, None, kr, vr, pt, page, 0, nh, nkv, hd)
    w_dev = _decode_copy(w.to(DEV), "qkv", nh=nh, nkv=nkv, hd=hd)
    assert o.qkv_rope_store_fits(x.to(DEV), w_dev, hd) and not o.qkv_rope_store_fits(x.to(DEV), w.to(DEV), hd)
    got = o.qkv_rope_store(x.to(DEV), w_dev, table.to(DEV), pos.to(DEV), slot.to(DEV), kc_g := kc.to(DEV),
                           vc_g := vc.to(DEV), pt.to(DEV), page, 0, nh, nkv, hd).cpu()
    sc = math.sqrt(K) * 0.1
    close(got[:, :nh * hd], qkv_ref[:, :nh * hd], dtype, scale=sc)
    for gotc, wantc in ((kc_g.cpu(), kr), (vc_g.cpu(), vr)):
        assert torch.equal(torch.isnan(gotc), torch.isnan(wantc))        # the same rows, nothing else
        close(torch.nan_to_num(gotc), torch.nan_to_num(wantc), dtype, scale=sc)
