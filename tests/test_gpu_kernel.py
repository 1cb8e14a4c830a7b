"""GPU parity of the reduction kernel (stands for _reduce_inplace_cuda, allreduce_cuda_impl.h:26-33)
through the C ABI, bit-exact against the oracle's scalar loop."""
import ctypes as C

import numpy as np
import pytest

import hip_lib as H
import oracle_lib as O

pytestmark = pytest.mark.gpu
torch = pytest.importorskip("torch")


def oracle_add(a, b):
    r = a.copy()
    O.lib().orc_reduce_inplace(O.DTYPE_OF[a.dtype], r.ctypes.data, b.ctypes.data, r.size)
    return r


def gpu_add(a, b, off_a=0, off_b=0, off_d=0, inplace=False):
    """a, b: host arrays; operands are placed off_* elements into 256-byte aligned device buffers."""
    dt = O.DTYPE_OF[a.dtype]
    n = a.size
    ta = torch.zeros(n + 64, dtype=torch.from_numpy(a[:0]).dtype, device="cuda")
    tb = torch.zeros_like(ta)
    td = torch.zeros_like(ta)
    td.view(torch.uint8).fill_(0xAB)
    ta[off_a:off_a + n] = torch.from_numpy(a).cuda()
    tb[off_b:off_b + n] = torch.from_numpy(b).cuda()
    es = a.itemsize
    dst = ta.data_ptr() + off_a * es if inplace else td.data_ptr() + off_d * es
    torch.cuda.synchronize()
    rc = H.lib().ibcomm_hip_reduce(dt, dst, ta.data_ptr() + off_a * es, tb.data_ptr() + off_b * es, n, None)
    assert rc == 0, H.last_error()
    torch.cuda.synchronize()
    if inplace:
        return ta[off_a:off_a + n].cpu().numpy(), None
    full = td.cpu().numpy()
    return full[off_d:off_d + n], full


@pytest.mark.parametrize("n", [0, 1, 2, 3, 4, 5, 63, 64, 65, 255, 256, 257, 1023, 1025, 4099, 16384, 262144 + 3, 2097152])
def test_f32_sizes(n):
    rng = np.random.default_rng(n)
    a = rng.standard_normal(n).astype(np.float32)
    b = (rng.standard_normal(n) * 1e-3).astype(np.float32)
    got, full = gpu_add(a, b)
    assert np.array_equal(O.bits(got), O.bits(oracle_add(a, b)))
    assert (full.view(np.uint32)[n:] == 0xABABABAB).all(), "wrote past the end"


@pytest.mark.parametrize("off_a,off_b,off_d", [(0, 0, 0), (1, 1, 1), (2, 2, 2), (3, 3, 3), (1, 0, 0), (0, 3, 0), (0, 0, 2), (1, 2, 3)])
def test_f32_every_alignment_phase(off_a, off_b, off_d):
    # chunk offsets are arbitrary element multiples, so operands can sit at any 4-byte phase
    for n in (1, 2, 3, 4, 5, 7, 8, 9, 4097, 100003):
        rng = np.random.default_rng(n + off_a)
        a = rng.standard_normal(n).astype(np.float32)
        b = rng.standard_normal(n).astype(np.float32)
        got, full = gpu_add(a, b, off_a, off_b, off_d)
        assert np.array_equal(O.bits(got), O.bits(oracle_add(a, b)))
        u = full.view(np.uint32)
        assert (u[:off_d] == 0xABABABAB).all() and (u[off_d + n:] == 0xABABABAB).all()


def test_f32_special_values_denormals_kept():
    tiny, dn, mx = np.float32(1e-45), np.float32(5.9e-39), np.finfo(np.float32).max
    a = np.array([0.0, -0.0, -0.0, tiny, dn, mx, -mx, np.inf, 1.0, 16777216.0, 1e-38, 3e-39] * 50, dtype=np.float32)
    b = np.array([-0.0, -0.0, 0.0, tiny, dn, mx, -mx, 1.0, -1.0, 1.0, -1.1e-38, 4e-39] * 50, dtype=np.float32)
    got, _ = gpu_add(a, b)
    want = oracle_add(a, b)
    assert np.array_equal(O.bits(got), O.bits(want))
    assert got[3] != 0 and got[4] != 0 and got[11] != 0  # denormal results are not flushed to zero


def test_f32_nan_and_inf_propagate():
    a = np.array([np.nan, 1.0, np.inf, -np.inf] * 8, dtype=np.float32)
    b = np.array([1.0, np.nan, -np.inf, -np.inf] * 8, dtype=np.float32)
    got, _ = gpu_add(a, b)
    assert np.isnan(got[0::4]).all() and np.isnan(got[1::4]).all() and np.isnan(got[2::4]).all()
    assert np.isneginf(got[3::4]).all()


def test_in_place_is_the_reference_form():
    # result[i] += value[i]: dst aliases the first operand
    rng = np.random.default_rng(7)
    a = rng.standard_normal(70001).astype(np.float32)
    b = rng.standard_normal(70001).astype(np.float32)
    got, _ = gpu_add(a, b, 1, 1, 0, inplace=True)
    assert np.array_equal(O.bits(got), O.bits(oracle_add(a, b)))


@pytest.mark.parametrize("dtype", [np.int32, np.float64, np.int64])
def test_other_element_types(dtype):
    rng = np.random.default_rng(3)
    for n in (1, 2, 3, 1000, 65537):
        if np.issubdtype(dtype, np.integer):
            info = np.iinfo(dtype)
            a = rng.integers(info.min, info.max, n, dtype=dtype)  # wraps on overflow like the reference's int +=
            b = rng.integers(info.min, info.max, n, dtype=dtype)
        else:
            a = rng.standard_normal(n).astype(dtype)
            b = rng.standard_normal(n).astype(dtype) * 1e-9
        for off in (0, 1):
            got, _ = gpu_add(a, b, off, off, off)
            assert np.array_equal(O.bits(got), O.bits(oracle_add(a, b)))


def test_segment_launch_matches_per_segment_results():
    rng = np.random.default_rng(11)
    k = H.lib().ibcomm_hip_max_segments()
    assert k >= 32
    sizes = [int(s) for s in rng.integers(0, 5000, k)]
    a = [rng.standard_normal(s).astype(np.float32) for s in sizes]
    b = [rng.standard_normal(s).astype(np.float32) for s in sizes]
    ta = [torch.from_numpy(x).cuda() for x in a]
    tb = [torch.from_numpy(x).cuda() for x in b]
    td = [torch.zeros(s, dtype=torch.float32, device="cuda") for s in sizes]
    vp = C.c_void_p
    torch.cuda.synchronize()
    rc = H.lib().ibcomm_hip_reduce_segments(H.F32, k, (vp * k)(*[t.data_ptr() for t in td]),
                                            (vp * k)(*[t.data_ptr() for t in ta]), (vp * k)(*[t.data_ptr() for t in tb]),
                                            (C.c_size_t * k)(*sizes), None)
    assert rc == 0, H.last_error()
    torch.cuda.synchronize()
    for i in range(k):
        assert np.array_equal(O.bits(td[i].cpu().numpy()), O.bits(oracle_add(a[i], b[i])))
    assert H.lib().ibcomm_hip_reduce_segments(H.F32, k + 1, None, None, None, None, None) == H.INVALID_ARGUMENT


@pytest.mark.parametrize("n", [1024 * 63 + 4, 1024 * 64, 1024 * 100 + 12, 1024 * 2048, 1024 * 2049 + 8, 1024 * 5000 + 4,
                               1024 * 8192 + 512, 1024 * 32768, 1024 * 32769 + 16])
def test_aligned_kernel_geometries(n):
    # Vector-aligned launches pick their workgroup size and tile order by segment size (256 threads up to
    # 2048 tiles of 1 Ki fp32, 128 beyond; permuted tile order from 64 up to 32768 tiles).  Every tile must
    # still be computed exactly once, including those beyond the last whole group of 64 workgroups.
    g = torch.Generator(device="cuda").manual_seed(n)
    a = torch.randn(n, device="cuda", generator=g)
    b = torch.randn(n, device="cuda", generator=g)
    d = torch.full((n + 256,), float("nan"), device="cuda")
    torch.cuda.synchronize()
    assert H.lib().ibcomm_hip_reduce(H.F32, d.data_ptr(), a.data_ptr(), b.data_ptr(), n, None) == 0, H.last_error()
    torch.cuda.synchronize()
    assert torch.equal(d[:n].view(torch.int32), (a + b).view(torch.int32))
    assert torch.isnan(d[n:]).all(), "wrote past the end"


@pytest.mark.parametrize("dtype", [torch.int32, torch.float64, torch.int64])
def test_aligned_kernel_geometries_other_types(dtype):
    code = {torch.int32: H.I32, torch.float64: H.F64, torch.int64: H.I64}[dtype]
    for n in (512 * 100 + 8, 1024 * 3000 + 4):
        g = torch.Generator(device="cuda").manual_seed(n)
        a = torch.randint(-2**31, 2**31 - 1, (n,), device="cuda", generator=g).to(dtype) if dtype != torch.float64 \
            else torch.randn(n, device="cuda", generator=g, dtype=dtype)
        b = a.flip(0).clone()
        d = torch.zeros_like(a)
        torch.cuda.synchronize()
        assert H.lib().ibcomm_hip_reduce(code, d.data_ptr(), a.data_ptr(), b.data_ptr(), n, None) == 0, H.last_error()
        torch.cuda.synchronize()
        assert torch.equal(d, a + b)


def test_aligned_segments_of_different_sizes_share_a_launch():
    # the grid is sized for the largest segment and the tile order is permuted per group of 64 workgroups:
    # the smaller segments must come out complete, and nothing may be written beyond any of them
    sizes = [1024 * 3, 1024 * 200 + 4, 1024 * 70, 0, 1024 * 2100 + 8, 4]
    k = len(sizes)
    g = torch.Generator(device="cuda").manual_seed(3)
    ta = [torch.randn(s, device="cuda", generator=g) for s in sizes]
    tb = [torch.randn(s, device="cuda", generator=g) for s in sizes]
    td = [torch.full((s + 64,), float("nan"), device="cuda") for s in sizes]
    vp = C.c_void_p
    torch.cuda.synchronize()
    rc = H.lib().ibcomm_hip_reduce_segments(H.F32, k, (vp * k)(*[t.data_ptr() for t in td]),
                                            (vp * k)(*[t.data_ptr() for t in ta]), (vp * k)(*[t.data_ptr() for t in tb]),
                                            (C.c_size_t * k)(*sizes), None)
    assert rc == 0, H.last_error()
    torch.cuda.synchronize()
    for i, s in enumerate(sizes):
        assert torch.equal(td[i][:s].view(torch.int32), (ta[i] + tb[i]).view(torch.int32)), "segment %d" % i
        assert torch.isnan(td[i][s:]).all(), "segment %d wrote past its end" % i


@pytest.mark.parametrize("n", [1024 * 64 + 1, 1024 * 100 + 3, 1024 * 2048 - 1, 1024 * 2049 + 2, 1024 * 8192 - 1, 4194304 * 3 + 4194303,
                               1024 * 32768 + 1, 1024 * 32769 + 3])
@pytest.mark.parametrize("phase", [0, 1, 3])
def test_peeled_kernel_geometries(n, phase):
    # Off the 16-byte grid (operands `phase` elements into their buffers, lengths that are no whole number of
    # vectors: config 5's ragged last ring step is 16,777,215 elements) the general kernel peels both ends and runs
    # the aligned kernel's geometry in between: 128/256 threads, permuted tile order, either store policy.  Every
    # element once, nothing outside, and the bits of the oracle's loop on a sampled stripe at each end.
    g = torch.Generator(device="cuda").manual_seed(n + phase)
    a = torch.randn(n + 8, device="cuda", generator=g)
    b = torch.randn(n + 8, device="cuda", generator=g)
    d = torch.full((n + 264,), float("nan"), device="cuda")
    es = 4
    torch.cuda.synchronize()
    assert H.lib().ibcomm_hip_reduce(H.F32, d.data_ptr() + phase * es, a.data_ptr() + phase * es, b.data_ptr() + phase * es, n, None) == 0, H.last_error()
    torch.cuda.synchronize()
    want = a[phase:phase + n] + b[phase:phase + n]
    assert torch.equal(d[phase:phase + n].view(torch.int32), want.view(torch.int32))
    assert torch.isnan(d[:phase]).all() and torch.isnan(d[phase + n:]).all(), "wrote outside the segment"
    for s in (slice(0, 4099), slice(n - 4099, n)):
        ha, hb = a[phase:phase + n][s].cpu().numpy(), b[phase:phase + n][s].cpu().numpy()
        assert np.array_equal(O.bits(d[phase:phase + n][s].cpu().numpy()), O.bits(oracle_add(ha, hb)))


@pytest.mark.parametrize("dtype", [torch.int32, torch.float64, torch.int64])
def test_peeled_kernel_other_types_adds_and_copies(dtype):
    code = {torch.int32: H.I32, torch.float64: H.F64, torch.int64: H.I64}[dtype]
    es = torch.empty(0, dtype=dtype).element_size()
    for n in (1024 * 300 + 1, 1024 * 3000 + 1):
        for phase in ((0, 1) if es == 8 else (0, 1, 2, 3)):
            g = torch.Generator(device="cuda").manual_seed(n + phase)
            a = torch.randint(-2**31, 2**31 - 1, (n + 4,), device="cuda", generator=g).to(dtype) if dtype != torch.float64 \
                else torch.randn(n + 4, device="cuda", generator=g, dtype=dtype)
            b = a.flip(0).clone()
            d = torch.zeros(n + 8, dtype=dtype, device="cuda")
            c = torch.zeros(n + 8, dtype=dtype, device="cuda")
            o = phase * es
            vp = C.c_void_p
            torch.cuda.synchronize()
            assert H.lib().ibcomm_hip_reduce(code, d.data_ptr() + o, a.data_ptr() + o, b.data_ptr() + o, n, None) == 0, H.last_error()
            assert H.lib().ibcomm_hip_copy_segments(code, 1, (vp * 1)(c.data_ptr() + o), (vp * 1)(a.data_ptr() + o), (C.c_size_t * 1)(n), None) == 0, H.last_error()
            torch.cuda.synchronize()
            assert torch.equal(d[phase:phase + n], a[phase:phase + n] + b[phase:phase + n])
            assert torch.equal(c[phase:phase + n], a[phase:phase + n])
            for t in (d, c):
                assert (t[:phase] == 0).all() and (t[phase + n:] == 0).all(), "wrote outside the segment"


def test_peeled_segments_of_different_sizes_and_phases_share_a_launch():
    # segments of one launch may each sit at their own 16-byte phase; those whose three operands do not share
    # one go element by element in the same launch
    sizes = [1024 * 3 + 1, 1024 * 2100 + 3, 1024 * 70, 0, 5, 1024 * 700 + 2, 1024 * 64 + 1]
    phases = [(1, 1, 1), (2, 2, 2), (0, 0, 0), (0, 0, 0), (3, 3, 3), (1, 2, 3), (0, 3, 0)]
    k = len(sizes)
    g = torch.Generator(device="cuda").manual_seed(13)
    ta = [torch.randn(s + 8, device="cuda", generator=g) for s in sizes]
    tb = [torch.randn(s + 8, device="cuda", generator=g) for s in sizes]
    td = [torch.full((s + 72,), float("nan"), device="cuda") for s in sizes]
    vp = C.c_void_p
    torch.cuda.synchronize()
    rc = H.lib().ibcomm_hip_reduce_segments(H.F32, k, (vp * k)(*[t.data_ptr() + 4 * p[0] for t, p in zip(td, phases)]),
                                            (vp * k)(*[t.data_ptr() + 4 * p[1] for t, p in zip(ta, phases)]),
                                            (vp * k)(*[t.data_ptr() + 4 * p[2] for t, p in zip(tb, phases)]), (C.c_size_t * k)(*sizes), None)
    assert rc == 0, H.last_error()
    torch.cuda.synchronize()
    for i, (s, p) in enumerate(zip(sizes, phases)):
        want = ta[i][p[1]:p[1] + s] + tb[i][p[2]:p[2] + s]
        assert torch.equal(td[i][p[0]:p[0] + s].view(torch.int32), want.view(torch.int32)), "segment %d" % i
        assert torch.isnan(td[i][:p[0]]).all() and torch.isnan(td[i][p[0] + s:]).all(), "segment %d wrote outside" % i


@pytest.mark.parametrize("n", [1024 * 100 + 3, 1024 * 2049 + 2, 1024 * 8192 - 1])
@pytest.mark.parametrize("phases", [(1, 2, 3), (0, 3, 0), (2, 0, 1), (0, 0, 1)])
def test_operands_at_different_phases_at_every_geometry(n, phases):
    # dst, a and b each at their own 4-byte phase: the vector body follows dst's 16-byte grid and the
    # operands are loaded as 16-byte vectors from element-aligned addresses
    pd, pa, pb = phases
    g = torch.Generator(device="cuda").manual_seed(n + pd * 16 + pa * 4 + pb)
    a = torch.randn(n + 8, device="cuda", generator=g)
    b = torch.randn(n + 8, device="cuda", generator=g)
    d = torch.full((n + 264,), float("nan"), device="cuda")
    torch.cuda.synchronize()
    assert H.lib().ibcomm_hip_reduce(H.F32, d.data_ptr() + 4 * pd, a.data_ptr() + 4 * pa, b.data_ptr() + 4 * pb, n, None) == 0, H.last_error()
    torch.cuda.synchronize()
    want = a[pa:pa + n] + b[pb:pb + n]
    assert torch.equal(d[pd:pd + n].view(torch.int32), want.view(torch.int32))
    assert torch.isnan(d[:pd]).all() and torch.isnan(d[pd + n:]).all(), "wrote outside the segment"
    # the copy of the same shape
    c = torch.full((n + 264,), float("nan"), device="cuda")
    vp = C.c_void_p
    assert H.lib().ibcomm_hip_copy_segments(H.F32, 1, (vp * 1)(c.data_ptr() + 4 * pd), (vp * 1)(a.data_ptr() + 4 * pa), (C.c_size_t * 1)(n), None) == 0
    torch.cuda.synchronize()
    assert torch.equal(c[pd:pd + n].view(torch.int32), a[pa:pa + n].view(torch.int32))
    assert torch.isnan(c[:pd]).all() and torch.isnan(c[pd + n:]).all(), "the copy wrote outside the segment"


def test_eight_byte_operands_at_different_phases():
    for dtype, code in ((torch.float64, H.F64), (torch.int64, H.I64)):
        for n in (1024 * 50 + 1, 1024 * 3000 + 1):
            for pd, pa, pb in ((0, 1, 0), (1, 0, 1), (1, 0, 0)):
                g = torch.Generator(device="cuda").manual_seed(n + pd + 2 * pa + 4 * pb)
                a = torch.randn(n + 4, device="cuda", generator=g, dtype=torch.float64)
                a = a if dtype == torch.float64 else (a * 1e15).to(torch.int64)
                b = a.flip(0).clone()
                d = torch.zeros(n + 8, dtype=dtype, device="cuda")
                torch.cuda.synchronize()
                assert H.lib().ibcomm_hip_reduce(code, d.data_ptr() + 8 * pd, a.data_ptr() + 8 * pa, b.data_ptr() + 8 * pb, n, None) == 0, H.last_error()
                torch.cuda.synchronize()
                assert torch.equal(d[pd:pd + n], a[pa:pa + n] + b[pb:pb + n])
                assert (d[:pd] == 0).all() and (d[pd + n:] == 0).all(), "wrote outside the segment"


def test_large_linear_property():
    # 256 MiB operands: compare with torch's own fp32 add on the device (IEEE add, same rounding)
    n = 67108864
    g = torch.Generator(device="cuda").manual_seed(5)
    a = torch.randn(n, device="cuda", generator=g)
    b = torch.randn(n, device="cuda", generator=g)
    d = torch.empty_like(a)
    torch.cuda.synchronize()
    assert H.lib().ibcomm_hip_reduce(H.F32, d.data_ptr(), a.data_ptr(), b.data_ptr(), n, None) == 0
    torch.cuda.synchronize()
    assert torch.equal(d.view(torch.int32), (a + b).view(torch.int32))
    # and a sampled stripe against the oracle on the host
    s = slice(n - 100003, n)
    assert np.array_equal(O.bits(d[s].cpu().numpy()), O.bits(oracle_add(a[s].cpu().numpy(), b[s].cpu().numpy())))


@pytest.mark.parametrize("dtype", [np.float32, np.int32, np.float64, np.int64])
def test_copy_segments_all_widths_and_phases(dtype):
    # the engine's copy launch on its own (ibcomm_hip_copy_segments): aligned one-segment kernel, aligned
    # table kernel (several segments) and the general kernel (odd offsets, ragged lengths), for 4- and 8-byte elements
    rng = np.random.default_rng(3)
    es = np.dtype(dtype).itemsize
    dt = O.DTYPE_OF[np.dtype(dtype)]
    for lens, offs in [([262144], [0]), ([4096, 65536, 16], [0, 0, 0]), ([1000, 3, 70001], [1, 0, 3]), ([0, 5, 0], [0, 1, 0])]:
        k = len(lens)
        src = [torch.from_numpy((rng.standard_normal(n + 8) * 100).astype(dtype)).cuda() for n in lens]
        dst = [torch.zeros(n + 8, dtype=src[0].dtype, device="cuda") for n in lens]
        for t in dst:
            t.view(torch.uint8).fill_(0xAB)
        vp = C.c_void_p
        d = (vp * k)(*[t.data_ptr() + o * es for t, o in zip(dst, offs)])
        a = (vp * k)(*[t.data_ptr() + o * es for t, o in zip(src, offs)])
        ln = (C.c_size_t * k)(*lens)
        torch.cuda.synchronize()
        assert H.lib().ibcomm_hip_copy_segments(dt, k, d, a, ln, None) == 0, H.last_error()
        torch.cuda.synchronize()
        for t_src, t_dst, n, o in zip(src, dst, lens, offs):
            got, want = t_dst.cpu().numpy(), t_src.cpu().numpy()
            assert np.array_equal(O.bits(got[o:o + n]), O.bits(want[o:o + n]))
            raw = got.view(np.uint8)
            assert (raw[:o * es] == 0xAB).all() and (raw[(o + n) * es:] == 0xAB).all(), "wrote outside the segment"


def test_one_segment_launch_and_table_launch_give_the_same_bits():
    # a launch of one segment takes its operands as plain kernel arguments, several segments go through the
    # table: the same data through both, and through the reference's association (one add per element)
    n = 1 << 20
    rng = np.random.default_rng(8)
    a = rng.standard_normal(n).astype(np.float32)
    b = (rng.standard_normal(n) * 1e-4).astype(np.float32)
    want = oracle_add(a, b)
    ta, tb = torch.from_numpy(a).cuda(), torch.from_numpy(b).cuda()
    one = torch.zeros(n, device="cuda")
    two = torch.zeros(n, device="cuda")
    vp = C.c_void_p
    L = H.lib()
    assert L.ibcomm_hip_reduce_segments(H.F32, 1, (vp * 1)(one.data_ptr()), (vp * 1)(ta.data_ptr()), (vp * 1)(tb.data_ptr()),
                                        (C.c_size_t * 1)(n), None) == 0
    h = n // 2
    assert L.ibcomm_hip_reduce_segments(H.F32, 2, (vp * 2)(two.data_ptr(), two.data_ptr() + 4 * h), (vp * 2)(ta.data_ptr(), ta.data_ptr() + 4 * h),
                                        (vp * 2)(tb.data_ptr(), tb.data_ptr() + 4 * h), (C.c_size_t * 2)(h, h), None) == 0
    torch.cuda.synchronize()
    assert np.array_equal(O.bits(one.cpu().numpy()), O.bits(want)) and np.array_equal(O.bits(two.cpu().numpy()), O.bits(want))
