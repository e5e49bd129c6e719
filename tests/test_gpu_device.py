"""GPU checks of the device layer of the C-ABI: fill, copies, streams and events."""
import ctypes

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def test_memset_any_alignment_and_size(hk, cuda):
    import torch
    lib = hk.lib()
    buf = torch.zeros(1 << 16, dtype=torch.uint8, device=cuda)
    for off, n in [(0, 0), (0, 1), (1, 1), (3, 13), (5, 16), (15, 17), (16, 4096), (7, 4099), (1, 40000), (9, 1 << 15)]:
        buf.fill_(0x11)
        torch.cuda.synchronize()
        hk.check(lib.hk_memset(ctypes.c_void_p(buf.data_ptr() + off), ctypes.c_int(0xAB), ctypes.c_size_t(n),
                               hk.current_stream()))
        torch.cuda.synchronize()
        got = buf.cpu().numpy()
        want = np.full(1 << 16, 0x11, dtype=np.uint8)
        want[off:off + n] = 0xAB
        assert np.array_equal(got, want), (off, n)
    big = torch.empty((1 << 26) + 3, dtype=torch.uint8, device=cuda)
    hk.check(lib.hk_memset(ctypes.c_void_p(big.data_ptr()), ctypes.c_int(0x5A), ctypes.c_size_t(big.numel()),
                           hk.current_stream()))
    torch.cuda.synchronize()
    assert int(big.min()) == 0x5A and int(big.max()) == 0x5A
    assert lib.hk_memset(None, 0, ctypes.c_size_t(8), hk.current_stream()) == -1


def test_copy_and_strided_copy(hk, cuda):
    import torch
    src = torch.arange(1 << 20, dtype=torch.int32, device=cuda)
    dst = torch.zeros_like(src)
    hk.copy_kernel(dst.view(torch.uint8), src.view(torch.uint8))
    torch.cuda.synchronize()
    assert torch.equal(dst, src)
    for dt in (torch.float32, torch.bfloat16, torch.int64, torch.uint8, torch.float64):
        x = (torch.arange(7 * 12 * 5, device=cuda) % 120).to(dt).reshape(7, 12, 5)
        view = x.permute(2, 0, 1)[:, ::2, 1:]
        out = torch.empty(view.shape, dtype=dt, device=cuda)
        hk.strided_copy(view, out)
        torch.cuda.synchronize()
        assert torch.equal(out, view.contiguous()), dt


def test_strided_scatter_is_the_inverse_of_the_gather(hk, cuda):
    """hk_strided_scatter lays a dense array over a view of any strides: the view then reads back as the array,
    and no element outside the view changes; eight dimensions, empty views and single elements included."""
    import torch
    for dt in (torch.float32, torch.bfloat16, torch.int64, torch.uint8, torch.float64):
        backing = torch.full((7, 12, 5), 99, dtype=dt, device=cuda)
        view = backing.permute(2, 0, 1)[:, ::2, 1:]
        dense = (torch.arange(view.numel(), device=cuda) % 90).to(dt).reshape(view.shape)
        hk.strided_scatter(dense, view)
        torch.cuda.synchronize()
        assert torch.equal(view.contiguous(), dense), dt
        untouched = torch.ones_like(backing, dtype=torch.bool)
        untouched.permute(2, 0, 1)[:, ::2, 1:] = False
        assert bool((backing[untouched] == 99).all()), dt
        back = torch.empty_like(dense)
        hk.strided_copy(view, back)
        torch.cuda.synchronize()
        assert torch.equal(back, dense), dt
    # eight dimensions, every one permuted; a column slice of a wider array; a single element; nothing at all
    b8 = torch.zeros((2, 3, 2, 2, 3, 2, 2, 3), dtype=torch.float32, device=cuda)
    v8 = b8.permute(7, 6, 5, 4, 3, 2, 1, 0)
    d8 = torch.arange(v8.numel(), dtype=torch.float32, device=cuda).reshape(v8.shape)
    hk.strided_scatter(d8, v8)
    wide = torch.zeros((33, 200), dtype=torch.bfloat16, device=cuda)
    pitched = wide[:, 8:136]
    dp = torch.randn(33, 128, device=cuda).to(torch.bfloat16)
    hk.strided_scatter(dp, pitched)
    one = torch.zeros((), dtype=torch.float32, device=cuda)
    hk.strided_scatter(torch.full((), 3.0, device=cuda), one)
    hk.strided_scatter(torch.empty((0, 4), device=cuda), torch.empty((4, 0), device=cuda).t())
    torch.cuda.synchronize()
    assert torch.equal(v8.contiguous(), d8)
    assert torch.equal(pitched.contiguous(), dp) and float(wide[:, :8].abs().sum()) == 0 and float(wide[:, 136:].abs().sum()) == 0
    assert float(one) == 3.0
    lib = hk.lib()
    shape9 = (ctypes.c_int64 * 9)(*([1] * 9))
    assert lib.hk_strided_scatter(0, ctypes.c_void_p(one.data_ptr()), ctypes.c_void_p(one.data_ptr()), 9, shape9, shape9,
                                  hk.current_stream()) != 0


@pytest.mark.parametrize("dt", ["uint8", "bfloat16", "float32", "int64"])
def test_permuted_views_take_the_tiled_path(hk, cuda, dt):
    """Views whose contiguous dimension is not the last one (every permutation of three and four dimensions, extents
    around the 64-element tile, sliced and with a dimension of 1) gather into, and scatter from, a dense array
    exactly as torch's own copy does; nothing outside a scattered view changes."""
    import itertools
    import torch
    td = getattr(torch, dt)
    cases = []
    for shape in ((65, 130, 3), (3, 64, 200), (17, 1, 100, 33), (2, 70, 5, 129), (4, 130, 258)):
        for perm in itertools.permutations(range(len(shape))):
            cases.append((shape, perm))
    for shape, perm in cases:
        n = int(np.prod(shape))
        base = (torch.arange(n, device=cuda) % 251).to(td).reshape(shape)
        view = base.permute(perm)
        out = torch.empty(view.shape, dtype=td, device=cuda)
        hk.strided_copy(view, out)
        assert torch.equal(out, view.contiguous()), (shape, perm)
        backing = torch.zeros(shape, dtype=td, device=cuda)
        hk.strided_scatter(out, backing.permute(perm))
        assert torch.equal(backing, base), (shape, perm)
    # a sliced transposed view: strides that are not products of the extents, and a covered region with holes
    backing = torch.full((300, 260), 9, dtype=td, device=cuda)
    view = backing.t()[3:200:2, 10:290]          # [99, 280]: rows step 2 columns of the backing, columns are its rows
    dense = (torch.arange(view.numel(), device=cuda) % 200).to(td).reshape(view.shape)
    hk.strided_scatter(dense, view)
    assert torch.equal(view.contiguous(), dense)
    covered = torch.zeros_like(backing, dtype=torch.bool)
    covered.t()[3:200:2, 10:290] = True
    assert bool((backing[~covered] == 9).all())
    back = torch.empty_like(dense)
    hk.strided_copy(view, back)
    assert torch.equal(back, dense)
    # rows contiguous on both sides: whole 16-byte vectors when the pitch, the width and the start allow it
    # (columns 16 .. 144 of a 208-column array), element by element when they do not (columns 3 .. 131)
    for lo, hi in ((16, 144), (3, 131)):
        wide = torch.full((5, 37, 208), 9, dtype=td, device=cuda)
        view = wide.permute(1, 0, 2)[:, :, lo:hi]
        dense = (torch.arange(view.numel(), device=cuda) % 200).to(td).reshape(view.shape)
        hk.strided_scatter(dense, view)
        assert torch.equal(view.contiguous(), dense)
        assert bool((wide[:, :, :lo] == 9).all()) and bool((wide[:, :, hi:] == 9).all())
        back = torch.empty_like(dense)
        hk.strided_copy(view, back)
        assert torch.equal(back, dense)


def test_streams_events_and_ordering(hk, cuda):
    import torch
    lib = hk.lib()
    s1, s2 = ctypes.c_void_p(), ctypes.c_void_p()
    hk.check(lib.hk_stream_create(ctypes.byref(s1)))
    hk.check(lib.hk_stream_create(ctypes.byref(s2)))
    a = torch.zeros(1 << 24, dtype=torch.uint8, device=cuda)
    b = torch.zeros_like(a)
    torch.cuda.synchronize()
    e0, e1 = hk.Event(), hk.Event()
    e0.record(s1)
    hk.check(lib.hk_memset(ctypes.c_void_p(a.data_ptr()), ctypes.c_int(7), ctypes.c_size_t(a.numel()), s1))
    e1.record(s1)
    # s2 copies a -> b only after s1's fill: ordered by the event, not by the host
    hk.check(lib.hk_stream_wait_event(s2, e1.h))
    hk.check(lib.hk_copy_kernel(ctypes.c_void_p(b.data_ptr()), ctypes.c_void_p(a.data_ptr()),
                                ctypes.c_size_t(a.numel()), s2))
    hk.check(lib.hk_stream_sync(s2))
    assert int(b.min()) == 7 and int(b.max()) == 7
    e1.sync()
    done = ctypes.c_int(0)
    hk.check(lib.hk_event_query(e1.h, ctypes.byref(done)))
    assert done.value == 1
    ns = e1.elapsed_ns_since(e0)
    assert 0 < ns < 50_000_000            # a 16 MiB fill takes microseconds, not 50 ms
    hk.check(lib.hk_stream_destroy(s1))
    hk.check(lib.hk_stream_destroy(s2))


def test_device_queries(hk, cuda):
    lib = hk.lib()
    n = ctypes.c_int()
    hk.check(lib.hk_device_count(ctypes.byref(n)))
    assert n.value >= 1
    cus = ctypes.c_int()
    hk.check(lib.hk_device_cu_count(0, ctypes.byref(cus)))
    assert cus.value >= 64
    free, total = ctypes.c_size_t(), ctypes.c_size_t()
    hk.check(lib.hk_mem_get_info(ctypes.byref(free), ctypes.byref(total)))
    assert 0 < free.value <= total.value and total.value > (64 << 30)
    p = ctypes.c_void_p()
    hk.check(lib.hk_malloc(ctypes.byref(p), ctypes.c_size_t(1 << 20)))
    assert p.value and p.value % 256 == 0
    hk.check(lib.hk_free(p))
    h = ctypes.c_void_p()
    hk.check(lib.hk_host_malloc(ctypes.byref(h), ctypes.c_size_t(4096)))
    assert h.value
    hk.check(lib.hk_host_free(h))
