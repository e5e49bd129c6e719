"""The yardsticks of the benchmark library move the bytes they claim to: a roof measured with a kernel that
skips or repeats tiles would be no roof.  Every shape of the pipelined persistent probe, at sizes that leave a
ragged last round, against the XOR of its inputs; the one-shot / persistent probe against a plain copy."""
import pytest

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("threads", [256, 512, 1024])
@pytest.mark.parametrize("barrier", [False, True])
def test_ring_probe_writes_every_tile_once(hk, cuda, threads, barrier):
    import torch
    tile = threads * 16
    for tiles in (1, 2, 255, 256, 257, 1000, 1537):
        n = tiles * tile
        a = torch.randint(0, 256, (n,), dtype=torch.uint8, device=cuda)
        b = torch.randint(0, 256, (n,), dtype=torch.uint8, device=cuda)
        want = a.view(torch.int32) ^ b.view(torch.int32)
        for depth in (1, 2, 3, 4):
            for per_cu in (1, 2):
                d = torch.zeros(n + tile, dtype=torch.uint8, device=cuda)
                hk.ring_probe(d[:n], a, b, threads, depth, barrier, per_cu)
                torch.cuda.synchronize()
                got = d[:n].view(torch.int32).clone()
                if barrier:
                    # the barrier variant folds a per-tile checksum into the last word of every vector, as a row
                    # kernel would use its reduction: the other three words are the plain XOR
                    got4, want4 = got.view(-1, 4), want.view(-1, 4)
                    assert torch.equal(got4[:, :3], want4[:, :3]), (tiles, depth, per_cu)
                else:
                    assert torch.equal(got, want), (tiles, depth, per_cu)
                assert int(d[n:].max()) == 0, "wrote past the last tile"
    with pytest.raises(hk.HkError):
        hk.ring_probe(torch.zeros(100, dtype=torch.uint8, device=cuda), a, b, threads, 2, barrier, 1)   # not whole tiles
    with pytest.raises(hk.HkError):
        hk.ring_probe(d[:n], a, b, threads, 5, barrier, 1)


def test_stream_probe_copies(hk, cuda):
    import torch
    n = (1 << 20) + 4096 + 16
    src = torch.randint(0, 256, (n,), dtype=torch.uint8, device=cuda)
    for threads in (64, 256, 1024):
        for vectors in (1, 2, 4):
            for per_cu in (0, 1, 4):
                dst = torch.zeros(n + 64, dtype=torch.uint8, device=cuda)
                hk.stream_probe([dst[:n]], [src], threads, vectors, True, True, per_cu)
                torch.cuda.synchronize()
                assert torch.equal(dst[:n], src), (threads, vectors, per_cu)
                assert int(dst[n:].max()) == 0
