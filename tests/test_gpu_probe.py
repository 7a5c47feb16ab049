"""The measurement library (libteletron_probe.so) does what its header says: the copy yardstick copies,
and every built mix of the stream probe writes, to written tensor j, the dword-wise sum of the tensors
it reads plus j -- so the bandwidth figures quoted for a mix are figures for that many tensors really
read and written.  Not part of the operator path."""
import pytest
import torch

pytestmark = pytest.mark.gpu

# (reads, writes) -> accesses per lane the mix is built for
BUILT = {(1, 0): (1, 2, 6), (2, 0): (1, 2, 6), (0, 1): (1, 2, 6), (1, 1): (1, 2, 6), (2, 1): (1, 2, 6),
         (3, 1): (1, 6), (2, 2): (1, 6), (4, 2): (1, 6)}


@pytest.fixture(scope="module")
def probe(gpu_device):
    from teletron_amd import probe as p
    p.lib()
    return p


def test_stream_copy_yardstick(probe, gpu_device):
    for n in (16, 6144 * 4 * 3 + 16 * 5, 16 * 1000003):
        src = torch.randint(0, 255, (n,), dtype=torch.uint8, device=gpu_device)
        dst = torch.zeros_like(src)
        probe.stream_copy(dst, src)
        assert torch.equal(dst, src)


@pytest.mark.parametrize("reads,writes", sorted(BUILT))
def test_probe_moves_the_bytes_it_claims(probe, gpu_device, reads, writes):
    for per_lane in BUILT[(reads, writes)]:
        run = per_lane * 64 * 16                     # bytes one wavefront moves per tensor
        for runs, blocks in ((1, 0), (37, 0), (37, 3), (1030, 5)):
            nbytes = runs * run
            n32 = nbytes // 4
            gen = torch.Generator(device=gpu_device).manual_seed(reads * 100 + writes * 10 + per_lane)
            a = torch.randint(-2**31, 2**31 - 1, (2 * n32,), dtype=torch.int32, device=gpu_device, generator=gen)
            b = torch.randint(-2**31, 2**31 - 1, (2 * n32,), dtype=torch.int32, device=gpu_device, generator=gen)
            for through in ((False, True) if writes else (False,)):
                if through and (reads, writes) not in ((0, 1), (1, 1), (2, 1), (3, 1), (2, 2), (4, 2)):
                    continue
                # a margin behind what the call may write, to see that it stops where it says
                d = torch.full(((2 if writes == 2 else 1) * n32 + 1024,), 0x5A5A5A5A, dtype=torch.int32, device=gpu_device)
                before = d.clone()
                probe.stream(d[:max(writes, 1) * n32], a, b, nbytes, reads, writes, per_lane, blocks, through)
                torch.cuda.synchronize()
                if writes == 0:
                    assert torch.equal(d, before)    # a read-only probe stores nothing
                    continue
                srcs = [a[:n32], b[:n32], a[n32:], b[n32:]][:reads]
                if reads:
                    want = srcs[0].clone()
                    for s in srcs[1:]:
                        want += s                    # int32 addition wraps like the kernel's dword addition
                else:
                    want = torch.tensor([0, 1, 2, 3], dtype=torch.int32, device=gpu_device).repeat(n32 // 4)
                    want[0::4] = torch.arange(n32 // 4, device=gpu_device, dtype=torch.int32) // (run // 16)
                for j in range(writes):
                    got = d[j * n32:(j + 1) * n32]
                    assert torch.equal(got, want + j), (reads, writes, per_lane, runs, blocks, through, j)
                assert torch.equal(d[writes * n32:], before[writes * n32:]), "wrote past the tensors it was given"


def test_probe_refuses_before_launching(probe, gpu_device):
    short = torch.zeros(4096, dtype=torch.uint8, device=gpu_device)
    long = torch.zeros(8192, dtype=torch.uint8, device=gpu_device)
    cases = (
        (long, dict(reads=3, writes=1, accesses_per_lane=2), 2),       # 3 + 1 is built for 1 and 6 accesses only
        (long, dict(reads=4, writes=1, accesses_per_lane=1), 2),       # no kernel for 4 + 1
        (long, dict(reads=1, writes=1, accesses_per_lane=3), 2),
        (short, dict(reads=3, writes=1, accesses_per_lane=1), 1),      # the third tensor read needs 2 x nbytes in a
        (short, dict(reads=4, writes=2, accesses_per_lane=1), 1),
        (short, dict(reads=2, writes=2, accesses_per_lane=1), 1),      # the second tensor written needs 2 x nbytes in dst
        (long, dict(reads=5, writes=1, accesses_per_lane=1), 1),
    )
    for buf, kw, status in cases:
        with pytest.raises(probe.ProbeError) as e:
            probe.stream(buf, buf, buf, 4096, persistent_blocks=0, **kw)
        assert e.value.status == status, kw
    torch.cuda.synchronize()
    assert not short.any() and not long.any()                           # nothing ran
