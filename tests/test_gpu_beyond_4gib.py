"""Buffers larger than 4 GiB per rank, and with more than 2^32 elements: every index in the kernels
and their tables is 64 bits wide, the grids stop at 262,144 workgroups and stride over the rest.
Expected values are computed on the GPU with torch's own elementwise kernels (integer sums wrap
around in both; fp32 sums in the ring's order, the division by a power of two being exact), since
the CPU oracle would take minutes at these sizes. Run with -m gpu (needs about 45 GiB of HBM)."""

import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.fixture(autouse=True)
def tidy():
    yield
    from tandem_amd._lib import lib

    assert lib().tdm_set_ring_form(-1) == 0
    torch.cuda.empty_cache()


def same(a, b):
    return a.dtype == b.dtype and a.shape == b.shape and bool(torch.equal(a.view(torch.uint8) if a.element_size() == 1 else a.view(torch.int32), b.view(torch.uint8) if b.element_size() == 1 else b.view(torch.int32)))


def test_two_ranks_of_int8_with_more_than_2_to_the_32_elements():
    from tandem_amd import LocalWorld
    from tandem_amd._lib import lib

    dev = torch.device("cuda", 0)
    n = (1 << 32) + 4099 + 77
    gen = torch.Generator(device=dev).manual_seed(1)
    xs = [torch.randint(-128, 128, (n,), dtype=torch.int8, device=dev, generator=gen) for _ in range(2)]
    total = xs[0] + xs[1]  # wraps, as the kernels' sum does
    assert not same(total, xs[0])
    lw = LocalWorld(2)
    sizes = [1 << 32, n - (1 << 32)]  # chunk 0 alone is 4 GiB; chunk 1 starts beyond the 32-bit range
    for form in (0, 1):
        assert lib().tdm_set_ring_form(form) == 0
        print(f"int8 x 2 ranks, {n} elements, ring form {form}", flush=True)
        bufs = [x.clone() for x in xs]
        lw.all_reduce(bufs, algorithm="ring")
        assert same(bufs[0], total) and same(bufs[1], total), form
        bufs = [x.clone() for x in xs]
        mine = lw.reduce_scatter(bufs, sizes)
        assert same(bufs[0][:sizes[0]], total[:sizes[0]]) and same(bufs[0][sizes[0]:], xs[0][sizes[0]:]), form
        assert same(bufs[1][:sizes[0]], xs[1][:sizes[0]]) and same(bufs[1][sizes[0]:], total[sizes[0]:]), form
        assert mine[1].data_ptr() == bufs[1].data_ptr() + sizes[0]
        lw.all_gather(bufs, sizes)
        assert same(bufs[0], total) and same(bufs[1], total), form
        del bufs, mine
    bufs = [x.clone() for x in xs]
    lw.all_reduce(bufs, algorithm="fold")
    assert same(bufs[0], total) and same(bufs[1], total)


def test_four_ranks_of_fp32_beyond_four_gib_each():
    from tandem_amd import LocalWorld
    from tandem_amd._lib import lib
    from tandem_amd.local import chunk_bounds

    dev = torch.device("cuda", 0)
    world, n = 4, (1 << 30) + 4099
    gen = torch.Generator(device=dev).manual_seed(2)
    xs = [torch.randn(n, device=dev, generator=gen) * 1e-2 for _ in range(world)]
    bounds = chunk_bounds(n, world)

    def partial(c, upto):  # chunk c after `upto` ranks of the ring have added theirs
        lo, hi = bounds[c]
        acc = xs[(c + 1) % world][lo:hi] * 0.25
        for k in range(2, upto + 1):
            acc = xs[(c + k) % world][lo:hi] * 0.25 + acc
        return acc

    want = torch.cat([partial(c, world) for c in range(world)])
    lw = LocalWorld(world)
    for form in (1, 0):
        assert lib().tdm_set_ring_form(form) == 0
        print(f"fp32 x 4 ranks, {n} elements, ring form {form}", flush=True)
        bufs = [x.clone() for x in xs]
        lw.reduce_scatter(bufs, op="avg")
        for c, (lo, hi) in enumerate(bounds):
            for k in range(1, world + 1):
                assert same(bufs[(c + k) % world][lo:hi], partial(c, k)), (form, c, k)
        lw.all_gather(bufs)
        for r in range(world):
            assert same(bufs[r], want), (form, r)
        del bufs
    bufs = [x.clone() for x in xs]
    lw.all_reduce(bufs, op="avg", algorithm="fold")
    for r in range(world):
        assert same(bufs[r], want), r


def test_bucket_table_and_adamw_over_a_tensor_beyond_four_gib():
    from tandem_amd import LocalWorld, ShardedAdamW

    dev = torch.device("cuda", 0)
    n = (1 << 30) + 4099
    gen = torch.Generator(device=dev).manual_seed(3)
    grads = [[torch.randn(n, device=dev, generator=gen) * 1e-3, torch.randn(33, device=dev, generator=gen)] for _ in range(2)]
    want = [a * 0.5 + b * 0.5 for a, b in zip(*grads)]
    print(f"bucket table over {n} + 33 elements, 2 ranks", flush=True)
    table = LocalWorld(2).bucket_table(grads, [[1, 0]])
    table.run(average=True)
    for r in range(2):
        for i in range(2):
            assert same(grads[r][i], want[i]), (r, i)
    del table, want
    # K3 against torch's own AdamW on the GPU (its order of operations: order="device")
    kw = dict(lr=3e-4, betas=(0.9, 0.95), eps=1e-8, weight_decay=0.1)
    g = grads[0][0]
    del grads
    p0 = torch.randn(n, device=dev, generator=gen) * 0.02
    pt = torch.nn.Parameter(p0.clone())
    topt = torch.optim.AdamW([pt], foreach=False, fused=False, **kw)
    ours = ShardedAdamW(order="device", **kw)
    print(f"AdamW over {n} elements", flush=True)
    for _ in range(2):
        pt.grad = g
        topt.step()
        ours.update(0, p0, g)
    st = topt.state[pt]
    assert same(ours.state[0][1], st["exp_avg"]) and same(ours.state[0][2], st["exp_avg_sq"])
    assert same(p0, pt.detach())
