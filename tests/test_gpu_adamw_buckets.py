"""K3 (sharded AdamW) and K2 (bucket fold) on the GPU against the CPU oracle,
the reference's fixtures and torch's own AdamW. Run with -m gpu on an MI355X."""

import math

import numpy as np
import pytest
import torch

from helpers import bits, golden_json, golden_npz, npz_json, seeded

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def dev():
    assert torch.cuda.is_available(), "these tests need the MI355X"
    return torch.device("cuda", 0)


def test_adamw_bit_exact_with_oracle(dev):
    """Twenty steps with the benchmark's hyper-parameters, on a shard whose length
    is not a multiple of anything; then the other branches (no decay, beta1 < 0.5)
    and a shard that starts 4 bytes off a 16-byte boundary."""
    from oracle.adamw import AdamW as Oracle
    from tandem_amd import ShardedAdamW

    n = 100_003
    g = torch.Generator().manual_seed(5)
    p0 = torch.randn(n, generator=g) * 0.02
    p0[:6] = torch.tensor([0.0, -0.0, 1e-30, -3e-39, 1e-45, 5.0])
    for kw, shift in ((dict(lr=3e-4, betas=(0.9, 0.95), eps=1e-8, weight_decay=0.1), 0),
                      (dict(lr=1e-3, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.0), 0),
                      (dict(lr=1e-2, betas=(0.3, 0.7), eps=1e-6, weight_decay=0.5), 1)):
        ours, ref = ShardedAdamW(**kw), Oracle(**kw)
        store = torch.zeros(n + 4, device=dev)
        p = store[shift:shift + n]
        p.copy_(p0)
        pn = p0.numpy().copy()
        for step in range(20):
            gr = torch.randn(n, generator=g) * 1e-3
            gr[:3] = 0.0
            ours.update("k", p, gr.to(dev))
            ref.update("k", pn, gr.numpy())
        _, m, v = ours.state["k"]
        assert np.array_equal(bits(m.cpu().numpy()), bits(ref.state["k"][1])), kw
        assert np.array_equal(bits(v.cpu().numpy()), bits(ref.state["k"][2])), kw
        assert np.array_equal(bits(p.cpu().numpy()), bits(pn)), kw
        assert ours.state["k"][0] == 20.0 and ours.state_bytes() == 2 * 4 * n


def test_adamw_against_reference_fixture(dev):
    """The reference ran on torch's CPU kernels, whose vectorised sqrt is not
    correctly rounded: moments must match bit for bit, parameters to 1 ulp of the
    update term per step."""
    from tandem_amd import ShardedAdamW

    d = golden_npz("adamw.npz")
    h = npz_json(d, "hyper_json")["main"]
    opt = ShardedAdamW(h["lr"], tuple(h["betas"]), h["eps"], h["weight_decay"])
    p = torch.from_numpy(d["p0"].copy()).to(dev)
    for s in range(h["steps"]):
        opt.update("k", p, torch.from_numpy(d["grads"][s].copy()).to(dev))
        if s == 0:
            _, m, v = opt.state["k"]
            assert np.array_equal(bits(m.cpu().numpy()), bits(d["m1"]))
            assert np.array_equal(bits(v.cpu().numpy()), bits(d["v1"]))
            upd = np.abs(d["p1"].astype(np.float64) - d["p0"].astype(np.float64) * (1 - h["lr"] * h["weight_decay"]))
            tol = np.spacing(upd.astype(np.float32)).astype(np.float64) + np.spacing(np.abs(d["p1"])).astype(np.float64)
            assert np.all(np.abs(p.cpu().numpy().astype(np.float64) - d["p1"]) <= tol)
    _, m, v = opt.state["k"]
    assert np.array_equal(bits(m.cpu().numpy()), bits(d["m20"]))
    assert np.array_equal(bits(v.cpu().numpy()), bits(d["v20"]))
    got = p.cpu().numpy()
    assert np.abs(got.astype(np.float64) - d["p20"]).max() <= 20 * 2 * np.spacing(np.float32(h["lr"]))
    assert (bits(got) != bits(d["p20"])).mean() < 0.05


def test_adamw_device_order_matches_torch_on_the_gpu(dev):
    """torch.optim.AdamW(foreach=False) run on the GPU itself: its addcdiv_ kernel
    computes fma(step, m/d, p); order="device" reproduces that bit for bit."""
    from tandem_amd import ShardedAdamW

    n = 250_000
    g = torch.Generator().manual_seed(8)
    p0 = torch.randn(n, generator=g) * 0.02
    kw = dict(lr=3e-4, betas=(0.9, 0.95), eps=1e-8, weight_decay=0.1)
    pt = torch.nn.Parameter(p0.clone().to(dev))
    topt = torch.optim.AdamW([pt], foreach=False, fused=False, **kw)
    ours = ShardedAdamW(order="device", **kw)
    p = p0.clone().to(dev)
    for _ in range(20):
        gr = (torch.randn(n, generator=g) * 1e-3).to(dev)
        pt.grad = gr.clone()
        topt.step()
        ours.update(0, p, gr)
    st = topt.state[pt]
    assert torch.equal(ours.state[0][1].view(torch.int32), st["exp_avg"].view(torch.int32))
    assert torch.equal(ours.state[0][2].view(torch.int32), st["exp_avg_sq"].view(torch.int32))
    assert torch.equal(p.view(torch.int32), pt.detach().view(torch.int32))


def test_adamw_writing_further_copies(dev):
    """The update that also writes the other ranks' copies of the shard (update and
    all-gather in one pass): the same bits as the plain update in p, m, v, and the new
    p in every copy; aligned and unaligned, one and seven copies; overlap refused."""
    from tandem_amd import ShardedAdamW

    kw = dict(lr=3e-4, betas=(0.9, 0.95), eps=1e-8, weight_decay=0.1)
    g = torch.Generator().manual_seed(9)
    for n, ncopies, shift in ((100_003, 1, 0), (4099, 7, 0), (65_536, 3, 0), (10_007, 3, 1)):
        p0 = torch.randn(n, generator=g) * 0.02
        plain, fused = ShardedAdamW(**kw), ShardedAdamW(**kw)
        p = p0.clone().to(dev)
        q_store = torch.zeros(n + 4, device=dev)
        q = q_store[shift:shift + n]
        q.copy_(p0)
        stores = [torch.full((n + 8,), -7.0, device=dev) for _ in range(ncopies)]
        copies = [st[shift + 1:shift + 1 + n] if shift else st[4:4 + n] for st in stores]
        for step in range(3):
            gr = (torch.randn(n, generator=g) * 1e-3).to(dev)
            plain.update("k", p, gr)
            fused.update("k", q, gr, copies)
            for c in copies:
                assert torch.equal(c.view(torch.int32), p.view(torch.int32)), (n, ncopies, step)
        assert torch.equal(q.view(torch.int32), p.view(torch.int32))
        for i in (1, 2):
            assert torch.equal(fused.state["k"][i].view(torch.int32), plain.state["k"][i].view(torch.int32))
        for st in stores:  # nothing outside the copies was written
            lo = shift + 1 if shift else 4
            assert float((st[:lo] + 7.0).abs().sum()) == 0 and float((st[lo + n:] + 7.0).abs().sum()) == 0
    with pytest.raises(ValueError, match="overlap"):
        fused.update("k", q, gr, [q])
    with pytest.raises(ValueError, match="shape"):
        fused.update("k", q, gr, [torch.zeros(n + 1, device=dev)])
    with pytest.raises(ValueError, match="at most 7"):
        fused.update("k", q, gr, [torch.zeros(n, device=dev) for _ in range(8)])


@pytest.mark.parametrize("order", ["host", "device"])
def test_adamw_on_a_shard_off_the_16_byte_grid(dev, order):
    """tensor_split shards start anywhere. With p, g, m, v (and the copies) all at the
    same distance from a 16-byte boundary the launcher peels that head and runs vectors,
    and when they also share their distance from a 128-byte boundary it peels up to that
    line (as many as 31 elements); with streams that disagree within 16 bytes it goes
    element by element. All against the plain aligned update on the same numbers, which
    the tests above pin to the oracle and to torch: phases of 1..31 elements, streams that
    agree only within 16 bytes, lengths that leave a head, a tail, both, fewer elements than
    the head, with and without copies; guard elements around every stream stay untouched."""
    import ctypes

    from tandem_amd import _lib
    from tandem_amd._lib import check, lib, stream_ptr
    from tandem_amd.optim import step_scalars

    kw = dict(lr=3e-4, betas=(0.9, 0.95), eps=1e-8, weight_decay=0.1)
    code = _lib.ADAMW_HOST_ORDER if order == "host" else _lib.ADAMW_DEVICE_ORDER
    gen = torch.Generator().manual_seed(12)
    st = stream_ptr(dev)

    def run(n, phases, ncopies):
        """Three steps over streams laid at the given phases (elements off a 16-byte boundary) inside guarded stores."""
        pad = 64  # two cache lines of guard elements either side
        stores = [torch.full((n + 2 * pad,), -7.0, device=dev) for _ in range(4 + ncopies)]
        views = [s_[pad + ph:pad + ph + n] for s_, ph in zip(stores, phases)]
        for v_, ph in zip(views, phases):
            assert v_.data_ptr() % 128 == 4 * ph
        views[0].copy_(p0[:n])
        views[2].zero_()
        views[3].zero_()
        for step in range(3):
            views[1].copy_(grads[step][:n])
            s_ = step_scalars(step + 1.0, kw["lr"], kw["betas"], kw["eps"], kw["weight_decay"])
            ptr = [ctypes.c_void_p(v_.data_ptr()) for v_ in views]
            if ncopies:
                arr = (ctypes.c_void_p * ncopies)(*[v_.data_ptr() for v_ in views[4:]])
                check(lib().tdm_k3_adamw_gather(ptr[0], ptr[1], ptr[2], ptr[3], n, ctypes.byref(s_), code, arr, ncopies, st))
            else:
                check(lib().tdm_k3_adamw(ptr[0], ptr[1], ptr[2], ptr[3], n, ctypes.byref(s_), code, st))
        for s_, ph in zip(stores, phases):  # nothing outside the streams was written
            assert float((s_[:pad + ph] + 7.0).abs().sum()) == 0 and float((s_[pad + ph + n:] + 7.0).abs().sum()) == 0
        return [v_.clone() for v_ in views]

    for n in (1, 2, 3, 5, 30, 31, 33, 127, 4099, 100_003):
        p0 = torch.randn(n, generator=gen).to(dev) * 0.02
        grads = [(torch.randn(n, generator=gen) * 1e-3).to(dev) for _ in range(3)]
        for ncopies in (0, 2):
            want = run(n, [0] * (4 + ncopies), ncopies)
            layouts = [[ph] * 6 for ph in (1, 2, 3, 4, 5, 17, 30, 31)]  # one phase for all: peeled to the cache line, vectors
            layouts += [[1, 5, 9, 13, 17, 29], [3, 3, 7, 3, 31, 3]]     # agreeing within 16 bytes only: peeled to the vector
            layouts += [[1, 0, 3, 2, 1, 2]]                             # disagreeing: element by element
            for phases in layouts:
                got = run(n, phases[:4 + ncopies], ncopies)
                for a, b in zip(want, got):
                    assert torch.equal(a.view(torch.int32), b.view(torch.int32)), (n, phases, ncopies, order)


def test_optimizer_state_follows_the_shards_phase(dev):
    """ShardedAdamW lays a shard's exp_avg and exp_avg_sq out at the shard's own distance from
    a 128-byte boundary, and ZeRO's gradient shard likewise, so that the update of a
    tensor_split shard that starts anywhere still runs on vectors."""
    from tandem_amd import ShardedAdamW
    from tandem_amd.optim import zeros_at_phase_of

    flat = torch.zeros(1000, device=dev)
    opt = ShardedAdamW()
    for lo in (0, 1, 2, 3, 29):
        p = flat[lo:lo + 333]
        g = zeros_at_phase_of(p)
        assert g.numel() == 333 and g.data_ptr() % 128 == p.data_ptr() % 128 and float(g.abs().sum()) == 0
        opt.update(lo, p, g)
        _, m, v = opt.state[lo]
        assert m.data_ptr() % 128 == v.data_ptr() % 128 == p.data_ptr() % 128
        assert m.numel() == v.numel() == 333
    assert opt.state_bytes() == 5 * 2 * 4 * 333
    half = torch.zeros(64, device=dev, dtype=torch.float16)[3:40]
    assert zeros_at_phase_of(half).data_ptr() % 128 == half.data_ptr() % 128 and zeros_at_phase_of(half, 5).numel() == 5


def _raw(t):
    t = t.detach().cpu()
    return t.view(torch.int16).numpy().view(np.uint16).copy() if t.element_size() == 2 else t.numpy().copy()


@pytest.mark.parametrize("case", ["main", "other"])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float64])
def test_adamw_bf16_and_f64_against_the_reference_fixture(dev, dtype, case):
    """tests/golden/adamw_dtypes.npz: the reference's ShardedAdamW on bfloat16 and float64 shards, 20 steps of
    the benchmark's hyper-parameters and 3 steps of the other branches. Against the fixture: bfloat16 bit for
    bit in p, m, v; float64 bit for bit in the moments and within 1 ulp of each step's update term in p (the
    reference ran torch's vectorised CPU sqrt, which is not correctly rounded). Against the oracle (pinned by
    the same fixture with torch's sqrt substituted): bit for bit in everything."""
    from oracle.adamw import AdamW as Oracle
    from tandem_amd import ShardedAdamW

    name = {torch.bfloat16: "bf16", torch.float16: "f16", torch.float64: "f64"}[dtype]
    d = golden_npz("adamw_dtypes.npz")
    h = npz_json(d, "hyper_json")[case]
    kw = dict(lr=h["lr"], betas=tuple(h["betas"]), eps=h["eps"], weight_decay=h["weight_decay"])
    last = h["steps"]

    def dev_tensor(a):
        t = torch.from_numpy(np.ascontiguousarray(a).copy())
        return (t.view(dtype) if name != "f64" else t).to(dev)

    ours, ref = ShardedAdamW(**kw), Oracle(**kw, kind=name if name != "f64" else None)
    p = dev_tensor(d[f"{name}_p0"])
    pn = (d[f"{name}_p0"].view(np.uint16) if name != "f64" else d[f"{name}_p0"]).copy()
    for s in range(last):
        g = d[f"{name}_grads"][s]
        ours.update("k", p, dev_tensor(g))
        ref.update("k", pn, np.ascontiguousarray(g.view(np.uint16) if name != "f64" else g))
    _, m, v = ours.state["k"]
    assert m.dtype == dtype and v.dtype == dtype
    assert np.array_equal(bits(_raw(m)), bits(ref.state["k"][1])) and np.array_equal(bits(_raw(v)), bits(ref.state["k"][2]))
    assert np.array_equal(bits(_raw(p)), bits(pn))
    assert np.array_equal(bits(_raw(m)), bits(d[f"{name}_{case}_m{last}"]))
    assert np.array_equal(bits(_raw(v)), bits(d[f"{name}_{case}_v{last}"]))
    want = d[f"{name}_{case}_p{last}"]
    if name == "bf16":
        assert np.array_equal(bits(_raw(p)), bits(want))
    elif name == "f16":
        # float16 cannot hold eps = 1e-8 nor the squares of these gradients: a good part of the reference's parameters are
        # infinities and NaNs. Infinities bit for bit, NaNs by position (stored here as the canonical 0x7e00), the rest bit for bit.
        got, w = _raw(p), want.view(np.uint16)
        nan = (w & 0x7fff) > 0x7c00
        assert np.array_equal((got & 0x7fff) > 0x7c00, nan) and np.array_equal(got[~nan], w[~nan])
        assert np.all(got[nan] == 0x7e00) and (case != "main" or nan.sum() > 50)
    else:
        assert np.abs(_raw(p) - want).max() <= last * 2 * np.spacing(h["lr"])
        assert (bits(_raw(p)) != bits(want)).mean() < 0.05


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float64])
def test_adamw_bf16_and_f64_on_odd_shards_with_copies(dev, dtype):
    """The typed kernel's vector path (8 bf16 or 2 doubles per 16 bytes), its peeled head (up to a cache line),
    its tail, the element-by-element path for streams that disagree, and the copies written in the same pass:
    three steps against the oracle, guard elements untouched."""
    from oracle.adamw import AdamW as Oracle
    from tandem_amd import ShardedAdamW

    kw = dict(lr=1e-3, betas=(0.9, 0.95), eps=1e-6, weight_decay=0.1)
    gen = torch.Generator().manual_seed(31)
    per_line = 128 // torch.empty(0, dtype=dtype).element_size()
    for n in (1, 7, 9, 63, 65, 4099, 50_001):
        p0 = (torch.randn(n, generator=gen, dtype=torch.float64) * 0.02).to(dtype)
        grads = [(torch.randn(n, generator=gen, dtype=torch.float64) * 1e-3).to(dtype) for _ in range(3)]
        ref = Oracle(**kw, kind={torch.bfloat16: "bf16", torch.float16: "f16"}.get(dtype))
        pn = _raw(p0)
        for g in grads:
            ref.update("k", pn, _raw(g))
        for phases, ncopies in (([0, 0, 0, 0], 0), ([1, 1, 1, 1, 1, 1], 2), ([per_line - 1] * 5, 1), ([3, 3 + 8, 3, 3 + 16], 0), ([1, 0, 2, 1], 0)):
            pad = 2 * per_line
            stores = [torch.full((n + 2 * pad,), -7.0, dtype=dtype, device=dev) for _ in range(4 + ncopies)]
            views = [s_[pad + ph:pad + ph + n] for s_, ph in zip(stores, phases)]
            p, g, copies = views[0], views[1], views[4:]
            p.copy_(p0)
            ours = ShardedAdamW(**kw)
            ours.state["k"] = [0.0, views[2].zero_(), views[3].zero_()]
            for gr in grads:
                g.copy_(gr)
                ours.update("k", p, g, copies)
            what = (dtype, n, phases)
            assert np.array_equal(bits(_raw(p)), bits(pn)), what
            assert np.array_equal(bits(_raw(views[2])), bits(ref.state["k"][1])), what
            assert np.array_equal(bits(_raw(views[3])), bits(ref.state["k"][2])), what
            for c in copies:
                assert np.array_equal(bits(_raw(c)), bits(pn)), what
            for s_, ph in zip(stores, phases):
                assert float((s_[:pad + ph].double() + 7.0).abs().sum()) == 0 and float((s_[pad + ph + n:].double() + 7.0).abs().sum()) == 0, what


def test_bf16_square_roots_and_divisors_over_every_second_moment(dev):
    """The bfloat16 kernel takes the hardware's square root and a product with 1/bc2_sqrt where the oracle takes the
    correctly rounded root and a true division, and goes the oracle's way only near a rounding tie, for floats the
    root instruction does not take, and for divisors outside [2^-30, 2^30]. Every one of the 65,536 bit patterns as
    the second moment (zeros, denormals, negative numbers, infinities, NaNs among them; beta2 = 1 and a zero gradient
    leave it as it is), sixteen first moments each so that a denominator one step off shows in the parameter, against
    divisors from the steps of three beta2, the window's two ends, values beyond them, 0, infinity, NaN and a negative
    number: bit for bit with the oracle."""
    import ctypes

    from oracle import lib as oracle_lib
    from tandem_amd import _lib

    L, O = _lib.lib(), oracle_lib()
    moments = (np.arange(16, dtype=np.uint16) << 3) + 0x3f80  # 1, 1.0625 ... 1.9375 as bf16 patterns
    moments[8:] |= 0x8000
    v0 = np.repeat(np.arange(65536, dtype=np.uint32).astype(np.uint16), moments.size)
    m0 = np.tile(moments, 65536)
    n = v0.size
    divisors = [math.sqrt(1 - b ** t) for b in (0.95, 0.999, 0.98) for t in (1, 2, 3, 7, 20, 100, 1000)]
    divisors += [1.0, 2.0 ** -30, 2.0 ** 30, 2.0 ** -31, 2.0 ** 31, 1e-38, 3.0, 0.0, math.inf, math.nan, -0.5]
    f = ctypes.c_float
    for k, c in enumerate(divisors):
        c = float(np.float32(c))
        eps = (1e-8, 0.0, 1e-3)[k % 3]
        h = _lib.AdamwHyper(use_decay=0, decay=1.0, w1=0.0, beta2=1.0, one_m_b2=0.0, bc2_sqrt=c, eps=eps, neg_step=-1.0)
        t = [torch.from_numpy(a.view(np.int16).copy()).view(torch.bfloat16).to(dev) for a in (np.zeros(n, np.uint16), np.zeros(n, np.uint16), m0, v0)]
        _lib.check(L.tdm_k3_adamw_typed(*(x.data_ptr() for x in t), n, _lib.DTYPES[torch.bfloat16], ctypes.byref(h), _lib.ADAMW_HOST_ORDER, None, 0, _lib.stream_ptr(dev)))
        want = [np.zeros(n, np.uint16), np.zeros(n, np.uint16), m0.copy(), v0.copy()]
        O.orc_adamw_bf16(*(ctypes.c_void_p(a.ctypes.data) for a in want), ctypes.c_int64(n), ctypes.c_int(0), f(1.0), f(0.0), f(1.0), f(0.0),
                         f(c), f(eps), f(-1.0))
        for name, got, w in zip("pgmv", t, want):
            got = _raw(got)
            bad = np.flatnonzero(got != w)
            assert bad.size == 0, (c, name, bad.size, [(hex(v0[i]), hex(m0[i]), hex(got[i]), hex(w[i])) for i in bad[:5]])


def test_adamw_rejects_what_it_cannot_do(dev):
    from tandem_amd import ShardedAdamW

    opt = ShardedAdamW()
    with pytest.raises(ValueError):
        opt.update("cpu", torch.zeros(4), torch.zeros(4))
    with pytest.raises(ValueError):
        opt.update("int", torch.zeros(4, device=dev, dtype=torch.int32), torch.zeros(4, device=dev, dtype=torch.int32))
    with pytest.raises(ValueError, match="same dtype"):
        opt.update("mixed", torch.zeros(4, device=dev, dtype=torch.bfloat16), torch.zeros(4, device=dev))
    with pytest.raises(ValueError, match="fp32 shards only"):
        ShardedAdamW(order="device").update("d", torch.zeros(4, device=dev, dtype=torch.float64), torch.ones(4, device=dev, dtype=torch.float64))
    opt.update("empty", torch.zeros(0, device=dev), torch.zeros(0, device=dev))
    assert opt.state["empty"][0] == 1.0
    p = torch.zeros(8, device=dev)
    with pytest.raises(ValueError):
        opt.update("alias", p, p)  # p and g overlap


@pytest.mark.parametrize("world", [2, 3, 4])
def test_bucket_fold_equals_flatten_allreduce_unflatten(dev, world):
    """K2 against the oracle's ring all-reduce of each flattened bucket, for the
    small GPT's parameter list with the reference's packing (plans.json)."""
    from oracle import ring
    from tandem_amd import LocalWorld
    from tandem_amd.buckets import pack

    plan = golden_json("plans.json")
    names = [n for n, _ in plan["small_params"]]
    numels = [math.prod(s) for _, s in plan["small_params"]]
    order = list(range(len(numels)))[::-1]
    groups = pack([numels[i] * 4 for i in order], 4 << 10)
    buckets = [[order[k] for k in grp] for grp in groups]
    assert [[names[i] for i in b] for b in buckets] == plan["small_ddp_4KiB"]
    grads = [[(seeded(r, i, numels[i]) * 1e-3) for i in range(len(numels))] for r in range(world)]
    dgrads = [[t.to(dev) for t in grads[r]] for r in range(world)]
    lw = LocalWorld(world)
    table = lw.bucket_table(dgrads, buckets)
    assert table.elements == sum(numels)
    table.run(average=True)
    for b in buckets:
        flat = [np.concatenate([grads[r][i].numpy() for i in b]) for r in range(world)]
        want = ring.expected_all_reduce(flat, True)
        off = 0
        for i in b:
            for r in range(world):
                assert np.array_equal(bits(dgrads[r][i].cpu().numpy()), bits(want[off:off + numels[i]])), (world, i, r)
            off += numels[i]


def test_bucket_fold_into_other_buffers_and_odd_sizes(dev):
    from oracle import ring
    from tandem_amd import LocalWorld

    world = 4
    numels = [1, 3, 1025, 7, 4096, 10_007, 2]
    grads = [[seeded(r + 5, i, n) for i, n in enumerate(numels)] for r in range(world)]
    dgrads = [[t.to(dev) for t in grads[r]] for r in range(world)]
    outs = [[torch.zeros_like(t) for t in dgrads[r]] for r in range(world)]
    buckets = [[6, 5, 4], [3, 2], [1, 0]]
    LocalWorld(world).bucket_table(dgrads, buckets, outs).run(average=False)
    for b in buckets:
        flat = [np.concatenate([grads[r][i].numpy() for i in b]) for r in range(world)]
        want = ring.expected_all_reduce(flat, False)
        off = 0
        for i in b:
            for r in range(world):
                assert np.array_equal(bits(outs[r][i].cpu().numpy()), bits(want[off:off + numels[i]]))
                assert torch.equal(dgrads[r][i].cpu(), grads[r][i])  # sources untouched
            off += numels[i]


@pytest.mark.parametrize("dtype", [torch.float64, torch.bfloat16, torch.float16, torch.int64, torch.int32, torch.int16, torch.int8, torch.uint8])
def test_bucket_fold_of_every_element_type(dev, dtype):
    """The table-driven fold over the other element types the header names: odd tensor sizes, so most
    segments start off the 16-byte grid; integers over their whole range, so their sums wrap around."""
    from oracle import ring
    from tandem_amd import LocalWorld

    kind = {torch.float64: "f64", torch.bfloat16: "bf16", torch.float16: "f16", torch.int64: "i64", torch.int32: "i32",
            torch.int16: "i16", torch.int8: "i8", torch.uint8: "u8"}[dtype]
    world = 3
    numels = [1, 3, 1025, 7, 4096, 10_007, 2, 33]
    def make(r, i, n):
        if dtype.is_floating_point:
            return seeded(r + 11, i, n).to(dtype)
        g = torch.Generator().manual_seed(100 * r + i)
        if dtype == torch.int64:
            return torch.randint(-(1 << 40), 1 << 40, (n,), generator=g)
        info = torch.iinfo(dtype)
        return torch.randint(info.min, info.max + 1, (n,), generator=g).to(dtype)
    def raw(t):
        t = t.cpu()
        return t.view(torch.int16).numpy().view(np.uint16) if dtype in (torch.bfloat16, torch.float16) else t.numpy()
    grads = [[make(r, i, n) for i, n in enumerate(numels)] for r in range(world)]
    dgrads = [[t.to(dev) for t in grads[r]] for r in range(world)]
    buckets = [[7, 6, 5], [4, 3], [2, 1, 0]]
    average = dtype.is_floating_point
    LocalWorld(world).bucket_table(dgrads, buckets).run(average=average)
    for b in buckets:
        flat = [np.concatenate([raw(grads[r][i]) for i in b]) for r in range(world)]
        want = ring.expected_all_reduce(flat, average, kind)
        off = 0
        for i in b:
            for r in range(world):
                assert np.array_equal(bits(raw(dgrads[r][i])), bits(want[off:off + numels[i]])), (dtype, i, r)
            off += numels[i]
