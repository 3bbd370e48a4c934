"""The AdamW oracle against the reference's ShardedAdamW outputs (tests/golden/adamw.npz),
against torch.optim.AdamW(foreach=False) (what the reference itself is tested
against), and against a float64 evaluation of the textbook formulas."""

import numpy as np
import pytest
import torch

from oracle.adamw import AdamW, scalars

from helpers import bits, golden_npz, npz_json


def torch_sqrt(v):
    return torch.from_numpy(v).sqrt().numpy()


def run(opt, p0, grads, steps, snaps=()):
    p = p0.copy()
    out = {}
    for s in range(steps):
        opt.update("k", p, np.ascontiguousarray(grads[s]))
        if s + 1 in snaps:
            _, m, v = opt.state["k"]
            out[s + 1] = (p.copy(), m.copy(), v.copy())
    return p, out


def test_bit_exact_with_reference_when_torch_sqrt_is_substituted():
    d = golden_npz("adamw.npz")
    h = npz_json(d, "hyper_json")["main"]
    opt = AdamW(h["lr"], tuple(h["betas"]), h["eps"], h["weight_decay"], sqrt=torch_sqrt)
    _, snaps = run(opt, d["p0"], d["grads"], h["steps"], snaps=(1, 2, 20))
    for s, (p, m, v) in snaps.items():
        assert np.array_equal(bits(m), bits(d[f"m{s}"])), s
        assert np.array_equal(bits(v), bits(d[f"v{s}"])), s
        assert np.array_equal(bits(p), bits(d[f"p{s}"])), s
    h2 = npz_json(d, "hyper_json")["nowd"]
    opt2 = AdamW(h2["lr"], tuple(h2["betas"]), h2["eps"], h2["weight_decay"], sqrt=torch_sqrt)
    p, _ = run(opt2, d["p0"], d["grads"], 3)
    assert np.array_equal(bits(p), bits(d["nowd_p3"]))


def test_correctly_rounded_sqrt_moments_exact_params_within_one_ulp_of_the_update():
    """torch's vectorised CPU sqrt is 1 ulp off on a fraction of a percent of
    inputs; with the IEEE sqrtf the moments are still bit-identical and each
    step's parameter differs by at most 1 ulp of that step's update term."""
    d = golden_npz("adamw.npz")
    h = npz_json(d, "hyper_json")["main"]
    opt = AdamW(h["lr"], tuple(h["betas"]), h["eps"], h["weight_decay"])
    _, snaps = run(opt, d["p0"], d["grads"], h["steps"], snaps=(1, 20))
    p1, m1, v1 = snaps[1]
    assert np.array_equal(bits(m1), bits(d["m1"])) and np.array_equal(bits(v1), bits(d["v1"]))
    p20, m20, v20 = snaps[20]
    assert np.array_equal(bits(m20), bits(d["m20"])) and np.array_equal(bits(v20), bits(d["v20"]))
    # one step: |dp| <= ulp(update) + ulp(p) (the sum is rounded once more)
    upd = np.abs(d["p1"].astype(np.float64) - d["p0"].astype(np.float64) * (1 - h["lr"] * h["weight_decay"]))
    tol1 = np.spacing(upd.astype(np.float32)).astype(np.float64) + np.spacing(np.abs(d["p1"])).astype(np.float64)
    assert np.all(np.abs(p1.astype(np.float64) - d["p1"]) <= tol1)
    assert (bits(p1) != bits(d["p1"])).mean() < 0.02
    # twenty steps: the update is ~lr per step
    assert np.abs(p20.astype(np.float64) - d["p20"]).max() <= 20 * 2 * np.spacing(np.float32(h["lr"]))
    assert (bits(p20) != bits(d["p20"])).mean() < 0.05


def test_matches_torch_adamw_single_tensor_path():
    n = 4099
    g = torch.Generator().manual_seed(3)
    p0 = (torch.randn(n, generator=g) * 0.02)
    grads = [torch.randn(n, generator=g) * 1e-2 for _ in range(5)]
    for kw in (dict(lr=3e-3, weight_decay=0.1), dict(lr=1e-3, betas=(0.5, 0.999), weight_decay=0.0),
               dict(lr=1e-2, betas=(0.3, 0.7), eps=1e-6, weight_decay=0.5)):  # beta1 < 0.5: lerp's other branch
        pt = torch.nn.Parameter(p0.clone())
        topt = torch.optim.AdamW([pt], foreach=False, **kw)
        opt = AdamW(sqrt=torch_sqrt, **{"betas": (0.9, 0.999), "eps": 1e-8, **kw})
        p = p0.numpy().copy()
        for gr in grads:
            pt.grad = gr.clone()
            topt.step()
            opt.update(0, p, gr.numpy())
        st = topt.state[pt]
        assert np.array_equal(bits(opt.state[0][1]), bits(st["exp_avg"].numpy())), kw
        assert np.array_equal(bits(opt.state[0][2]), bits(st["exp_avg_sq"].numpy())), kw
        assert np.array_equal(bits(p), bits(pt.detach().numpy())), kw


def test_against_float64_textbook_adamw():
    """Independent of torch: the textbook recurrences in float64 agree to fp32 rounding."""
    n, steps = 2048, 10
    rng = np.random.default_rng(0)
    p0 = (rng.standard_normal(n) * 0.02).astype(np.float32)
    grads = (rng.standard_normal((steps, n)) * 1e-3).astype(np.float32)
    lr, b1, b2, eps, wd = 3e-4, 0.9, 0.95, 1e-8, 0.1
    opt = AdamW(lr, (b1, b2), eps, wd)
    p, _ = run(opt, p0, grads, steps)
    P, M, V = p0.astype(np.float64), np.zeros(n), np.zeros(n)
    for t in range(1, steps + 1):
        g = grads[t - 1].astype(np.float64)
        P = P * (1 - lr * wd)
        M = b1 * M + (1 - b1) * g
        V = b2 * V + (1 - b2) * g * g
        P = P - lr / (1 - b1 ** t) * M / (np.sqrt(V) / np.sqrt(1 - b2 ** t) + eps)
    assert np.abs(p - P).max() < 5e-8
    assert np.abs(opt.state["k"][1] - M).max() < 1e-9 and np.abs(opt.state["k"][2] - V).max() < 1e-12


def test_scalars_and_empty_shard():
    s = scalars(1.0, 3e-4, (0.9, 0.95), 1e-8, 0.1)
    assert s["use_decay"] == 1 and s["decay"] == float(np.float32(1 - 3e-4 * 0.1))
    assert s["neg_step"] == float(np.float32(-(3e-4 / (1 - 0.9 ** 1.0))))
    opt = AdamW()
    opt.update("e", np.zeros(0, np.float32), np.zeros(0, np.float32))
    assert opt.state["e"][0] == 1.0  # the step still counts (tandem/optim.py:24-27)


def test_16bit_conversions_match_numpy_and_torch():
    import ctypes

    from oracle import lib

    allbits = np.arange(65536, dtype=np.uint16)
    out = np.empty(65536, np.float32)
    lib().orc_f16_to_f32(ctypes.c_void_p(allbits.ctypes.data), ctypes.c_void_p(out.ctypes.data), ctypes.c_int64(65536))
    want = allbits.view(np.float16).astype(np.float32)
    assert np.array_equal(bits(out), bits(want))
    rng = np.random.default_rng(1)
    f = np.concatenate([rng.standard_normal(200000).astype(np.float32) * s for s in (1, 1e-5, 1e-7, 7e4)])
    f = np.concatenate([f, out[np.isfinite(out)], np.float32([65504, 65519.99, 65520, 65536, 1e9, 2.0 ** -25, 2.0 ** -24 * 1.5, 0.0, -0.0, np.inf, -np.inf])])
    f = np.ascontiguousarray(f)
    got = np.empty(f.size, np.uint16)
    lib().orc_f32_to_f16(ctypes.c_void_p(f.ctypes.data), ctypes.c_void_p(got.ctypes.data), ctypes.c_int64(f.size))
    with np.errstate(over="ignore"):
        assert np.array_equal(got, f.astype(np.float16).view(np.uint16))
    lib().orc_f32_to_bf16(ctypes.c_void_p(f.ctypes.data), ctypes.c_void_p(got.ctypes.data), ctypes.c_int64(f.size))
    want = torch.from_numpy(f).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(got, want)


def test_a_nan_narrows_to_the_canonical_quiet_nan():
    """The stated policy for 16-bit results: every float NaN, whatever its sign and payload, narrows to
    0x7fc0 (bf16) / 0x7e00 (f16); infinities keep their sign. torch marks the same positions as NaN but
    its bits differ between builds, so only the positions are compared with it."""
    import ctypes

    from oracle import lib

    nan_bits = np.array([0x7fc00000, 0xffc00000, 0x7f800001, 0xff800001, 0x7fffffff, 0xffffffff, 0x7fa00000, 0xffb12345], np.uint32)
    f = np.ascontiguousarray(np.concatenate([nan_bits.view(np.float32), np.float32([np.inf, -np.inf, 1.0, -0.0])]))
    got = np.empty(f.size, np.uint16)
    lib().orc_f32_to_bf16(ctypes.c_void_p(f.ctypes.data), ctypes.c_void_p(got.ctypes.data), ctypes.c_int64(f.size))
    assert list(got) == [0x7fc0] * 8 + [0x7f80, 0xff80, 0x3f80, 0x8000]
    assert np.array_equal(torch.from_numpy(f).to(torch.bfloat16).isnan().numpy(), got == 0x7fc0)
    lib().orc_f32_to_f16(ctypes.c_void_p(f.ctypes.data), ctypes.c_void_p(got.ctypes.data), ctypes.c_int64(f.size))
    assert list(got) == [0x7e00] * 8 + [0x7c00, 0xfc00, 0x3c00, 0x8000]
    assert np.array_equal(torch.from_numpy(f).to(torch.float16).isnan().numpy(), got == 0x7e00)


def test_cpu_baseline_optimizer_is_the_same_update():
    """The torch-op optimizer that bench.py times as tandem's CPU backend gives the
    oracle's bits when the oracle uses torch's CPU sqrt: p, exp_avg, exp_avg_sq over
    six steps, both lerp branches, with and without weight decay, empty shard."""
    from oracle.cpu_engine import TorchCpuAdamW

    for kw in (dict(lr=3e-4, betas=(0.9, 0.95), eps=1e-8, weight_decay=0.1), dict(lr=1e-2, betas=(0.3, 0.999), eps=1e-6, weight_decay=0.0)):
        timed_one = TorchCpuAdamW(**kw)
        checker = AdamW(**kw, sqrt=lambda v: torch.from_numpy(v).sqrt().numpy())
        gen = torch.Generator().manual_seed(5)
        p = torch.randn(10_007, generator=gen) * 0.02
        pn = p.numpy().copy()
        for step in range(6):
            g = torch.randn(10_007, generator=gen) * 1e-3
            timed_one.update("k", p, g)
            checker.update("k", pn, g.numpy())
            assert np.array_equal(bits(p.numpy()), bits(pn)), f"step {step}"
        assert np.array_equal(bits(timed_one.state["k"]["m"].numpy()), bits(checker.state["k"][1]))
        assert np.array_equal(bits(timed_one.state["k"]["v"].numpy()), bits(checker.state["k"][2]))
        timed_one.update("empty", torch.zeros(0), torch.zeros(0))
        assert timed_one.state["empty"]["t"] == 1.0


def _raw16(t):
    return t.view(torch.int16).numpy().view(np.uint16).copy()


@pytest.mark.parametrize("case", ["main", "other"])
def test_bf16_and_f64_match_the_reference_fixture(case):
    """tests/golden/adamw_dtypes.npz: the reference's ShardedAdamW on bfloat16, float16 and float64 shards (its seven torch
    operations take any floating dtype, tandem/optim.py:28-37), 20 steps with the benchmark's hyper-parameters and
    3 steps of the other branches (beta1 < 0.5, no decay). bfloat16: parameters and both moments bit for bit (fp32
    arithmetic, rounded to bf16 after each operation; torch's fp32 sqrt being 1 ulp off changes a bf16 result about
    once in five million elements). float64: both moments bit for bit; the parameters bit for bit with torch's own
    CPU sqrt substituted, and within 1 ulp of each step's update term with the correctly rounded one (torch's
    vectorised double sqrt is off by one ulp on about 0.7 % of inputs, as its float sqrt is)."""
    from helpers import golden_npz, npz_json

    d = golden_npz("adamw_dtypes.npz")
    h = npz_json(d, "hyper_json")[case]
    kw = dict(lr=h["lr"], betas=tuple(h["betas"]), eps=h["eps"], weight_decay=h["weight_decay"])
    last = h["steps"]
    # bfloat16 and float16. With float16 the benchmark's hyper-parameters break down, for the reference as for anyone: eps = 1e-8
    # rounds to 0 and the second moment underflows, so a good part of the parameters end as infinities and NaNs. Infinities keep
    # their sign and are compared bit for bit; NaNs are compared by position (the stated policy: the canonical NaN here, whatever
    # torch's build stores).
    for kind, nan_above in (("bf16", 0x7f80), ("f16", 0x7c00)):
        o = AdamW(**kw, kind=kind)
        p = d[f"{kind}_p0"].view(np.uint16).copy()

        def same(got, want, what):
            nan = (want & 0x7fff) > nan_above
            assert np.array_equal((got & 0x7fff) > nan_above, nan), (kind, what)
            assert np.array_equal(got[~nan], want[~nan]), (kind, what)
            assert kind == "f16" or not nan.any()
            return int(nan.sum())

        for s in range(last):
            o.update("k", p, np.ascontiguousarray(d[f"{kind}_grads"][s].view(np.uint16)))
            if s == 0:
                for got, key in ((p, "p1"), (o.state["k"][1], "m1"), (o.state["k"][2], "v1")):
                    same(got, d[f"{kind}_{case}_{key}"].view(np.uint16), key)
        nans = [same(got, d[f"{kind}_{case}_{key}"].view(np.uint16), key)
                for got, key in ((p, f"p{last}"), (o.state["k"][1], f"m{last}"), (o.state["k"][2], f"v{last}"))]
        if kind == "f16" and case == "main":
            assert nans[0] > 50 and nans[1] == nans[2] == 0  # the breakdown is the reference's, and it is reproduced
    # float64
    for sqrt in (lambda v: torch.from_numpy(v).sqrt().numpy(), None):
        o = AdamW(**kw, sqrt=sqrt)
        p = d["f64_p0"].copy()
        for s in range(last):
            o.update("k", p, np.ascontiguousarray(d["f64_grads"][s]))
        assert np.array_equal(o.state["k"][1].view(np.uint64), d[f"f64_{case}_m{last}"].view(np.uint64))
        assert np.array_equal(o.state["k"][2].view(np.uint64), d[f"f64_{case}_v{last}"].view(np.uint64))
        want = d[f"f64_{case}_p{last}"]
        if sqrt is not None:
            assert np.array_equal(p.view(np.uint64), want.view(np.uint64))
        else:
            assert np.abs(p - want).max() <= last * 2 * np.spacing(h["lr"])
            assert (p.view(np.uint64) != want.view(np.uint64)).mean() < 0.05


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float64])
def test_bf16_and_f64_match_torch_adamw_on_the_cpu(dtype):
    """torch.optim.AdamW(foreach=False) is what the reference says it reproduces operation for operation
    (tandem/optim.py:1-6) and what its own tests compare with (tests/test_zero.py:46-54): 20 steps on a shard of
    20,001 elements, parameters and moments bit for bit (float64 with torch's sqrt substituted)."""
    # (float16 with an eps it can hold and gradients whose squares it can hold: the case where the numbers mean something)
    kw = dict(lr=3e-4, betas=(0.9, 0.95), eps=1e-8 if dtype != torch.float16 else 1e-4, weight_decay=0.1)
    n = 20_001
    g = torch.Generator().manual_seed(3)
    p0 = (torch.randn(n, generator=g, dtype=torch.float64) * 0.02).to(dtype)
    pt = torch.nn.Parameter(p0.clone())
    opt = torch.optim.AdamW([pt], foreach=False, **kw)
    if dtype != torch.float64:
        raw = _raw16
        o = AdamW(**kw, kind="bf16" if dtype == torch.bfloat16 else "f16")
    else:
        raw = lambda t: t.detach().numpy().copy()
        o = AdamW(**kw, sqrt=lambda v: torch.from_numpy(v).sqrt().numpy())
    pn = raw(p0)
    for s in range(20):
        gr = (torch.randn(n, generator=g, dtype=torch.float64) * (1e-3 if dtype != torch.float16 else 3e-2)).to(dtype)
        pt.grad = gr.clone()
        opt.step()
        o.update("k", pn, raw(gr))
    st = opt.state[pt]
    assert np.isfinite(pt.detach().double().numpy()).all()
    assert np.array_equal(bits(pn), bits(raw(pt.detach())))
    assert np.array_equal(bits(o.state["k"][1]), bits(raw(st["exp_avg"])))
    assert np.array_equal(bits(o.state["k"][2]), bits(raw(st["exp_avg_sq"])))


def _to_bf16_bits(x):
    """float32 array -> bfloat16 bit patterns, nearest even (finite inputs)."""
    u = x.view(np.uint32).astype(np.uint64)
    return ((u + 0x7fff + ((u >> 16) & 1)) >> 16).astype(np.uint16)


def test_sqrt_of_a_bfloat16_stays_clear_of_rounding_ties():
    """What lets the bfloat16 kernel (tandem_amd/csrc/kernels_device.h, AdamwMath16::root_over) take a square root that is
    only within 1 ulp of fp32: for every positive bfloat16 in the range of normal floats the exact root lies tens of fp32
    ulps away from every value half way between two bfloat16 neighbours, so any float within a few ulps of it rounds
    to the same bfloat16 as the correctly rounded one."""
    v = (np.arange(0x0080, 0x7f80, dtype=np.uint32) << 16).view(np.float32).astype(np.float64)
    root = np.sqrt(v)  # within 2^-53 of exact
    f = root.astype(np.float32)
    ulp = np.spacing(np.abs(f)).astype(np.float64)
    below = ((f.view(np.uint32) & 0xffff0000) | 0x8000).view(np.float32).astype(np.float64)  # the tie inside this bf16 step
    steps = np.abs(root - below) / ulp
    assert steps.min() > 30
    for shift in (-3, -2, -1, 1, 2, 3):
        near = (f.view(np.uint32).astype(np.int64) + shift).astype(np.uint32).view(np.float32)
        assert np.array_equal(_to_bf16_bits(near), _to_bf16_bits(f))


def test_product_with_the_reciprocal_rounds_like_the_division_away_from_ties():
    """The other half of that shortcut: d * fl(1 / c) lies within two fp32 steps of fl(d / c) for every bfloat16 d that
    a square root can be and c in [2^-30, 2^30], so the two round to different bfloat16 only when the product's low 16
    bits are within a few steps of 0x8000: where the kernel's window (6 on either side) sends the element to the division."""
    d = (np.arange(0x1f80, 0x5f81, dtype=np.uint32) << 16).view(np.float32)  # 2^-64 .. 2^64: the roots of all normal bf16
    rng = np.random.default_rng(12)
    cs = [np.sqrt(1 - b ** t) for b in (0.95, 0.999, 0.98, 0.9) for t in range(1, 60)]
    cs += list(np.exp2(rng.uniform(-30, 30, 300))) + [2.0 ** -30, 2.0 ** 30, 1.0, 1 - 2.0 ** -24, 1 + 2.0 ** -23]
    worst = 0
    for c in cs:
        c = np.float32(c)
        inv = np.float32(1.0 / np.float64(c))
        q, r = d * inv, d / c
        away = np.abs(q.view(np.uint32).astype(np.int64) - r.view(np.uint32).astype(np.int64))
        worst = max(worst, int(away.max()))
        differ = _to_bf16_bits(q) != _to_bf16_bits(r)
        low = (q.view(np.uint32) & 0xffff).astype(np.int64)
        assert np.all(np.abs(low[differ] - 0x8000) <= 2), float(c)
    assert worst <= 2
