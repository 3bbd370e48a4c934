"""The GPT and the data loader against digests taken from the reference
(tests/golden/data.json, plans.json): same registration order and shapes, same
seeded initialisation, same batches."""

import hashlib
import math

import torch

from helpers import golden_json
from tandem_amd.data import synthetic
from tandem_amd.model import GPT, Config, count_params


def sha(t):
    return hashlib.sha256(t.detach().contiguous().numpy().tobytes()).hexdigest()


def test_parameter_order_shapes_and_units_match_reference():
    plan = golden_json("plans.json")
    with torch.device("meta"):
        medium = GPT(Config.preset("medium"))
        small = GPT(Config(seq=32, layers=2, heads=2, dim=32))
    assert [[n, list(p.shape)] for n, p in medium.named_parameters()] == plan["medium_params"]
    assert [[n, list(p.shape)] for n, p in small.named_parameters()] == plan["small_params"]
    assert [sum(p.numel() for p in m.parameters()) for m in medium.units()] == plan["medium_units"]
    assert count_params(medium) == 85_842_432 and len(medium.units()) == 14


def test_seeded_init_matches_reference():
    want = golden_json("data.json")
    torch.manual_seed(0)
    model = GPT(Config(seq=32, layers=2, heads=2, dim=32))
    w = torch.cat([p.detach().reshape(-1) for p in model.parameters()])
    assert w.numel() == want["gpt_small_numel"]
    assert w[:8].tolist() == want["gpt_small_seed0_first8"]
    assert sha(w) == want["gpt_small_seed0_sha256"]


def test_synthetic_text_and_batches_match_reference():
    want = golden_json("data.json")
    text = synthetic(20_000)
    assert text.data[:32].tolist() == want["synthetic_first32"]
    assert hashlib.sha256(text.data.to(torch.uint8).numpy().tobytes()).hexdigest() == want["synthetic_20000_sha256"]
    x, y = text.batch(3, 8, 32, rank=1, world=2)
    assert x.tolist() == want["batch_step3_b8_s32_rank1_world2_x"]
    assert sha(y) == want["batch_step3_b8_s32_rank1_world2_y_sha256"]
    # the ranks' rows tile the global batch
    gx, _ = text.batch(3, 8, 32)
    x0, _ = text.batch(3, 8, 32, rank=0, world=2)
    assert torch.equal(torch.cat([x0, x]), gx)


def test_forward_shapes():
    torch.manual_seed(0)
    cfg = Config(seq=16, layers=1, heads=2, dim=16)
    m = GPT(cfg)
    idx = torch.randint(0, 256, (2, 16))
    assert m(idx).shape == (2, 16, 256)
    assert math.isfinite(float(m(idx, idx).detach()))
