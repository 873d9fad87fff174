"""Host logic of the UpdateWeights mirror (tome_amd/weights.py) and its oracle restatement
(mlx-impl/node.py:102-164).  CPU only: the merge launch is replaced by the oracle's arithmetic so that
the bookkeeping - which weights become jobs, with which slices, scales and deltas - is what is tested."""
import math
import types

import numpy as np
import pytest
import torch

from oracle import logprob_oracle as oracle
from tome_amd import weights
from tome_amd.weights import LayerUpdate

NUM_HEADS, NUM_KV, HEAD_DIM, HID, INTER = 4, 2, 8, 32, 48
QKV = (NUM_HEADS + 2 * NUM_KV) * HEAD_DIM


def bits(rng, shape, scale=0.1):
    return oracle.bf16_round((rng.standard_normal(shape) * scale).astype(np.float32))


def toy_model(rng, n_layers=2):
    return [{"self_attn.qkv_proj": bits(rng, (QKV, HID)), "mlp.gate_up_proj": bits(rng, (2 * INTER, HID)),
             "mlp.down_proj": bits(rng, (HID, INTER))} for _ in range(n_layers)]


def as_modules(model):
    """dict model -> objects with .self_attn.qkv_proj.weight etc. holding CPU bf16 tensors."""
    t = lambda b: torch.from_numpy(b.view(np.int16).copy()).view(torch.bfloat16)
    return [types.SimpleNamespace(
        self_attn=types.SimpleNamespace(qkv_proj=types.SimpleNamespace(weight=t(l["self_attn.qkv_proj"])), num_heads=NUM_HEADS),
        mlp=types.SimpleNamespace(gate_up_proj=types.SimpleNamespace(weight=t(l["mlp.gate_up_proj"])),
                                  down_proj=types.SimpleNamespace(weight=t(l["mlp.down_proj"])))) for l in model]


def module_bits(layer, name):
    obj = layer
    for part in name.split("."):
        obj = getattr(obj, part)
    return obj.weight.contiguous().view(torch.int16).numpy().view(np.uint16)


def update(rng, layer, name, out_dim, in_dim, rank=8, scale=2.5):
    a, b = bits(rng, (rank, in_dim), 0.3), bits(rng, (out_dim, rank), 0.3)
    return LayerUpdate(layer, name, a.tobytes(), b.tobytes(), [rank, in_dim], [out_dim, rank], scale)


def oracle_merge(jobs):
    """Stand-in for the launch: the oracle's arithmetic, written into the job's output view."""
    tb = lambda t: None if t is None else t.contiguous().view(torch.int16).numpy().view(np.uint16)
    for base, out, a, b, scale in jobs:
        res = oracle.lora_merge_bf16(tb(base), tb(a), tb(b), scale)
        out.copy_(torch.from_numpy(res.view(np.int16).copy()).view(torch.bfloat16))


@pytest.fixture
def patched(monkeypatch):
    monkeypatch.setattr(weights, "lora_merge", oracle_merge)


# ---- the oracle's arithmetic ------------------------------------------------------------------
def test_oracle_merge_closed_forms():
    rng = np.random.default_rng(0)
    base = bits(rng, (24, 40))
    a, b = bits(rng, (8, 40), 0.5), bits(rng, (24, 8), 0.5)
    # zero A or zero B: the base, bit for bit
    z = np.zeros_like(a)
    np.testing.assert_array_equal(oracle.lora_merge_bf16(base, z, b, 2.5), base)
    np.testing.assert_array_equal(oracle.lora_merge_bf16(base, None, None, 1.0), base)
    # rank-1 outer product, brute force with exact sums
    a1, b1 = a[:1], b[:, :1]
    m = oracle.lora_merge64(base, a1, b1, 2.0)
    for i in (0, 7, 23):
        for j in (0, 13, 39):
            want = float(oracle.to_f64(base)[i, j]) + 2.0 * float(oracle.to_f64(b1)[i, 0]) * float(oracle.to_f64(a1)[0, j])
            assert m[i, j] == want
    # B selecting rows of A: delta row i = A[sel[i]]
    sel = rng.integers(0, 8, size=24)
    bsel = np.zeros((24, 8), dtype=np.float32)
    bsel[np.arange(24), sel] = 1.0
    got = oracle.lora_merge64(np.zeros_like(base), a, oracle.bf16_round(bsel), 1.0)
    np.testing.assert_array_equal(got, oracle.to_f64(a)[sel])
    # general entries against math.fsum
    full = oracle.lora_merge64(base, a, b, 2.5)
    a64, b64, base64 = oracle.to_f64(a), oracle.to_f64(b), oracle.to_f64(base)
    for i, j in ((0, 0), (5, 17), (23, 39)):
        want = base64[i, j] + 2.5 * math.fsum(b64[i, k] * a64[k, j] for k in range(8))
        assert abs(full[i, j] - want) <= 1e-15 * max(1.0, abs(want))


def test_oracle_merge_rounding_steps():
    """On inputs whose products and sums are exact, each rounding is visible on its own."""
    one = oracle.bf16_round(np.float32([[1.0]]))
    # d = 1 + 2^-8 is not a bf16 value (8 significand bits): the product rounds to 1.0 (tie to even)
    a = oracle.bf16_round(np.float32([[1.0], [2.0 ** -8]]))          # [rank 2, in 1]
    b = oracle.bf16_round(np.float32([[1.0, 1.0]]))                  # [out 1, rank 2]
    zero = oracle.bf16_round(np.float32([[0.0]]))
    assert oracle.bf16_to_f32(oracle.lora_merge_bf16(zero, a, b, 1.0))[0, 0] == 1.0
    # the scalar is cast to bf16 first: 2.51 -> 2.515625, so 1 * scale gives the bf16 of THAT, 2.515625
    got = oracle.bf16_to_f32(oracle.lora_merge_bf16(zero, one, one, 2.51))[0, 0]
    assert got == 2.515625
    # the final sum rounds once more: 256 + 1 -> 256 (tie to even), 256 + 3 -> 260 (bf16 spacing 2 at 256)
    base = oracle.bf16_round(np.float32([[256.0]]))
    assert oracle.bf16_to_f32(oracle.lora_merge_bf16(base, one, one, 1.0))[0, 0] == 256.0
    assert oracle.bf16_to_f32(oracle.lora_merge_bf16(base, one, one, 3.0))[0, 0] == 260.0
    # and it matches the unrounded closed form to bf16 resolution on random data
    rng = np.random.default_rng(1)
    base, a, b = bits(rng, (64, 96)), bits(rng, (16, 96), 0.2), bits(rng, (64, 16), 0.2)
    exact = oracle.lora_merge64(base, a, b, 2.5)
    got = oracle.to_f64(oracle.lora_merge_bf16(base, a, b, 2.5))
    assert np.abs(got - exact).max() <= 2.0 ** -8 * np.abs(exact).max() + 2.0 ** -7 * np.abs(exact - oracle.to_f64(base)).max()


def test_oracle_bf16_of_f64_is_one_correct_rounding():
    rng = np.random.default_rng(2)
    x = rng.standard_normal(20000) * 10.0 ** rng.integers(-6, 6, 20000)
    got = oracle.bf16_to_f32(oracle._bf16_of_f64(x)).astype(np.float64)
    lo = oracle.bf16_to_f32(oracle._bf16_step(oracle._bf16_of_f64(x), -1)).astype(np.float64)
    hi = oracle.bf16_to_f32(oracle._bf16_step(oracle._bf16_of_f64(x), +1)).astype(np.float64)
    assert (np.abs(got - x) <= np.abs(lo - x)).all() and (np.abs(got - x) <= np.abs(hi - x)).all()
    # a value a hair above a midpoint must round up even though float32 would see the midpoint itself
    mid = 1.0 + 2.0 ** -8
    assert oracle._bf16_of_f64(np.array([mid * (1 + 1e-13)]))[0] == 0x3F81
    assert oracle._bf16_of_f64(np.array([mid]))[0] == 0x3F80           # exact tie: even


# ---- bookkeeping: oracle against hand-derived expectations --------------------------------------
def test_oracle_update_weights_known_answers():
    rng = np.random.default_rng(3)
    ref = toy_model(rng)
    pol = [{k: v.copy() for k, v in l.items()} for l in ref]
    pol[1]["mlp.down_proj"] = bits(rng, (HID, INTER))                  # an earlier LoRA effect on layer 1
    earlier = pol[1]["mlp.down_proj"].copy()
    q = update(rng, 0, "self_attn.q_proj", NUM_HEADS * HEAD_DIM, HID)
    gate1 = update(rng, 0, "mlp.gate_up_proj", 2 * INTER, HID, scale=0.0)           # scale 0 means 1.0
    gate2 = update(rng, 0, "mlp.gate_up_proj", 2 * INTER, HID, rank=16, scale=0.5)  # last update of a param wins
    empty = LayerUpdate(1, "mlp.down_proj", b"", b"", [], [], 1.0)                  # skipped
    other = update(rng, 0, "self_attn.o_proj", HID, HID)                            # not a merged parameter
    n = oracle.update_weights(pol, ref, [q, gate1, gate2, empty, other], num_heads=NUM_HEADS, num_kv_heads=NUM_KV,
                              head_dim=HEAD_DIM)
    assert n == 2
    qs = NUM_HEADS * HEAD_DIM
    A = lambda u: np.frombuffer(u.lora_A, np.uint16).reshape(u.shape_A)
    B = lambda u: np.frombuffer(u.lora_B, np.uint16).reshape(u.shape_B)
    want_q = oracle.lora_merge_bf16(ref[0]["self_attn.qkv_proj"][:qs], A(q), B(q), 2.5)
    np.testing.assert_array_equal(pol[0]["self_attn.qkv_proj"][:qs], want_q)
    np.testing.assert_array_equal(pol[0]["self_attn.qkv_proj"][qs:], ref[0]["self_attn.qkv_proj"][qs:])   # k, v: base
    np.testing.assert_array_equal(pol[0]["mlp.gate_up_proj"], oracle.lora_merge_bf16(ref[0]["mlp.gate_up_proj"], A(gate2), B(gate2), 0.5))
    np.testing.assert_array_equal(pol[0]["mlp.down_proj"], ref[0]["mlp.down_proj"])
    np.testing.assert_array_equal(pol[1]["mlp.down_proj"], earlier)    # untouched layer keeps its earlier state
    # scale 0 -> 1.0
    pol2 = [{k: v.copy() for k, v in l.items()} for l in ref]
    oracle.update_weights(pol2, ref, [gate1], num_heads=NUM_HEADS, num_kv_heads=NUM_KV, head_dim=HEAD_DIM)
    np.testing.assert_array_equal(pol2[0]["mlp.gate_up_proj"], oracle.lora_merge_bf16(ref[0]["mlp.gate_up_proj"], A(gate1), B(gate1), 1.0))
    # non-cumulative: applying the same update twice changes nothing more
    again = [{k: v.copy() for k, v in l.items()} for l in pol2]
    oracle.update_weights(again, ref, [gate1], num_heads=NUM_HEADS, num_kv_heads=NUM_KV, head_dim=HEAD_DIM)
    np.testing.assert_array_equal(again[0]["mlp.gate_up_proj"], pol2[0]["mlp.gate_up_proj"])
    # a whole-qkv delta wins over per-projection ones (node.py:136-139)
    whole = update(rng, 1, "self_attn.qkv_proj", QKV, HID)
    k_only = update(rng, 1, "self_attn.k_proj", NUM_KV * HEAD_DIM, HID)
    pol3 = [{k: v.copy() for k, v in l.items()} for l in ref]
    oracle.update_weights(pol3, ref, [k_only, whole], num_heads=NUM_HEADS, num_kv_heads=NUM_KV, head_dim=HEAD_DIM)
    np.testing.assert_array_equal(pol3[1]["self_attn.qkv_proj"], oracle.lora_merge_bf16(ref[1]["self_attn.qkv_proj"], A(whole), B(whole), 2.5))


# ---- the host mirror against the oracle -----------------------------------------------------
def test_apply_weight_update_matches_oracle(patched):
    rng = np.random.default_rng(4)
    ref = toy_model(rng, 3)
    pol = [{k: bits(rng, v.shape) for k, v in l.items()} for l in ref]   # policy starts somewhere else entirely
    ups = [update(rng, 0, "self_attn.q_proj", NUM_HEADS * HEAD_DIM, HID),
           update(rng, 0, "self_attn.v_proj", NUM_KV * HEAD_DIM, HID, rank=16, scale=0.0),
           update(rng, 2, "self_attn.qkv_proj", QKV, HID),
           update(rng, 2, "self_attn.k_proj", NUM_KV * HEAD_DIM, HID),
           update(rng, 2, "mlp.gate_up_proj", 2 * INTER, HID),
           update(rng, 2, "mlp.gate_up_proj", 2 * INTER, HID, rank=24, scale=0.125),
           update(rng, 0, "mlp.down_proj", HID, INTER),
           LayerUpdate(1, "mlp.down_proj", b"", b"", [], [], 1.0),
           update(rng, 1, "self_attn.o_proj", HID, HID)]
    pol_m, ref_m = as_modules(pol), as_modules(ref)
    n = weights.apply_weight_update(pol_m, ref_m, ups, num_heads=NUM_HEADS, num_kv_heads=NUM_KV, head_dim=HEAD_DIM)
    want_n = oracle.update_weights(pol, ref, ups, num_heads=NUM_HEADS, num_kv_heads=NUM_KV, head_dim=HEAD_DIM)
    assert n == want_n == 4
    for li in range(3):
        for name in ("self_attn.qkv_proj", "mlp.gate_up_proj", "mlp.down_proj"):
            np.testing.assert_array_equal(module_bits(pol_m[li], name), pol[li][name], err_msg=f"layer {li} {name}")
            np.testing.assert_array_equal(module_bits(ref_m[li], name), ref[li][name])      # the base is never written


def test_shared_storage_is_refused(patched):
    rng = np.random.default_rng(5)
    ref_m = as_modules(toy_model(rng, 1))
    with pytest.raises(ValueError, match="share weight storage"):
        weights.apply_weight_update(ref_m, ref_m, [update(rng, 0, "mlp.down_proj", HID, INTER)],
                                    num_heads=NUM_HEADS, num_kv_heads=NUM_KV, head_dim=HEAD_DIM)


def test_servicer_reports_failure_instead_of_raising(patched, monkeypatch):
    rng = np.random.default_rng(6)
    ref = toy_model(rng, 1)
    model = types.SimpleNamespace(layers=as_modules([{k: v.copy() for k, v in ref[0].items()}]))
    refm = types.SimpleNamespace(layers=as_modules(ref))
    cleared = []
    monkeypatch.setattr(torch.cuda, "current_stream", lambda *a, **k: types.SimpleNamespace(synchronize=lambda: None))
    svc = weights.WeightUpdateServicer(model, refm, head_dim=HEAD_DIM, num_kv_heads=NUM_KV, on_update=lambda: cleared.append(1))
    assert svc.num_heads == NUM_HEADS
    ok = svc.update_weights(types.SimpleNamespace(updates=[update(rng, 0, "mlp.down_proj", HID, INTER)]))
    assert ok.success and ok.policy_version == 1 and cleared == [1]
    bad_shape = update(rng, 0, "mlp.down_proj", HID, INTER)
    bad_shape.shape_A = [8, INTER + 1]                                   # bytes do not fit the declared shape
    r = svc.update_weights(types.SimpleNamespace(updates=[bad_shape]))
    assert not r.success and r.policy_version == 0 and svc.policy_version == 1 and cleared == [1]
    r = svc.update_weights(types.SimpleNamespace(updates=[update(rng, 7, "mlp.down_proj", HID, INTER)]))   # no such layer
    assert not r.success
    ok = svc.update_weights(types.SimpleNamespace(updates=[]))             # an empty request still bumps the version
    assert ok.success and ok.policy_version == 2


@pytest.mark.parametrize("name", ["m0", "m1", "m2", "m3"])
def test_oracle_merge_matches_golden_vectors(name):
    """tests/golden/lora_golden.npz: exact rational arithmetic + an independent bf16 rounding (make_lora_golden.py)."""
    import os
    g = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "lora_golden.npz"))
    got = oracle.lora_merge_bf16(g[f"{name}_base"], g[f"{name}_a"], g[f"{name}_b"], float(g[f"{name}_scale"]))
    np.testing.assert_array_equal(got, g[f"{name}_out"])
