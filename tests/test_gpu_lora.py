"""tome_lora_merge / apply_weight_update / grpo_pair_logprobs on the GPU against the oracle
(mlx-impl/node.py:102-164).  Bit-exact wherever the rank-r sums are exact in fp32; on random data
the fp32 accumulation order may flip a bf16 rounding of the product, so the bar there is: at most a
bf16 unit in the last place of the DELTA on a vanishing fraction of elements."""
import types

import numpy as np
import pytest
import torch

import tome_amd
from oracle import logprob_oracle as oracle
from tome_amd import weights
from tome_amd.weights import LayerUpdate
from conftest import bf16_bits_of

pytestmark = pytest.mark.gpu
TOL = 2e-3


@pytest.fixture(scope="module")
def dev():
    return torch.device("cuda:0")


def to_dev(bits, dev):
    return torch.from_numpy(bits.view(np.int16).copy()).to(dev).view(torch.bfloat16)


def exact_bits(rng, shape, denom=16, lim=8):
    """bf16 values k / denom with small integer k: products and rank-long sums are exact in fp32."""
    return oracle.bf16_round((rng.integers(-lim, lim + 1, size=shape) / denom).astype(np.float32))


def rand_bits(rng, shape, scale):
    return oracle.bf16_round((rng.standard_normal(shape) * scale).astype(np.float32))


@pytest.mark.parametrize("rows,cols,rank,scale", [
    (16, 512, 8, 2.5), (37, 1048, 16, 2.5), (4096, 1024, 8, 2.51), (300, 3072, 32, 0.5), (129, 520, 64, -1.25),
    (64, 1024, 128, 0.0625), (50, 264, 24, 3.0), (1, 8, 8, 1.0), (1000, 2560, 40, 2.5), (33, 1536, 96, 1.0)])
def test_merge_bit_exact_on_exact_sums(dev, rows, cols, rank, scale):
    rng = np.random.default_rng(rows * 7 + cols + rank)
    base = rand_bits(rng, (rows, cols), 0.05)
    a, b = exact_bits(rng, (rank, cols)), exact_bits(rng, (rows, rank))
    out = torch.full((rows, cols), 7.0, device=dev, dtype=torch.bfloat16)
    weights.lora_merge([(to_dev(base, dev), out, to_dev(a, dev), to_dev(b, dev), scale)])
    np.testing.assert_array_equal(bf16_bits_of(out), oracle.lora_merge_bf16(base, a, b, scale))


def test_merge_strides_in_place_copy_and_many_jobs(dev):
    rng = np.random.default_rng(11)
    jobs, want, outs = [], [], []
    for i in range(117):                                   # more jobs than one upload launch carries (56)
        rows, cols, rank = int(rng.integers(1, 90)), 8 * int(rng.integers(1, 140)), int(rng.choice([8, 16, 32, 64, 72]))
        base = rand_bits(rng, (rows, cols), 0.05)
        a, b = exact_bits(rng, (rank, cols)), exact_bits(rng, (rows, rank))
        scale = float(rng.choice([2.5, 1.0, 0.75]))
        bt = torch.zeros((rows, cols + 8 * (i % 3)), device=dev, dtype=torch.bfloat16)     # padded row stride
        bt[:, :cols] = to_dev(base, dev)
        if i % 4 == 0:                                     # in place
            ot = bt
        else:
            ot = torch.full((rows, cols + 16), -3.0, device=dev, dtype=torch.bfloat16)
        if i % 5 == 1:                                     # zeros_like delta: the base comes back
            jobs.append((bt[:, :cols], ot[:, :cols], None, None, 1.0))
            want.append(base)
        else:
            jobs.append((bt[:, :cols], ot[:, :cols], to_dev(a, dev), to_dev(b, dev), scale))
            want.append(oracle.lora_merge_bf16(base, a, b, scale))
        outs.append((ot, cols))
    weights.lora_merge(jobs)
    for i, ((ot, cols), w) in enumerate(zip(outs, want)):
        np.testing.assert_array_equal(bf16_bits_of(ot[:, :cols]), w, err_msg=f"job {i}")
        if ot.shape[1] == cols + 16 and i % 4 != 0:
            assert (ot[:, cols:].float() == -3.0).all(), f"job {i} wrote past its columns"


def test_merge_random_data_within_one_delta_ulp(dev):
    rng = np.random.default_rng(12)
    rows, cols, rank, scale = 2048, 1024, 16, 2.5
    base = rand_bits(rng, (rows, cols), 0.02)
    a, b = rand_bits(rng, (rank, cols), 0.05), rand_bits(rng, (rows, rank), 0.05)
    out = torch.empty((rows, cols), device=dev, dtype=torch.bfloat16)
    weights.lora_merge([(to_dev(base, dev), out, to_dev(a, dev), to_dev(b, dev), scale)])
    got, want = bf16_bits_of(out), oracle.lora_merge_bf16(base, a, b, scale)
    differ = got != want
    assert differ.mean() < 1e-4, f"{differ.sum()} of {differ.size} elements differ"
    exact = oracle.lora_merge64(base, a, b, scale)
    err = np.abs(oracle.to_f64(got) - exact)
    # never worse than the three roundings allow: half a unit of the result plus a unit of the delta
    bound = 2.0 ** -8 * np.abs(exact) + 2.0 ** -6 * np.abs(exact - oracle.to_f64(base)) + 1e-30
    assert (err <= bound).all()


def toy(rng, dev, n_layers, nh, nkv, hd, hid, inter):
    qkv = (nh + 2 * nkv) * hd
    model = [{"self_attn.qkv_proj": rand_bits(rng, (qkv, hid), 0.05), "mlp.gate_up_proj": rand_bits(rng, (2 * inter, hid), 0.05),
              "mlp.down_proj": rand_bits(rng, (hid, inter), 0.05)} for _ in range(n_layers)]
    mods = [types.SimpleNamespace(
        self_attn=types.SimpleNamespace(qkv_proj=types.SimpleNamespace(weight=to_dev(l["self_attn.qkv_proj"], dev)), num_heads=nh),
        mlp=types.SimpleNamespace(gate_up_proj=types.SimpleNamespace(weight=to_dev(l["mlp.gate_up_proj"], dev)),
                                  down_proj=types.SimpleNamespace(weight=to_dev(l["mlp.down_proj"], dev)))) for l in model]
    return model, mods


def test_update_weights_end_to_end(dev):
    """The UpdateWeights mirror on a small Qwen3-shaped stack: q/k/v slices, whole matrices, rank 4 (padded on the
    host), two requests in a row (non-cumulative), and the servicer's version counter."""
    rng = np.random.default_rng(13)
    nh, nkv, hd, hid, inter, L = 8, 4, 64, 512, 1536, 3
    ref, ref_m = toy(rng, dev, L, nh, nkv, hd, hid, inter)
    pol = [{k: v.copy() for k, v in l.items()} for l in ref]
    pol_m = [types.SimpleNamespace(
        self_attn=types.SimpleNamespace(qkv_proj=types.SimpleNamespace(weight=m.self_attn.qkv_proj.weight.clone()), num_heads=nh),
        mlp=types.SimpleNamespace(gate_up_proj=types.SimpleNamespace(weight=m.mlp.gate_up_proj.weight.clone()),
                                  down_proj=types.SimpleNamespace(weight=m.mlp.down_proj.weight.clone()))) for m in ref_m]

    def up(layer, name, out_dim, in_dim, rank, scale):
        a, b = exact_bits(rng, (rank, in_dim)), exact_bits(rng, (out_dim, rank))
        return LayerUpdate(layer, name, a.tobytes(), b.tobytes(), [rank, in_dim], [out_dim, rank], scale)

    first = [up(0, "self_attn.q_proj", nh * hd, hid, 8, 2.5), up(0, "self_attn.v_proj", nkv * hd, hid, 8, 2.5),
             up(1, "self_attn.qkv_proj", (nh + 2 * nkv) * hd, hid, 16, 0.0), up(1, "mlp.gate_up_proj", 2 * inter, hid, 4, 5.0),
             up(2, "mlp.down_proj", hid, inter, 8, 2.5), up(2, "mlp.gate_up_proj", 2 * inter, hid, 8, 2.5)]
    second = [up(0, "self_attn.k_proj", nkv * hd, hid, 8, 2.5), up(2, "mlp.down_proj", hid, inter, 32, 0.5)]
    svc = weights.WeightUpdateServicer(types.SimpleNamespace(layers=pol_m), types.SimpleNamespace(layers=ref_m),
                                       head_dim=hd, num_kv_heads=nkv)
    for k, req in enumerate((first, second)):
        r = svc.update_weights(types.SimpleNamespace(updates=req))
        assert r.success and r.policy_version == k + 1
        oracle.update_weights(pol, ref, req, num_heads=nh, num_kv_heads=nkv, head_dim=hd)
        for li in range(L):
            for name, mod in (("self_attn.qkv_proj", pol_m[li].self_attn.qkv_proj), ("mlp.gate_up_proj", pol_m[li].mlp.gate_up_proj),
                              ("mlp.down_proj", pol_m[li].mlp.down_proj)):
                np.testing.assert_array_equal(bf16_bits_of(mod.weight), pol[li][name], err_msg=f"request {k} layer {li} {name}")
    for li in range(L):                                     # the frozen base is never written
        np.testing.assert_array_equal(bf16_bits_of(ref_m[li].mlp.down_proj.weight), ref[li]["mlp.down_proj"])
    bad = up(0, "mlp.down_proj", hid, inter + 8, 8, 1.0)    # shapes that do not fit the weight
    r = svc.update_weights(types.SimpleNamespace(updates=[bad]))
    assert not r.success and svc.policy_version == 2


def test_merge_rejects_bad_inputs(dev):
    z = lambda *s: torch.zeros(s, device=dev, dtype=torch.bfloat16)
    with pytest.raises(TypeError):
        weights.lora_merge([(z(8, 16).float(), z(8, 16), z(8, 16), z(8, 8), 1.0)])
    with pytest.raises(ValueError):
        weights.lora_merge([(z(8, 16), z(8, 24), z(8, 16), z(8, 8), 1.0)])
    with pytest.raises(ValueError):
        weights.lora_merge([(z(8, 16), z(8, 16), z(8, 24), z(8, 8), 1.0)])
    with pytest.raises(ValueError):
        weights.lora_merge([(z(8, 16), z(8, 16), z(8, 16), None, 1.0)])
    with pytest.raises(RuntimeError):
        weights.lora_merge([(z(8, 16).cpu(), z(8, 16), None, None, 1.0)])
    with pytest.raises(ValueError):                        # rank beyond what the kernel holds in registers
        weights.lora_merge([(z(8, 16), z(8, 16), z(136, 16), z(8, 136), 1.0)])
    weights.lora_merge([])


@pytest.mark.parametrize("n,H", [(333, 512), (48, 1024)])      # the tiled sweep kernel; the small-batch one
@pytest.mark.parametrize("with_norm,shared_w", [(False, True), (True, True), (False, False), (True, False)])
def test_grpo_pair_matches_oracle(dev, with_norm, shared_w, n, H):
    """Policy and reference hidden states through a shared (or separate) lm_head, optionally pre-norm."""
    V = 5000
    rng = np.random.default_rng(21 + with_norm + 2 * shared_w + n)
    hp = rand_bits(rng, (n, H), 1.0)
    hr = oracle.bf16_round(oracle.bf16_to_f32(hp) + (rng.standard_normal((n, H)) * 0.05).astype(np.float32))
    wp = rand_bits(rng, (V, H), 0.05)
    wr = wp if shared_w else oracle.bf16_round(oracle.bf16_to_f32(wp) + (rng.standard_normal((V, H)) * 0.004).astype(np.float32))
    nw = oracle.bf16_round((1.0 + 0.1 * rng.standard_normal(H)).astype(np.float32))
    t = rng.integers(0, V, size=n).astype(np.int32)
    valid = (rng.random(n) < 0.7).astype(np.int32)
    r = tome_amd.grpo_pair_logprobs(to_dev(hp, dev), to_dev(hr, dev), to_dev(wp, dev), torch.from_numpy(t).to(dev), 0.8,
                                    w_ref=None if shared_w else to_dev(wr, dev), row_valid=torch.from_numpy(valid).to(dev),
                                    norm_weight=to_dev(nw, dev) if with_norm else None)
    hp_in = oracle.rms_norm_bf16(hp, nw) if with_norm else hp
    hr_in = oracle.rms_norm_bf16(hr, nw) if with_norm else hr
    pol = oracle.lmhead_stats(hp_in, wp, t, 0.8)
    ref = oracle.lmhead_stats(hr_in, wr, t, 0.8)
    m = valid.astype(bool)
    tol = 2 * TOL if with_norm else TOL                    # a normalised value may round to the neighbouring bf16
    np.testing.assert_allclose(r.lp.cpu().numpy()[m], pol["lp"][m], atol=tol, rtol=0)
    np.testing.assert_allclose(r.ref_lp.cpu().numpy()[m], ref["lp"][m], atol=tol, rtol=0)
    np.testing.assert_allclose(r.entropy.cpu().numpy()[m], pol["entropy"][m], atol=tol, rtol=0)
    np.testing.assert_allclose(r.k3.cpu().numpy()[m], oracle.k3(pol["lp"], ref["lp"])[m], atol=4 * tol, rtol=0)
    for o in r:
        assert (o.cpu().numpy()[~m] == 0).all()
    # the same hidden states for both models and one weight: the pair collapses to k3 = 0
    same = tome_amd.grpo_pair_logprobs(to_dev(hp, dev), to_dev(hp, dev), to_dev(wp, dev), torch.from_numpy(t).to(dev), 0.8,
                                       norm_weight=to_dev(nw, dev) if with_norm else None)
    assert np.abs(same.k3.cpu().numpy()).max() == 0.0
    # and it agrees with the one-hidden entry when only the weights differ
    if not with_norm and not shared_w:
        dual = tome_amd.grpo_dual_logprobs(to_dev(hp, dev), to_dev(wp, dev), to_dev(wr, dev), torch.from_numpy(t).to(dev), 0.8)
        pair = tome_amd.grpo_pair_logprobs(to_dev(hp, dev), to_dev(hp, dev), to_dev(wp, dev), torch.from_numpy(t).to(dev), 0.8,
                                           w_ref=to_dev(wr, dev))
        for x, y in zip(dual, pair):
            np.testing.assert_array_equal(x.cpu().numpy(), y.cpu().numpy())


@pytest.mark.parametrize("name", ["m0", "m1", "m2", "m3"])
def test_merge_matches_golden_vectors(dev, name):
    """The committed vectors (exact rational arithmetic, tests/golden/make_lora_golden.py); ranks 12 and 4 are
    zero-padded by the wrapper."""
    import os
    g = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "lora_golden.npz"))
    base, a, b = g[f"{name}_base"], g[f"{name}_a"], g[f"{name}_b"]
    out = torch.empty(base.shape, device=dev, dtype=torch.bfloat16)
    weights.lora_merge([(to_dev(base, dev), out, to_dev(a, dev), to_dev(b, dev), float(g[f"{name}_scale"]))])
    np.testing.assert_array_equal(bf16_bits_of(out), g[f"{name}_out"])


def test_update_weights_at_qwen3_0_6b_scale(dev):
    """All 84 matrices of a Qwen3-0.6B request in one call (the benchmark's workload), checked by properties that do
    not need the CPU oracle at this size: a torch fp32 restatement with the same three roundings (bit-equal except
    where fp32 summation order flips the product's rounding), base-only jobs returning the base, and a second
    identical call changing nothing (non-cumulative)."""
    g = torch.Generator(device=dev).manual_seed(7)
    shapes = [(4096, 1024), (6144, 1024), (1024, 3072)]
    jobs, bases, outs, loras = [], [], [], []
    for i in range(28 * 3):
        rows, cols = shapes[i % 3]
        base = (torch.randn((rows, cols), device=dev, generator=g) * 0.02).to(torch.bfloat16)
        out = torch.empty_like(base)
        a = (torch.randn((8, cols), device=dev, generator=g) * 0.05).to(torch.bfloat16)
        b = (torch.randn((rows, 8), device=dev, generator=g) * 0.05).to(torch.bfloat16)
        if i % 11 == 5:
            jobs.append((base, out, None, None, 1.0))
            loras.append(None)
        else:
            jobs.append((base, out, a, b, 2.5))
            loras.append((a, b))
        bases.append(base)
        outs.append(out)
    weights.lora_merge(jobs)
    first = [o.clone() for o in outs]
    weights.lora_merge(jobs)
    differ = total = 0
    for base, out, again, lo in zip(bases, outs, first, loras):
        assert torch.equal(out, again)
        if lo is None:
            assert torch.equal(out.view(torch.int16), (base.float() + 0.0).to(torch.bfloat16).view(torch.int16))
            continue
        a, b = lo
        d = (b.float() @ a.float()).to(torch.bfloat16).float()
        want = (base.float() + (2.5 * d).to(torch.bfloat16).float()).to(torch.bfloat16)
        ne = out.view(torch.int16) != want.view(torch.int16)
        differ += int(ne.sum())
        total += ne.numel()
        if ne.any():             # one flipped step of the product moves the scaled delta by up to 2^-6 of itself,
            gap = (out.float() - want.float()).abs()[ne]          # the sum then rounds once more
            bound = (2.0 ** -6 * (2.5 * d).abs() + 2.0 ** -7 * want.float().abs())[ne]
            assert (gap <= bound).all()
    assert differ <= total * 1e-4, f"{differ} of {total} elements differ from the torch restatement"
