"""KV append through the C ABI vs the oracle: bit-exact."""
import math

import numpy as np
import pytest
import torch

from aicomp_amd import ops, workloads
from oracle import paged_kv_oracle as orc
from helpers import raw

pytestmark = pytest.mark.gpu


def _bits(t):
    return raw(t)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float8_e4m3fn])
@pytest.mark.parametrize("hkv,d,bs", [(8, 128, 16), (3, 64, 8), (2, 20, 4)])
def test_append_raw_copy_bit_exact(device, dtype, hkv, d, bs):
    torch.manual_seed(0)
    nb, T = 37, 91
    if dtype == torch.float8_e4m3fn:
        mk = lambda *s: torch.randint(0, 256, s, dtype=torch.uint8).view(torch.float8_e4m3fn)
    else:
        mk = lambda *s: torch.randn(*s).to(dtype)
    k_pool, v_pool = mk(nb, hkv, bs, d), mk(nb, hkv, bs, d)
    key, val = mk(T, hkv, d), mk(T, hkv, d)
    slots = torch.randperm(nb * bs)[:T].to(torch.int64)
    slots[5] = -1                                            # padding row
    kp, vp = _bits(k_pool).copy(), _bits(v_pool).copy()
    orc.kv_append(_bits(key), _bits(val), kp, vp, slots.tolist())
    kd, vd = k_pool.to(device), v_pool.to(device)
    ops.kv_append(key.to(device), val.to(device), kd, vd, slots.to(device))
    torch.cuda.synchronize()
    assert np.array_equal(_bits(kd), kp)
    assert np.array_equal(_bits(vd), vp)


def test_append_strided_input_views(device):
    """Rows taken as views of a [B, Hq, n, D] tensor (the adapter's decode call)."""
    torch.manual_seed(1)
    B, hq, g, d, bs, nb = 5, 8, 4, 128, 16, 11
    hkv = hq // g
    k4 = torch.randn(B, hq, 1, d, dtype=torch.bfloat16, device=device)
    v4 = torch.randn(B, hq, 1, d, dtype=torch.bfloat16, device=device)
    key = k4[:, ::g, 0, :]                                   # [B, Hkv, D], strides (Hq*D, g*D, 1)
    val = v4[:, ::g, 0, :]
    assert not key.is_contiguous()
    k_pool = torch.zeros(nb, hkv, bs, d, dtype=torch.bfloat16, device=device)
    v_pool = torch.zeros_like(k_pool)
    slots = torch.tensor([3, 170, 16, 17, 99], dtype=torch.int64, device=device)
    ops.kv_append(key, val, k_pool, v_pool, slots)
    kp = np.zeros((nb, hkv, bs, d), dtype=np.uint16)
    vp = np.zeros_like(kp)
    orc.kv_append(_bits(key), _bits(val), kp, vp, slots.tolist())
    assert np.array_equal(_bits(k_pool), kp) and np.array_equal(_bits(v_pool), vp)


def test_append_empty_and_errors(device):
    k_pool = torch.zeros(4, 2, 16, 64, dtype=torch.bfloat16, device=device)
    v_pool = torch.zeros_like(k_pool)
    e = torch.zeros(0, 2, 64, dtype=torch.bfloat16, device=device)
    ops.kv_append(e, e, k_pool, v_pool, torch.zeros(0, dtype=torch.int64, device=device))
    key = torch.zeros(3, 2, 64, dtype=torch.bfloat16, device=device)
    with pytest.raises(RuntimeError):
        ops.kv_append(key, key, k_pool, v_pool, torch.zeros(2, dtype=torch.int64, device=device))
    with pytest.raises(RuntimeError):
        ops.kv_append(key, key, k_pool, v_pool, torch.zeros(3, dtype=torch.int32, device=device))
    with pytest.raises(RuntimeError):
        ops.kv_append(key[:, :1], key[:, :1], k_pool, v_pool, torch.zeros(3, dtype=torch.int64, device=device))
    with pytest.raises(RuntimeError):
        ops.kv_append(key.float(), key.float(), k_pool, v_pool, torch.zeros(3, dtype=torch.int64, device=device))
    # out-of-pool slots are skipped, never written
    ops.kv_append(key + 1, key + 1, k_pool, v_pool, torch.tensor([64, 10 ** 6, -5], dtype=torch.int64, device=device))
    torch.cuda.synchronize()
    assert float(k_pool.float().abs().sum()) == 0.0


@pytest.mark.parametrize("in_dtype", [torch.bfloat16, torch.float32])
def test_append_fp8_quantise_bit_exact(device, in_dtype):
    torch.manual_seed(2)
    hkv, d, bs, nb, T = 4, 128, 16, 9, 77
    key = (torch.randn(T, hkv, d) * 2).to(in_dtype)
    val = torch.randn(T, hkv, d).to(in_dtype)
    key[0, 0, :4] = torch.tensor([1e4, -1e4, 0.0, 448.0]).to(in_dtype)      # saturation
    ks = torch.from_numpy(orc.absmax_scales(key[1:].float().numpy()))
    vs = torch.from_numpy(orc.absmax_scales(val.float().numpy()))
    slots = torch.randperm(nb * bs)[:T].to(torch.int64)
    kp = np.full((nb, hkv, bs, d), 0x11, dtype=np.uint8)
    vp = np.full((nb, hkv, bs, d), 0x22, dtype=np.uint8)
    name = "bf16" if in_dtype == torch.bfloat16 else "f32"
    orc.kv_append(_bits(key), _bits(val), kp, vp, slots.tolist(), k_scale=ks.numpy(),
                  v_scale=vs.numpy(), pool_dtype="fp8", in_dtype=name)
    kd = torch.full((nb, hkv, bs, d), 0x11, dtype=torch.uint8, device=device).view(torch.float8_e4m3fn)
    vd = torch.full((nb, hkv, bs, d), 0x22, dtype=torch.uint8, device=device).view(torch.float8_e4m3fn)
    ops.kv_append(key.to(device), val.to(device), kd, vd, slots.to(device), ks.to(device), vs.to(device))
    assert np.array_equal(_bits(kd), kp)
    assert np.array_equal(_bits(vd), vp)


def test_append_fp8_all_bf16_values(device):
    """Every finite bf16 value through the device quantiser == torch's e4m3fn cast."""
    codes = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(torch.bfloat16)
    finite = torch.isfinite(codes.float())
    x = codes[finite]
    pad = (-x.numel()) % 128
    x = torch.cat([x, torch.zeros(pad, dtype=torch.bfloat16)]).view(-1, 1, 128)
    T = x.shape[0]
    nb = math.ceil(T / 16)
    kd = torch.zeros(nb, 1, 16, 128, dtype=torch.uint8, device=device).view(torch.float8_e4m3fn)
    vd = torch.zeros_like(kd)
    one = torch.ones(1, device=device)
    ops.kv_append(x.to(device), x.to(device), kd, vd, torch.arange(T, device=device), one, one)
    got = kd.view(torch.uint8).cpu().reshape(-1, 128)[:T].reshape(-1)
    want = x.float().clamp(-448, 448).to(torch.float8_e4m3fn).view(torch.uint8).reshape(-1)
    assert torch.equal(got, want)


def test_append_config_shapes(device):
    """Llama-3-8B decode step (64 rows) and the 2108-row chunked-prefill scatter: every
    row lands bit-exact, every other slot keeps its previous contents."""
    for name in ("llama3_8b_decode", "chunked_prefill_mixed"):
        w = workloads.make_workload(name, device=device, seed=0)
        before_k = w.k_pool.clone()
        before_v = w.v_pool.clone()
        ops.kv_append(w.new_key, w.new_value, w.k_pool, w.v_pool, w.slot_mapping)
        bs = w.shape.block_size
        sm = w.slot_mapping
        assert sm.unique().numel() == sm.numel()
        got_k = w.k_pool[sm // bs, :, sm % bs, :]
        got_v = w.v_pool[sm // bs, :, sm % bs, :]
        assert torch.equal(got_k.view(torch.int16), w.new_key.view(torch.int16))
        assert torch.equal(got_v.view(torch.int16), w.new_value.view(torch.int16))
        # untouched slots
        before_k[sm // bs, :, sm % bs, :] = w.new_key
        before_v[sm // bs, :, sm % bs, :] = w.new_value
        assert torch.equal(before_k.view(torch.int16), w.k_pool.view(torch.int16))
        assert torch.equal(before_v.view(torch.int16), w.v_pool.view(torch.int16))
        if name == "chunked_prefill_mixed":
            assert sm.numel() == 2108
