"""aicomp_paged_decode_attn_append_static: the decode step for callers that cannot allocate.

Called through the C ABI (ctypes, raw device pointers) and compared bit for bit, output and
pools, with aicomp_paged_decode_attn_append on a workspace of the caller's: two calls in a row
on the same GPU, the second with a smaller batch and shorter contexts, so that the second call
runs over whatever the first left in the library's scratch array.
"""
import math

import pytest
import torch

from aicomp_amd import _lib

pytestmark = pytest.mark.gpu

STATIC_SCRATCH_BYTES = 32 << 20


def _case(device, seed, B, hq, hkv, d, ctx_lo, ctx_hi, kv_dtype):
    g = torch.Generator().manual_seed(seed)
    ctx = torch.randint(ctx_lo, ctx_hi + 1, (B,), generator=g)          # lengths including the new token
    width = math.ceil(ctx_hi / 16) + 1
    nb = B * width + 5
    table = torch.randperm(nb, generator=g)[: B * width].reshape(B, width).to(torch.int32)
    k = torch.randn(nb, hkv, 16, d, generator=g) * 0.5
    v = torch.randn(nb, hkv, 16, d, generator=g) * 0.5
    ks = vs = None
    if kv_dtype == torch.float8_e4m3fn:
        ks = torch.full((hkv,), 2.5 / 448, dtype=torch.float32, device=device)
        vs = torch.full((hkv,), 2.5 / 448, dtype=torch.float32, device=device)
        k, v = (k / (2.5 / 448)).clamp(-448, 448), (v / (2.5 / 448)).clamp(-448, 448)
    return dict(B=B, hq=hq, hkv=hkv, d=d, nb=nb, width=width, kv_dtype=kv_dtype,
                table=table.to(device), ctx=ctx.to(torch.int32).to(device),
                k=k.to(kv_dtype).to(device), v=v.to(kv_dtype).to(device), ks=ks, vs=vs,
                q=torch.randn(B, hq, d, generator=g).to(torch.bfloat16).to(device),
                nk=(torch.randn(B, hkv, d, generator=g) * 0.5).to(torch.bfloat16).to(device),
                nv=(torch.randn(B, hkv, d, generator=g) * 0.5).to(torch.bfloat16).to(device))


def _ptr(t):
    return None if t is None else t.data_ptr()


def _run(lib, c, partition_size, static):
    """One fused append + decode call on copies of the case's pools; returns (out, k_pool, v_pool)."""
    k, v = c["k"].clone(), c["v"].clone()
    out = torch.full_like(c["q"], float("nan"))
    kd = _lib.FP8_E4M3 if c["kv_dtype"] == torch.float8_e4m3fn else _lib.BF16
    stream = torch.cuda.current_stream().cuda_stream
    head = (out.data_ptr(), c["q"].data_ptr(), c["nk"].data_ptr(), c["nv"].data_ptr(), c["nk"].stride(0),
            c["nk"].stride(1), k.data_ptr(), v.data_ptr(), c["table"].data_ptr(), c["table"].stride(0),
            c["ctx"].data_ptr(), c["B"], c["hq"], c["hkv"], c["d"], 16, c["width"], c["nb"],
            1.0 / math.sqrt(c["d"]), _lib.BF16, kd, _ptr(c["ks"]), _ptr(c["vs"]), partition_size)
    if static:
        rc = lib.aicomp_paged_decode_attn_append_static(*head, stream)
    else:
        need = lib.aicomp_paged_decode_workspace_bytes(c["B"], c["hq"], c["hkv"], c["d"], 16, c["width"],
                                                       _lib.BF16, kd, partition_size)
        ws = torch.empty(max(need, 16), dtype=torch.uint8, device=out.device)
        rc = lib.aicomp_paged_decode_attn_append(*head, ws.data_ptr(), need, stream)
    _lib.check(rc, lib)
    torch.cuda.synchronize()
    return out, k, v


def _same(a, b):
    return torch.equal(a.view(torch.uint8), b.view(torch.uint8))


@pytest.mark.parametrize("kv_dtype,d,partition_size", [
    (torch.bfloat16, 128, 0),             # balanced schedule: partials and row records in the scratch
    (torch.float8_e4m3fn, 128, 0),
    (torch.bfloat16, 128, 256),           # grid schedule, explicit split
    (torch.bfloat16, 64, 0),              # head_dim 64
])
def test_static_scratch_call_equals_workspace_call_twice_in_a_row(device, kv_dtype, d, partition_size):
    lib = _lib.load()
    big = _case(device, 11, B=24, hq=32, hkv=8, d=d, ctx_lo=300, ctx_hi=2500, kv_dtype=kv_dtype)
    small = _case(device, 12, B=5, hq=32, hkv=8, d=d, ctx_lo=1, ctx_hi=700, kv_dtype=kv_dtype)
    for name, c in (("first call", big), ("second, smaller call", small)):
        print(f"static-scratch decode: {name}, B={c['B']} d={d} kv={kv_dtype} partition={partition_size}", flush=True)
        got = _run(lib, c, partition_size, static=True)
        want = _run(lib, c, partition_size, static=False)
        assert not torch.isnan(got[0].float()).any(), f"{name}: output rows left unwritten"
        assert _same(got[0], want[0]), f"{name}: output differs from the workspace call"
        assert _same(got[1], want[1]) and _same(got[2], want[2]), f"{name}: pools differ from the workspace call"
        # the new rows did reach the pools
        assert not _same(got[1], c["k"]), f"{name}: K pool unchanged"


def test_static_scratch_refuses_shapes_beyond_its_size(device):
    lib = _lib.load()
    # 1024 sequences at 64 / 8 heads need far more than 32 MiB of partials
    need = lib.aicomp_paged_decode_workspace_bytes(1024, 64, 8, 128, 16, 64, _lib.BF16, _lib.BF16, 0)
    assert need > STATIC_SCRATCH_BYTES
    x = torch.zeros(16, dtype=torch.int32, device=device)        # never dereferenced: the size check comes first
    p = x.data_ptr()
    rc = lib.aicomp_paged_decode_attn_append_static(p, p, p, p, 1024, 128, p, p, p, 64, p, 1024, 64, 8, 128, 16,
                                                    64, 4096, 0.1, _lib.BF16, _lib.BF16, None, None, 0, None)
    assert rc == 4 and b"built-in scratch" in lib.aicomp_kv_last_error()
