"""Argument validation of the C ABI: every refusal below happens on the host, before any device
work, so the pointers are placeholders that are never followed (runs without a GPU)."""
import pytest

from aicomp_amd import _lib

P = 0x10000          # a non-null, 16-byte aligned placeholder
EINVAL, EUNSUPPORTED, EWORKSPACE = 1, 2, 4
F32, BF16, FP8 = _lib.F32, _lib.BF16, _lib.FP8_E4M3


@pytest.fixture(scope="module")
def lib():
    return _lib.load()


def err(lib):
    return lib.aicomp_kv_last_error().decode()


def decode(lib, **kw):
    a = dict(out=P, query=P, k_pool=P, v_pool=P, table=P, table_stride=8, lens=P, batch=4, hq=8, hkv=2, d=128,
             bs=16, max_blocks=8, num_blocks=64, scale=0.1, q_dtype=BF16, kv_dtype=BF16, k_scale=None,
             v_scale=None, partition=0, ws=None, ws_bytes=0, stream=None)
    a.update(kw)
    return lib.aicomp_paged_decode_attn(a["out"], a["query"], a["k_pool"], a["v_pool"], a["table"], a["table_stride"],
                                        a["lens"], a["batch"], a["hq"], a["hkv"], a["d"], a["bs"], a["max_blocks"],
                                        a["num_blocks"], a["scale"], a["q_dtype"], a["kv_dtype"], a["k_scale"],
                                        a["v_scale"], a["partition"], a["ws"], a["ws_bytes"], a["stream"])


def test_decode_refusals(lib):
    assert decode(lib, batch=-1) == EINVAL and "negative batch" in err(lib)
    assert decode(lib, batch=0) == 0                                     # nothing to do
    assert decode(lib, lens=None) == EINVAL and "null pointer" in err(lib)
    assert decode(lib, hq=8, hkv=3) == EINVAL and "not a multiple" in err(lib)
    assert decode(lib, d=0) == EINVAL and "bad sizes" in err(lib)
    assert decode(lib, num_blocks=0) == EINVAL
    assert decode(lib, q_dtype=7) == EINVAL and "unknown element type" in err(lib)
    assert decode(lib, kv_dtype=FP8) == EINVAL and "k_scale and v_scale" in err(lib)
    assert decode(lib, table_stride=7) == EINVAL and "stride" in err(lib)
    assert decode(lib, partition=24) == EINVAL and "multiple of block_size" in err(lib)
    assert decode(lib, partition=-16) == EINVAL
    # the balanced schedule and every split schedule need the caller's scratch
    assert decode(lib) == EWORKSPACE and "workspace" in err(lib)
    assert decode(lib, partition=64) == EWORKSPACE
    need = lib.aicomp_paged_decode_workspace_bytes(4, 8, 2, 128, 16, 8, BF16, BF16, 0)
    assert need > 0
    assert decode(lib, ws=P, ws_bytes=need - 1) == EWORKSPACE and str(need) in err(lib)
    assert decode(lib, ws=P + 4, ws_bytes=need) == EINVAL and "aligned" in err(lib)


def test_decode_append_refusals(lib):
    def call(new_key=P, new_value=P, tstride=256, hstride=128, batch=4):
        return lib.aicomp_paged_decode_attn_append(P, P, new_key, new_value, tstride, hstride, P, P, P, 8, P, batch, 8,
                                                   2, 128, 16, 8, 64, 0.1, BF16, BF16, None, None, 0, None, 0, None)
    assert call(new_key=None) == EINVAL and "new_key" in err(lib)
    assert call(new_value=None) == EINVAL
    assert call(hstride=64) == EINVAL and "new_key / new_value" in err(lib)
    assert call(tstride=-1) == EINVAL
    assert call(batch=0) == 0


def test_append_refusals(lib):
    def call(key=P, slots=P, tokens=3, hkv=2, d=128, bs=16, blocks=8, in_dtype=BF16, pool_dtype=BF16,
             tstride=256, hstride=128):
        return lib.aicomp_kv_append(key, P, tstride, hstride, P, P, slots, tokens, hkv, d, bs, blocks, in_dtype,
                                    pool_dtype, None, None, None)
    assert call(tokens=-1) == EINVAL
    assert call(tokens=0) == 0
    assert call(key=None) == EINVAL and "null pointer" in err(lib)
    assert call(slots=None) == EINVAL
    assert call(hkv=0) == EINVAL and "bad sizes" in err(lib)
    assert call(in_dtype=9) == EINVAL and "unknown element type" in err(lib)
    assert call(hstride=100) == EINVAL and "overlap" in err(lib)


def test_prefill_refusals(lib):
    def call(cu=P, num_seqs=2, total_q=40, max_q=30, hq=8, hkv=2, stride=8, max_blocks=8):
        return lib.aicomp_paged_prefill_attn(P, P, P, P, P, stride, P, cu, num_seqs, total_q, max_q, hq, hkv, 128, 16,
                                             max_blocks, 64, 0.1, BF16, BF16, None, None, None)
    assert call(num_seqs=-1) == EINVAL and "negative" in err(lib)
    assert call(num_seqs=0) == 0 and call(total_q=0) == 0
    assert call(cu=None) == EINVAL and "null pointer" in err(lib)
    assert call(hq=7) == EINVAL
    assert call(max_q=0) == EINVAL and "max_q_len" in err(lib)
    assert call(max_q=41) == EINVAL
    assert call(stride=4) == EINVAL and "stride" in err(lib)


def test_rope_refusals(lib):
    def call(q_in=P, in_dtype=BF16, pool_dtype=BF16, d=128, q_hstride=128, table_stride=128, q_tstride=1024,
             table_rows=64, k_scale=None, tokens=5):
        return lib.aicomp_rope_kv_append(q_in, P, q_tstride, q_hstride, 1024, 128, P, P, 256, 128, P, P, table_stride,
                                         table_rows, None, P, P, P, tokens, 8, 2, d, 16, 64, in_dtype, pool_dtype,
                                         k_scale, None, None)
    assert call(tokens=0) == 0
    assert call(q_in=None) == EINVAL and "null pointer" in err(lib)
    assert call(table_rows=0) == EINVAL
    assert call(in_dtype=FP8) == EUNSUPPORTED and "float32, bfloat16 or float16" in err(lib)
    assert call(pool_dtype=F32) == EUNSUPPORTED                      # bf16 input, fp32 pool
    assert call(pool_dtype=FP8) == EINVAL and "k_scale" in err(lib)
    assert call(d=72) == EUNSUPPORTED and "multiple of 16" in err(lib)
    assert call(q_hstride=64) == EINVAL and "overlap" in err(lib)
    assert call(q_tstride=1028) == EUNSUPPORTED and "16 bytes" in err(lib)
    assert call(q_in=P + 2) == EUNSUPPORTED and "aligned" in err(lib)


def test_sampler_refusals(lib):
    def call(out=P, uniforms=P, batch=2, vocab=100, stride=100, temperature=1.0, top_p=0.9, greedy=0, dtype=F32):
        return lib.aicomp_sample_tokens(out, P, stride, None, uniforms, batch, vocab, temperature, 50, top_p, greedy,
                                        dtype, None)
    assert call(batch=-1) == EINVAL
    assert call(batch=0) == 0
    assert call(out=None) == EINVAL
    assert call(stride=99) == EINVAL and "row stride" in err(lib)
    assert call(dtype=FP8) == EUNSUPPORTED
    assert call(uniforms=None) == EINVAL and "uniforms" in err(lib)
    assert call(temperature=0.0) == EINVAL and "temperature" in err(lib)
    assert call(top_p=float("nan")) == EINVAL and "NaN" in err(lib)
