"""The C-ABI library loads and exports every function include/aicomp_kv.h declares
(no compute calls: this runs without a GPU)."""
import ctypes
import os
import re

from aicomp_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_functions():
    text = open(os.path.join(ROOT, "include", "aicomp_kv.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(aicomp_\w+)\s*\(", text)))


def test_header_and_binding_agree():
    names = declared_functions()
    assert names, "no declarations found"
    assert sorted(_lib.SYMBOLS) == names


def test_library_exports_every_declared_symbol():
    lib = ctypes.CDLL(_lib.LIB_PATH)
    for name in declared_functions():
        assert hasattr(lib, name), f"{name} missing from {_lib.LIB_PATH}"


def test_host_only_entry_points():
    lib = _lib.load()
    assert lib.aicomp_kv_version() >= 200
    # sizing helpers are pure host arithmetic
    ps = lib.aicomp_paged_decode_partition_size(64, 32, 8, 128, 16, 257, _lib.BF16, _lib.BF16)
    assert ps > 0 and ps % 16 == 0
    need = lib.aicomp_paged_decode_workspace_bytes(64, 32, 8, 128, 16, 257, _lib.BF16, _lib.BF16, 0)
    parts = -(-257 * 16 // ps)
    assert need >= 64 * 32 * parts * (128 + 2) * 4      # partial (output, max, sum) per row, head, partition
    explicit = lib.aicomp_paged_decode_workspace_bytes(64, 32, 8, 128, 16, 257, _lib.BF16, _lib.BF16, ps)
    assert explicit == 64 * 32 * parts * (128 + 2) * 4
    assert lib.aicomp_paged_decode_workspace_bytes(4, 8, 2, 128, 16, 4, _lib.BF16, _lib.BF16, 64) == 0
    # argument validation happens before any device work
    rc = lib.aicomp_paged_decode_attn(None, None, None, None, None, 0, None, 4, 8, 2, 128, 16, 4, 16,
                                      1.0, _lib.BF16, _lib.BF16, None, None, 0, None, 0, None)
    assert rc == 1 and b"null pointer" in lib.aicomp_kv_last_error()
    rc = lib.aicomp_kv_append(None, None, 0, 0, None, None, None, -1, 1, 1, 1, 1, 0, 0, None, None, None)
    assert rc == 1
    assert lib.aicomp_kv_append(None, None, 0, 0, None, None, None, 0, 1, 1, 1, 1, 0, 0, None, None, None) == 0


def test_ops_refuse_cpu_tensors():
    import pytest
    import torch
    from aicomp_amd import ops
    k = torch.zeros(2, 1, 16, 64, dtype=torch.bfloat16)
    x = torch.zeros(1, 1, 64, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError):
        ops.kv_append(x, x, k, k, torch.zeros(1, dtype=torch.int64))


def test_prefill_kernel_waits_for_its_tile_loads_before_the_step_barrier():
    """The direct-to-LDS tile of a step is loaded by all four waves, and the compiler's own waits only
    order a wave's loads against that same wave's later reads; the kernel therefore has to wait for its
    outstanding loads itself right before the barrier that opens the step.  Losing that line gives a wrong
    result once in some hundred runs, which no parity test catches reliably, so the source is checked."""
    src = open(os.path.join(ROOT, "aicomp_amd", "csrc", "prefill_mfma.hip")).read()
    code = re.sub(r"//[^\n]*", "", src)
    step = code[code.index("auto step = "):]
    first_barrier = step.index("__syncthreads()")
    before = re.sub(r"\s+", " ", step[:first_barrier]).strip()
    assert before.endswith("if constexpr (DMA) { __builtin_amdgcn_s_waitcnt(0x0F70);"), before[-200:]


def test_routing_threshold_is_one_word_shared_by_sizing_and_calls():
    """The small-call threshold is process state behind a setter (not an environment lookup per
    call): set returns the previous value, a negative argument only queries, and the sizing helpers
    answer for the value in force."""
    from aicomp_amd import ops
    lib = _lib.load()
    prev = lib.aicomp_kv_set_small_decode_tokens(-1)
    try:
        assert lib.aicomp_kv_set_small_decode_tokens(0) == prev
        assert lib.aicomp_kv_set_small_decode_tokens(-5) == 0
        args = (2, 32, 8, 128, 16, 40, _lib.BF16, _lib.BF16)          # 2 rows x 640 tokens: a small call
        balanced = lib.aicomp_paged_decode_workspace_bytes(*args, 0)
        assert balanced > 0                                            # balanced schedule: always a merge
        assert lib.aicomp_kv_set_small_decode_tokens(32768) == 0
        assert lib.aicomp_paged_decode_workspace_bytes(*args, 0) == 0  # whole rows on the grid schedule
        assert lib.aicomp_paged_decode_partition_size(*args) == 640
        # the Python wrapper bumps an epoch so that prepared calls ask for their size again
        e0 = ops._route_epoch
        assert ops.set_small_decode_tokens(0) == 32768 and ops._route_epoch == e0 + 1
        assert ops.set_small_decode_tokens(0) == 0 and ops._route_epoch == e0 + 1
    finally:
        lib.aicomp_kv_set_small_decode_tokens(prev)


def test_torch_operator_library_registers_the_named_ops():
    """libaicomp_kv_torch.so (built from csrc/torch_ops.cpp) registers the C ABI under
    torch.ops.mi355_kv with the signatures the integration notes give; loading needs no GPU."""
    ns = _lib.torch_ops()
    for name in ("kv_append", "paged_decode_attn", "paged_decode_attn_append", "paged_prefill_attn", "decode_step"):
        assert hasattr(ns, name), name
    s = str(ns.paged_decode_attn.default._schema)
    assert s.startswith("mi355_kv::paged_decode_attn(Tensor(a!) out, Tensor query, Tensor k_pool, Tensor v_pool, "
                        "Tensor block_table, Tensor context_lens, float scale")
    assert "Tensor(a!) k_pool" in str(ns.kv_append.default._schema)
    assert str(ns.decode_step.default._schema).endswith("-> Tensor")
