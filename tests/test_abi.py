"""CPU-side checks of the C-ABI library: it loads, exports every symbol that
include/electrock_moe.h declares, and validates arguments before any launch
(no compute call is made here — there is no GPU in this environment)."""
import ctypes
import os
import re

import pytest

from electrock_infer_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "electrock_moe.h")


def declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(em_[a-z0-9_]+)\s*\(", text)))


def test_header_and_binding_agree():
    assert declared_symbols() == sorted(_lib.EXPORTED_SYMBOLS)


def test_library_exports_every_declared_symbol():
    lib = _lib.load()
    for name in declared_symbols():
        assert getattr(lib, name) is not None, name
    assert lib.em_version() >= 100
    assert lib.em_error_string(0) == b"success"
    assert b"workspace" in lib.em_error_string(-5)


def test_diagnostic_switches_live_in_their_own_header():
    """Stage masks and kernel-choice switches are for benchmarks and tests: the product header names none of them,
    the binding's values are those of the diagnostic header, and no two flags share a bit."""
    diag = open(os.path.join(ROOT, "include", "electrock_moe_diag.h")).read()
    main = re.sub(r"/\*.*?\*/", "", open(HEADER).read(), flags=re.S)
    flags = {}
    for text in (main, diag):
        for name, bit in re.findall(r"#define\s+EM_FLAG_(\w+)\s+\(1u << (\d+)\)", text):
            assert name not in flags
            flags[name] = 1 << int(bit)
    assert len(set(flags.values())) == len(flags)
    for name in ("SKIP_ROUTER", "SKIP_ALIGN", "SKIP_GEMM1", "SKIP_GEMM2", "SKIP_COMBINE", "FORCE_GENERIC", "NO_PERSIST",
                 "ONE_GROUP_SORT"):
        assert f"EM_FLAG_{name}" not in main and f"EM_FLAG_{name}" in diag
    for name, value in flags.items():
        assert getattr(_lib, f"FLAG_{name}") == value, name


def test_float16_w2_query():
    """Which shapes may keep w2 as float16 at every batch size: those the tuned kernels take."""
    lib = _lib.load()
    assert lib.em_moe_w2_f16_max_tokens(4096, 14336, 8, 2) >= 32768
    assert lib.em_moe_w2_f16_max_tokens(6144, 16384, 8, 2) >= 32768
    assert lib.em_moe_w2_f16_max_tokens(256, 512, 8, 2) >= 32768
    assert lib.em_moe_w2_f16_max_tokens(136, 200, 8, 2) == 0        # only the shape-generic kernels take it
    assert lib.em_moe_w2_f16_max_tokens(4097, 512, 8, 2) == 0       # not a valid shape at all
    # every batch size below the answer really is accepted with the flag: the layout call applies the same plan
    for T in (1, 9, 64, 65, 32768):
        assert lib.em_moe_workspace_bytes(T, 4096, 14336, 8, 2, _lib.FLAG_W2_F16) > 0


def test_signatures_carry_no_torch_types():
    code = re.sub(r"/\*.*?\*/", "", open(HEADER).read(), flags=re.S)   # comments cite reference files
    assert "torch" not in code and "at::" not in code and "#include <hip" not in code


def test_argument_errors_are_reported_before_any_launch():
    lib = _lib.load()
    # shape errors come first, then null pointers; nothing reaches the device
    assert lib.em_topk_softmax(None, 0, 4, 128, 2, 1, None, None, None) == -2     # E > 64
    assert lib.em_topk_softmax(None, 0, 4, 8, 9, 1, None, None, None) == -2       # k > E
    assert lib.em_topk_softmax(None, 7, 4, 8, 2, 1, None, None, None) == -3       # dtype
    assert lib.em_topk_softmax(None, 0, 4, 8, 2, 1, None, None, None) == -1       # null
    assert lib.em_topk_softmax(None, 0, 0, 8, 2, 1, None, None, None) == 0        # empty batch: no-op
    assert lib.em_moe_align_block_size(None, 0, 16, 8, 0, None, 0, None, 0, None, None) == -2
    assert lib.em_moe_align_block_size(None, 5, 16, 8, 16, None, 0, None, 0, None, None) == -3
    assert lib.em_moe_align_block_size(None, 0, 16, 8, 16, None, 136, None, 9, None, None) == -1
    assert lib.em_silu_and_mul(None, None, 4, 8, 9, None) == -3
    assert lib.em_silu_and_mul(None, None, 4, 8, 1, None) == -1
    assert lib.em_silu_and_mul(None, None, 0, 8, 1, None) == 0
    assert lib.em_moe_sum(None, None, 4, 0, 8, 1, None) == -2
    assert lib.em_moe_sum(None, None, 4, 2, 8, 1, None) == -1
    assert lib.em_moe_forward(None, None, 1, None, None, None, 4, 4097, 512, 8, 2, 1, None, 0, 0, None) == -2
    assert lib.em_moe_forward(None, None, 1, None, None, None, 4, 4096, 512, 8, 2, 1, None, 0, 0, None) == -1


def test_workspace_layout_is_consistent():
    lib = _lib.load()
    for T, H, I in [(1, 4096, 14336), (64, 4096, 14336), (256, 4096, 14336), (8192, 4096, 14336),
                    (64, 256, 512), (4096, 6144, 16384)]:
        L = _lib.workspace_layout(T, H, I, 8, 2)
        assert lib.em_moe_workspace_bytes(T, H, I, 8, 2, 0) == L.total_bytes
        assert L.block_size == (16 if T <= 64 else 32)    # 32: the tiled kernel's fragment height
        assert L.sorted_len % L.block_size == 0 and L.sorted_len >= T * 2 + 8 * (L.block_size - 1)
        assert L.expert_ids_len * L.block_size == L.sorted_len
        offs = [L.topk_weights_off, L.topk_ids_off, L.sorted_ids_off, L.expert_ids_off, L.post_pad_off,
                L.seg_begin_off, L.tickets_off, L.saturated_off, L.sort_scratch_off, L.act_off, L.y_off, L.total_bytes]
        assert L.saturated_off == L.tickets_off + 64 and L.saturated_off % 4 == 0
        # one histogram row per 256 ids and one per 1024, of one int32 per expert
        assert L.act_off - L.sort_scratch_off >= -(-T * 2 // 1024) * 5 * 8 * 4
        offs.remove(L.saturated_off)
        assert offs == sorted(offs) and all(o % 256 == 0 for o in offs)
        assert L.act_lo_off == -1                       # the tuned kernels keep no rounding residuals
        assert L.y_off - L.act_off >= L.sorted_len * I * 2
        assert L.total_bytes - L.y_off >= L.ksplit * T * 2 * H * 4
        # the routing results sit at the same offsets whatever the flags; the generic kernels' default form adds act_lo
        G = _lib.workspace_layout(T, H, I, 8, 2, _lib.FLAG_FORCE_GENERIC)
        assert (G.topk_ids_off, G.sorted_ids_off, G.expert_ids_off, G.post_pad_off) == \
               (L.topk_ids_off, L.sorted_ids_off, L.expert_ids_off, L.post_pad_off)
        assert G.act_lo_off - G.act_off >= G.sorted_len * I * 2 and G.y_off - G.act_lo_off >= G.sorted_len * I * 2
        B = _lib.workspace_layout(T, H, I, 8, 2, _lib.FLAG_FORCE_GENERIC | _lib.FLAG_BF16_ACT)
        assert B.act_lo_off == -1 and B.total_bytes < G.total_bytes
    assert lib.em_moe_workspace_bytes(4, 4097, 512, 8, 2, 0) == 0
    assert lib.em_moe_workspace_bytes(4, 4096, 512, 8, 2, 1 << 30) == 0      # unknown flag bit


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", str(tmp_path / "nope.so"))
    with pytest.raises(RuntimeError, match="no fallback"):
        _lib.load()
