"""em_moe_forward_static, the entry point that allocates nothing (its scratch memory is a fixed array inside the
library), against em_moe_forward on a caller-provided workspace: same kernels, same inputs, so the outputs must be
equal bit for bit -- on two calls in a row, the second with a smaller batch (the shared array still holds the first
call's contents), for both output types; and shapes beyond the fixed array are refused before anything is launched."""
import ctypes

import pytest
import torch

from electrock_infer_amd import _lib
from tests.gpu_util import DEV, announce, gpu_inputs

pytestmark = pytest.mark.gpu


def _forward(lib, x, lg, w13, w2, out, flags, ws=None):
    T, H = x.shape
    E, two_i, _ = w13.shape
    stream = torch.cuda.current_stream().cuda_stream
    head = (x.data_ptr(), lg.data_ptr(), _lib.dtype_code(lg.dtype), w13.data_ptr(), w2.data_ptr(), out.data_ptr(),
            T, H, two_i // 2, E, 2, 1)
    if ws is None:
        return lib.em_moe_forward_static(*head, flags, stream)
    return lib.em_moe_forward(*head, ws.data_ptr(), ctypes.c_size_t(ws.numel()), flags, stream)


@pytest.mark.parametrize("H,I", [(512, 1024), (4096, 14336)])
def test_static_entry_point_matches_workspace_entry_point(H, I):
    lib = _lib.load()
    E = 8
    x, lg, w13, w2 = gpu_inputs(64, H, I, E, seed=17)
    for T in (64, 5):                      # the second call is the smaller one
        for flags in (0, _lib.FLAG_OUT_F32, _lib.FLAG_BF16_ACT):
            announce(f"static entry point H={H} I={I} T={T} flags={flags}")
            xt, lt = x[:T].contiguous(), lg[:T].contiguous()
            odt = torch.float32 if flags & _lib.FLAG_OUT_F32 else torch.bfloat16
            need = lib.em_moe_workspace_bytes(T, H, I, E, 2, flags)
            assert 0 < need <= _lib.STATIC_SCRATCH_BYTES
            ws = torch.empty(need, dtype=torch.uint8, device=DEV)
            want = torch.full((T, H), float("nan"), dtype=odt, device=DEV)
            got = torch.full((T, H), float("nan"), dtype=odt, device=DEV)
            assert _forward(lib, xt, lt, w13, w2, want, flags, ws) == 0
            # (the first call on a device looks the array's address up, which is when the runtime places the array)
            assert _forward(lib, xt, lt, w13, w2, got, flags) == 0
            got.fill_(float("nan"))
            torch.cuda.synchronize()
            free_before, held_before = torch.cuda.mem_get_info()[0], torch.cuda.memory_allocated()
            assert _forward(lib, xt, lt, w13, w2, got, flags) == 0
            torch.cuda.synchronize()
            # nothing was taken from the device (the same kernels ran just before, so no code is loaded either)
            assert torch.cuda.mem_get_info()[0] >= free_before and torch.cuda.memory_allocated() == held_before
            assert torch.isfinite(want.float()).all()
            assert torch.equal(got, want)


def test_static_entry_point_with_the_tiled_kernels_and_changing_batch_sizes():
    """A small shape lets batches of hundreds of tokens into the fixed array: the 64- / 128-row kernels and the 256-row
    kernels, whose tile tickets then live in that array and are cleared by the sort in front of them.  Calls of
    changing size in a row (large after small, small after large: the array holds whatever the call before left,
    tickets and the saturation counter included), each against em_moe_forward on a fresh workspace with every
    bit set: equal bit for bit."""
    lib = _lib.load()
    H, I, E = 512, 1024, 8
    x, lg, w13, w2 = gpu_inputs(1024, H, I, E, seed=23)
    w2h = w2.to(torch.float16)
    for T, flags in ((300, 0), (1024, 0), (70, _lib.FLAG_OUT_F32), (1024, _lib.FLAG_W2_F16 | _lib.FLAG_OUT_F32), (5, 0),
                     (600, _lib.FLAG_W2_F16), (1024, _lib.FLAG_BF16_ACT)):
        announce(f"static entry point, tiled kernels: T={T} flags={flags}")
        xt, lt = x[:T].contiguous(), lg[:T].contiguous()
        w2t = w2h if flags & _lib.FLAG_W2_F16 else w2
        odt = torch.float32 if flags & _lib.FLAG_OUT_F32 else torch.bfloat16
        need = lib.em_moe_workspace_bytes(T, H, I, E, 2, flags)
        assert 0 < need <= _lib.STATIC_SCRATCH_BYTES
        ws = torch.full((need,), 0xFF, dtype=torch.uint8, device=DEV)
        want = torch.full((T, H), float("nan"), dtype=odt, device=DEV)
        got = torch.full((T, H), float("nan"), dtype=odt, device=DEV)
        assert _forward(lib, xt, lt, w13, w2t, want, flags, ws) == 0
        assert _forward(lib, xt, lt, w13, w2t, got, flags) == 0
        torch.cuda.synchronize()
        assert torch.isfinite(want.float()).all()
        assert torch.equal(got, want)


def test_static_entry_point_refuses_what_does_not_fit():
    lib = _lib.load()
    announce("static entry point, size limit")
    T, H, I, E = 4096, 512, 1024, 8
    assert lib.em_moe_workspace_bytes(T, H, I, E, 2, 0) > _lib.STATIC_SCRATCH_BYTES
    x, lg, w13, w2 = gpu_inputs(T, H, I, E, seed=3)
    out = torch.zeros(T, H, dtype=torch.bfloat16, device=DEV)
    rc = _forward(lib, x, lg, w13, w2, out, 0)
    torch.cuda.synchronize()
    assert rc == _lib.ERR_STATIC_LIMIT and not out.any()          # nothing was launched
    assert b"EM_STATIC_SCRATCH_BYTES" in lib.em_error_string(rc)
    with pytest.raises(RuntimeError, match="scratch"):
        _lib.check(rc, "em_moe_forward_static")
