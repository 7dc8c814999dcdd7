"""The build's guard around the hand-counted copy pipelines (electrock_infer_amd/_build.py): the compiler's
resource remarks are parsed, and a kernel with scratch memory, spilled vector registers or registers beyond a
wave's share fails the build; so does a compiler other than the validated release."""
import pytest

from electrock_infer_amd import _build

REMARKS = """
gemm_tile.hip:74:1: remark: Function Name: _ZN2em12_GLOBAL__N_116gemm_tile_kernelILi1ELb0ELi0ELb1EEEvNS_10MoeProblemEPKiiiiiPi [-Rpass-analysis=kernel-resource-usage]
   74 |                                                                int ntiles_n, int kslice) {
      | ^
gemm_tile.hip:74:1: remark:     TotalSGPRs: 106 [-Rpass-analysis=kernel-resource-usage]
gemm_tile.hip:74:1: remark:     VGPRs: %(vgprs)d [-Rpass-analysis=kernel-resource-usage]
gemm_tile.hip:74:1: remark:     AGPRs: 0 [-Rpass-analysis=kernel-resource-usage]
gemm_tile.hip:74:1: remark:     ScratchSize [bytes/lane]: %(scratch)d [-Rpass-analysis=kernel-resource-usage]
gemm_tile.hip:74:1: remark:     Dynamic Stack: False [-Rpass-analysis=kernel-resource-usage]
gemm_tile.hip:74:1: remark:     Occupancy [waves/SIMD]: 2 [-Rpass-analysis=kernel-resource-usage]
gemm_tile.hip:74:1: remark:     SGPRs Spill: 21 [-Rpass-analysis=kernel-resource-usage]
gemm_tile.hip:74:1: remark:     VGPRs Spill: %(spill)d [-Rpass-analysis=kernel-resource-usage]
gemm_tile.hip:74:1: remark:     LDS Size [bytes/block]: 0 [-Rpass-analysis=kernel-resource-usage]
gemm_tile_mid.hip:330:1: remark: Function Name: _ZN2em12_GLOBAL__N_120gemm_tile_mid_kernelILi1ELi1ELb0EEEvNS_10MoeProblemEPKiiiiii [-Rpass-analysis=kernel-resource-usage]
gemm_tile_mid.hip:330:1: remark:     VGPRs: 104 [-Rpass-analysis=kernel-resource-usage]
gemm_tile_mid.hip:330:1: remark:     AGPRs: 0 [-Rpass-analysis=kernel-resource-usage]
gemm_tile_mid.hip:330:1: remark:     ScratchSize [bytes/lane]: 0 [-Rpass-analysis=kernel-resource-usage]
gemm_tile_mid.hip:330:1: remark:     VGPRs Spill: 0 [-Rpass-analysis=kernel-resource-usage]
gemm_tile_mid.hip:330:1: remark:     LDS Size [bytes/block]: 0 [-Rpass-analysis=kernel-resource-usage]
gemm_stream.hip:47:1: remark: Function Name: _ZN2em12_GLOBAL__N_118gemm_stream_kernelILi1ELb0EEEvNS_10MoeProblemEPKiii [-Rpass-analysis=kernel-resource-usage]
gemm_stream.hip:47:1: remark:     VGPRs: 195 [-Rpass-analysis=kernel-resource-usage]
gemm_stream.hip:47:1: remark:     AGPRs: 0 [-Rpass-analysis=kernel-resource-usage]
gemm_stream.hip:47:1: remark:     ScratchSize [bytes/lane]: 0 [-Rpass-analysis=kernel-resource-usage]
gemm_stream.hip:47:1: remark:     VGPRs Spill: 0 [-Rpass-analysis=kernel-resource-usage]
gemm_stream.hip:47:1: remark:     LDS Size [bytes/block]: 36864 [-Rpass-analysis=kernel-resource-usage]
router.hip:10:1: remark: Function Name: _ZN2em13router_kernelEv [-Rpass-analysis=kernel-resource-usage]
router.hip:10:1: remark:     VGPRs: 20 [-Rpass-analysis=kernel-resource-usage]
router.hip:10:1: remark:     ScratchSize [bytes/lane]: 64 [-Rpass-analysis=kernel-resource-usage]
"""


def report(vgprs=245, scratch=0, spill=0):
    return _build.parse_kernel_resources(REMARKS % {"vgprs": vgprs, "scratch": scratch, "spill": spill})


def test_remarks_are_parsed_per_kernel():
    res = report()
    tile = next(v for k, v in res.items() if "16gemm_tile_kernel" in k)
    assert tile == {"sgprs": 106, "vgprs": 245, "agprs": 0, "scratch": 0, "sgpr_spill": 21, "vgpr_spill": 0, "lds": 0}
    assert len(res) == 4
    checked = _build.check_kernel_resources(res)          # the unguarded router kernel may use scratch
    assert len(checked) == 3


@pytest.mark.parametrize("kw,what", [({"scratch": 132, "spill": 33}, "scratch 132"), ({"spill": 4}, "4 spilled"),
                                     ({"vgprs": 300}, "outside"), ({"vgprs": 64}, "outside")])
def test_guard_rejects_compiler_made_memory_traffic(kw, what):
    with pytest.raises(RuntimeError, match=what):
        _build.check_kernel_resources(report(**kw))


def test_guard_needs_a_report_for_every_guarded_kernel():
    res = {k: v for k, v in report().items() if "gemm_tile_mid" not in k}
    with pytest.raises(RuntimeError, match="no resource report for any gemm_tile_mid_kernel"):
        _build.check_kernel_resources(res)


def test_compiler_release_is_pinned(tmp_path, monkeypatch):
    fake = tmp_path / "hipcc"
    fake.write_text("#!/bin/sh\necho 'HIP version: 9.9.1-abc'\necho 'AMD clang version 30.0.0git (roc-9.9.0)'\n")
    fake.chmod(0o755)
    monkeypatch.delenv("ELECTROCK_ALLOW_ANY_HIPCC", raising=False)
    with pytest.raises(RuntimeError, match="not the validated release"):
        _build.check_compiler(str(fake))
    monkeypatch.setenv("ELECTROCK_ALLOW_ANY_HIPCC", "1")
    assert "9.9.1" in _build.check_compiler(str(fake))
    assert _build.VALIDATED_HIP in _build.check_compiler(_build.hipcc_path())      # the image's own compiler
