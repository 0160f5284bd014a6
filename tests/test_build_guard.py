"""The build refuses a kernel with a hand-counted load pipeline that spills or uses scratch memory
(ksanallm_amd/build.py: check_resources reads the compiler's kernel-resource-usage remarks)."""
import pytest

from ksanallm_amd import build as kbuild

REMARK = "csrc/x.h:9:1: remark:     %s: %d [-Rpass-analysis=kernel-resource-usage]"


def remarks(name, vgprs=200, scratch=0, sgpr_spill=0, vgpr_spill=0, lds=0):
    rows = [("TotalSGPRs", 60), ("VGPRs", vgprs), ("AGPRs", 0), ("ScratchSize [bytes/lane]", scratch),
            ("Occupancy [waves/SIMD]", 2), ("SGPRs Spill", sgpr_spill), ("VGPRs Spill", vgpr_spill),
            ("LDS Size [bytes/block]", lds)]
    head = "csrc/x.h:9:1: remark: Function Name: %s [-Rpass-analysis=kernel-resource-usage]" % name
    quoted = ["    9 | __global__ void k(P p) {", "      | ^"]
    return "\n".join([head] + quoted + [REMARK % r for r in rows])


def test_clean_kernels_pass_and_are_parsed():
    text = remarks("_ZN3ksq15fp8_tile_kernelINS_4BF16ELb0ELi8EEEvNS_13Fp8TileParamsE", vgprs=220) + "\n" + \
        remarks("_ZN3ksq12other_kernelEv", vgprs=40, scratch=64, vgpr_spill=3)      # not a guarded family
    table = kbuild.check_resources(text)
    assert table["_ZN3ksq15fp8_tile_kernelINS_4BF16ELb0ELi8EEEvNS_13Fp8TileParamsE"]["vgprs"] == 220
    assert table["_ZN3ksq12other_kernelEv"]["scratch"] == 64


@pytest.mark.parametrize("kw", [dict(vgpr_spill=6, scratch=28), dict(scratch=528), dict(lds=170 * 1024)])
@pytest.mark.parametrize("name", ["_ZN3ksq17w4a16_tile_kernelINS_3F16ELi16ELb0ELb0ELi128EEEvNS_10TileParamsE",
                                  "_ZN3ksq19w4a16_splitk_kernelINS_4BF16ELi2ELi8ELi4ELi2ELi2ELi128ELb1ELb0ELi0ELi32EEEvNS_12SplitKParamsE"])
def test_spills_scratch_and_oversized_lds_fail_the_build(name, kw):
    with pytest.raises(RuntimeError) as e:
        kbuild.check_resources(remarks(name, **kw), "x.hip")
    assert name in str(e.value)


def test_scalar_spills_alone_are_tolerated():
    kbuild.check_resources(remarks("_ZN3ksq17w4a16_tile_kernelINS_3F16ELi8ELb1ELb0ELi64EEEvNS_10TileParamsE", sgpr_spill=12))
