"""The build refuses kernels that keep state in scratch memory: the reader of the compiler's remarks and the rule."""
from sparseattention_amd.build import MAX_SPILLED_VGPRS, kernel_resources, scratch_offenders

REMARKS = """\
In file included from csrc/k.hip:4:
csrc/k.h:62:1: remark: Function Name: _Z6kernelILi0EEv1P [-Rpass-analysis=kernel-resource-usage]
   62 | __global__ __launch_bounds__(256, 2) void kernel(const P p) {
      | ^
csrc/k.h:62:1: remark:     TotalSGPRs: 106 [-Rpass-analysis=kernel-resource-usage]
csrc/k.h:62:1: remark:     VGPRs: 184 [-Rpass-analysis=kernel-resource-usage]
csrc/k.h:62:1: remark:     AGPRs: 0 [-Rpass-analysis=kernel-resource-usage]
csrc/k.h:62:1: remark:     ScratchSize [bytes/lane]: 72 [-Rpass-analysis=kernel-resource-usage]
csrc/k.h:62:1: remark:     Dynamic Stack: False [-Rpass-analysis=kernel-resource-usage]
csrc/k.h:62:1: remark:     Occupancy [waves/SIMD]: 2 [-Rpass-analysis=kernel-resource-usage]
csrc/k.h:62:1: remark:     SGPRs Spill: 11 [-Rpass-analysis=kernel-resource-usage]
csrc/k.h:62:1: remark:     VGPRs Spill: 0 [-Rpass-analysis=kernel-resource-usage]
csrc/k.h:62:1: remark:     LDS Size [bytes/block]: 0 [-Rpass-analysis=kernel-resource-usage]
csrc/k.h:62:1: remark: Function Name: _Z6kernelILi1EEv1P [-Rpass-analysis=kernel-resource-usage]
csrc/k.h:62:1: remark:     VGPRs: 256 [-Rpass-analysis=kernel-resource-usage]
csrc/k.h:62:1: remark:     ScratchSize [bytes/lane]: 36 [-Rpass-analysis=kernel-resource-usage]
csrc/k.h:62:1: remark:     VGPRs Spill: 8 [-Rpass-analysis=kernel-resource-usage]
csrc/k.h:62:1: remark: Function Name: _Z6kernelILi2EEv1P [-Rpass-analysis=kernel-resource-usage]
csrc/k.h:62:1: remark:     VGPRs: 240 [-Rpass-analysis=kernel-resource-usage]
csrc/k.h:62:1: remark:     ScratchSize [bytes/lane]: 0 [-Rpass-analysis=kernel-resource-usage]
csrc/k.h:62:1: remark:     VGPRs Spill: 0 [-Rpass-analysis=kernel-resource-usage]
"""


def test_remarks_are_read_per_kernel():
    res = kernel_resources(REMARKS)
    assert list(res) == ["_Z6kernelILi0EEv1P", "_Z6kernelILi1EEv1P", "_Z6kernelILi2EEv1P"]
    assert res["_Z6kernelILi0EEv1P"] == {"TotalSGPRs": 106, "VGPRs": 184, "AGPRs": 0, "ScratchSize": 72, "DynamicStack": 0,
                                         "Occupancy": 2,
                                         "SGPRsSpill": 11, "VGPRsSpill": 0, "LDSSize": 0}
    assert res["_Z6kernelILi1EEv1P"] == {"VGPRs": 256, "ScratchSize": 36, "VGPRsSpill": 8}
    assert kernel_resources("") == {} and kernel_resources("k.hip:1:1: warning: unused variable 'x'") == {}


def test_arrays_in_scratch_and_heavy_spills_are_refused():
    res = kernel_resources(REMARKS)
    # scratch memory without a spilled register is an array the compiler could not split: refused;
    # a few spilled registers are tolerated; none at all is the normal case
    assert list(scratch_offenders(res)) == ["_Z6kernelILi0EEv1P"]
    res["_Z6kernelILi1EEv1P"]["VGPRsSpill"] = MAX_SPILLED_VGPRS + 1
    assert list(scratch_offenders(res)) == ["_Z6kernelILi0EEv1P", "_Z6kernelILi1EEv1P"]
    assert scratch_offenders({"k": {"VGPRs": 10, "ScratchSize": 0, "DynamicStack": 1}}) == {"k": {"VGPRs": 10, "ScratchSize": 0, "DynamicStack": 1}}
    # registers moved to the other half of the register file (no scratch) are no concern
    assert scratch_offenders({"k": {"VGPRs": 256, "AGPRs": 200, "ScratchSize": 0, "VGPRsSpill": 32}}) == {}
