"""The build's check on mla_decode_w4_kernel: its 256 accumulators live under fixed register names that only inline
assembly touches, which is sound only while the compiler uses all 256 accumulation registers for the kernel and
spills nothing.  The check reads the compiler's own resource report; these tests pin the reading of that report."""
from xllm_amd import build

REPORT = """\
paged_decode_mla.hip:1443:1: remark: Function Name: _ZN10xllm_mi35512_GLOBAL__N_120mla_decode_w4_kernelINS_4BF16EEEvNS0_7MlaArgsE [-Rpass-analysis=kernel-resource-usage]
 1443 | __global__ __launch_bounds__(kW4Threads) void mla_decode_w4_kernel(MlaArgs a) {
      | ^
paged_decode_mla.hip:1443:1: remark:     TotalSGPRs: 106 [-Rpass-analysis=kernel-resource-usage]
paged_decode_mla.hip:1443:1: remark:     VGPRs: 254 [-Rpass-analysis=kernel-resource-usage]
paged_decode_mla.hip:1443:1: remark:     AGPRs: {agprs} [-Rpass-analysis=kernel-resource-usage]
paged_decode_mla.hip:1443:1: remark:     ScratchSize [bytes/lane]: {scratch} [-Rpass-analysis=kernel-resource-usage]
paged_decode_mla.hip:1443:1: remark:     Dynamic Stack: False [-Rpass-analysis=kernel-resource-usage]
paged_decode_mla.hip:1443:1: remark:     Occupancy [waves/SIMD]: 1 [-Rpass-analysis=kernel-resource-usage]
paged_decode_mla.hip:1443:1: remark:     SGPRs Spill: 62 [-Rpass-analysis=kernel-resource-usage]
paged_decode_mla.hip:1443:1: remark:     VGPRs Spill: {spill} [-Rpass-analysis=kernel-resource-usage]
paged_decode_mla.hip:1443:1: remark:     LDS Size [bytes/block]: 0 [-Rpass-analysis=kernel-resource-usage]
paged_decode_mla.hip:2779:1: remark: Function Name: _ZN10xllm_mi35512_GLOBAL__N_122mla_merge_tiles_kernelINS_4FP16EEEvNS0_7MlaArgsE [-Rpass-analysis=kernel-resource-usage]
paged_decode_mla.hip:2779:1: remark:     VGPRs: 80 [-Rpass-analysis=kernel-resource-usage]
paged_decode_mla.hip:2779:1: remark:     AGPRs: 0 [-Rpass-analysis=kernel-resource-usage]
paged_decode_mla.hip:2779:1: remark:     VGPRs Spill: 0 [-Rpass-analysis=kernel-resource-usage]
"""


def check(**kw):
    fields = dict(agprs=256, scratch=0, spill=0)
    fields.update(kw)
    text = REPORT
    for name, value in fields.items():
        text = text.replace("{" + name + "}", str(value))
    reports = build.resource_report(text, build.GUARDED_KERNEL)
    return reports, build.accumulators_untouched(reports)


def test_a_full_accumulator_file_without_spills_passes():
    reports, (ok, why) = check()
    assert len(reports) == 1 and reports[0]["VGPRs"] == "254"   # (the merge kernel's report is not the guarded one's)
    assert ok, why


def test_anything_else_trips_the_guard():
    assert not check(agprs=252)[1][0]
    assert not check(spill=3)[1][0]
    assert not check(scratch=16)[1][0]
    assert not build.accumulators_untouched([])[0]
