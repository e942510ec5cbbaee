"""The builder's guard for kernels that must be compiled without spilled registers."""
import pytest


def test_a_spill_in_a_kernel_that_reads_registers_behind_the_compilers_back_fails_the_build():
    import llama_cu_amd  # noqa: F401
    from llama_cu_amd.kernels import build
    ok = ("x.hip:1:1: remark: Function Name: _Z24attention_prefill_kernelILi128ELb1ELb1EEvPK [-Rpass-analysis=kernel-resource-usage]\n"
          "x.hip:1:1: remark:     VGPRs: 217 [-Rpass-analysis=kernel-resource-usage]\n"
          "x.hip:1:1: remark:     ScratchSize [bytes/lane]: 0 [-Rpass-analysis=kernel-resource-usage]\n"
          "x.hip:1:1: remark: Function Name: _Z23attention_decode_kernelILi128ELb1EEvPK [-Rpass-analysis=kernel-resource-usage]\n"
          "x.hip:1:1: remark:     ScratchSize [bytes/lane]: 24 [-Rpass-analysis=kernel-resource-usage]\n")
    build._check_no_spill("attention_mfma", ok)                       # another kernel's spill is its own business
    with pytest.raises(build.BuildError, match="spilled"):
        build._check_no_spill("attention_mfma", ok.replace("ScratchSize [bytes/lane]: 0", "ScratchSize [bytes/lane]: 52"))
    with pytest.raises(build.BuildError, match="names none"):
        build._check_no_spill("attention_mfma", "no report at all\n")
