"""bench.py's contract at the edges that need no GPU: more than one GPU is refused with one line and exit
code 2, and sampling options belong to the decode-only mode."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _bench(*args):
    return subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), *args], capture_output=True, text=True,
                          timeout=300, cwd=ROOT)


def test_more_than_one_gpu_is_refused_with_one_line():
    p = _bench("--gpus", "2", "--steps", "3", "--warmup", "1")
    assert p.returncode == 2
    lines = [l for l in p.stdout.splitlines() if l.strip()]
    assert len(lines) == 1 and "one GPU" in lines[0]


def test_sampling_options_go_with_the_decode_mode_only():
    p = _bench("--temperature", "0.8")
    assert p.returncode == 2 and "--only decode" in p.stdout


def test_the_build_names_kernels_that_keep_registers_in_memory():
    """What the build reads out of the compiler's remarks: a kernel's name and how many registers it spilled."""
    from denno_beta_amd.build import spilling_kernels
    remarks = "\n".join([
        "gemm.hip:501:1: remark: Function Name: _ZN6skinny11gemm_kernelILi4ELi2EEEvv [-Rpass-analysis=kernel-resource-usage]",
        "gemm.hip:501:1: remark:     VGPRs: 256 [-Rpass-analysis=kernel-resource-usage]",
        "gemm.hip:501:1: remark:     ScratchSize [bytes/lane]: 196 [-Rpass-analysis=kernel-resource-usage]",
        "gemm.hip:501:1: remark:     SGPRs Spill: 0 [-Rpass-analysis=kernel-resource-usage]",
        "gemm.hip:501:1: remark:     VGPRs Spill: 48 [-Rpass-analysis=kernel-resource-usage]",
        "gemm.hip:732:1: remark: Function Name: _ZN6skinny13gemm16_kernelILi8EEEvv [-Rpass-analysis=kernel-resource-usage]",
        "gemm.hip:732:1: remark:     VGPRs: 120 [-Rpass-analysis=kernel-resource-usage]",
        "gemm.hip:732:1: remark:     VGPRs Spill: 0 [-Rpass-analysis=kernel-resource-usage]",
    ])
    assert spilling_kernels(remarks) == [("_ZN6skinny11gemm_kernelILi4ELi2EEEvv", 48)]
    assert spilling_kernels("") == []
