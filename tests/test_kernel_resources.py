"""Register and scratch budget of the tuned kernels, read from the metadata of the device code inside the built
library (no GPU needed): a kernel that starts to spill into scratch memory inside its tile loop loses tens of
percent without failing any parity test, so the budget is pinned here.  The code objects are taken out of the
library's .hip_fatbin section with the ROCm LLVM tools (one offload bundle per translation unit)."""
import os
import re
import shutil
import subprocess

import pytest

from dmf_amd import _lib

LLVM = "/opt/rocm/llvm/bin"
TOOLS = [os.path.join(LLVM, t) for t in ("llvm-objcopy", "clang-offload-bundler", "llvm-readelf")]
pytestmark = pytest.mark.skipif(not all(os.path.exists(t) for t in TOOLS), reason="ROCm LLVM tools not installed")
MAGIC = b"__CLANG_OFFLOAD_BUNDLE__"


@pytest.fixture(scope="module")
def kernels(tmp_path_factory):
    """{mangled kernel name: {vgpr_count, vgpr_spill_count, private_segment_fixed_size, group_segment_fixed_size}}"""
    lib = _lib.LIB_PATH
    if not os.path.exists(lib):
        pytest.skip("library not built")
    tmp = tmp_path_factory.mktemp("codeobj")
    fat = tmp / "fat.bin"
    subprocess.run([TOOLS[0], f"--dump-section=.hip_fatbin={fat}", lib, str(tmp / "discard.so")], check=True)
    data = fat.read_bytes()
    starts = [m.start() for m in re.finditer(re.escape(MAGIC), data)]
    assert starts, "no offload bundle in the library"
    out = {}
    for i, s in enumerate(starts):
        bundle, co = tmp / f"b{i}.bin", tmp / f"co{i}.elf"
        bundle.write_bytes(data[s:starts[i + 1] if i + 1 < len(starts) else len(data)])
        subprocess.run([TOOLS[1], "--type=o", "--targets=hipv4-amdgcn-amd-amdhsa--gfx950", f"--input={bundle}", f"--output={co}",
                        "--unbundle"], check=True)
        notes = subprocess.run([TOOLS[2], "--notes", str(co)], check=True, capture_output=True, text=True).stdout
        for m in re.finditer(r"\.name:\s+(\S+)\n(.*?)\.wavefront_size", notes, re.S):
            fields = dict(re.findall(r"\.(\w+):\s+(\d+)", m.group(2)))
            out[m.group(1)] = {k: int(v) for k, v in fields.items()}
    shutil.rmtree(tmp, ignore_errors=True)
    return out


def _fwd(D, jvp, nw, qn=False, kn=False):
    b = lambda x: "1" if x else "0"
    return f"_ZN3dmf20attn_fwd_bf16_kernelILi{D}ELb{b(jvp)}ELi{nw}ELb{b(qn)}ELb{b(kn)}EEEvNS_9FwdParamsE"


def test_every_tuned_kernel_is_in_the_library(kernels):
    for D in (64, 72, 80, 96, 128):
        for jvp in (False, True):
            assert _fwd(D, jvp, 8) in kernels and _fwd(D, jvp, 4) in kernels
        assert f"_ZN3dmf23attn_bwd_dq_bf16_kernelILi{D}ELi2EEEvNS_9BwdParamsE" in kernels
        assert f"_ZN3dmf24attn_bwd_dkv_bf16_kernelILi{D}ELi4EEEvNS_9BwdParamsE" in kernels
    for D in (64, 72, 80, 96):
        assert f"_ZN3dmf26attn_bwd_fused_bf16_kernelILi{D}EEEvNS_9BwdParamsE" in kernels


@pytest.mark.parametrize("D", [64, 72, 80])
def test_model_head_dims_do_not_spill(kernels, D):
    """Head dims 64 and 72 are the model's (DMFT-B/2, -XL/2), 80 shares their code shape: no vector register of any
    tuned forward or backward kernel goes to scratch memory, with or without the in-kernel q / k norm."""
    names = [n for n in kernels if re.search(rf"attn_(fwd|bwd_dq|bwd_dkv|bwd_fused)_bf16_kernelILi{D}E", n)]
    assert len(names) >= 8
    for n in names:
        assert kernels[n]["vgpr_spill_count"] == 0, (n, kernels[n])


def test_benchmark_kernels_fit_two_waves_per_simd_without_scratch(kernels):
    """The six kernels the bench line reports (head dim 72): at most 256 VGPRs (two waves per SIMD for the 8-wave
    work-groups), no spills, no private segment."""
    names = [_fwd(72, True, 8), _fwd(72, False, 8), "_ZN3dmf23attn_bwd_dq_bf16_kernelILi72ELi2EEEvNS_9BwdParamsE",
             "_ZN3dmf24attn_bwd_dkv_bf16_kernelILi72ELi4EEEvNS_9BwdParamsE", "_ZN3dmf26attn_bwd_fused_bf16_kernelILi72EEEvNS_9BwdParamsE"]
    for n in names:
        k = kernels[n]
        assert k["vgpr_count"] <= 256 and k["vgpr_spill_count"] == 0 and k["private_segment_fixed_size"] == 0, (n, k)
    assert kernels[_fwd(72, False, 8)]["vgpr_count"] <= 128    # primal forward: four waves per SIMD


def test_head_dim_128_forward_jvp_keeps_its_operands_out_of_scratch(kernels):
    """Head dim 128 with tangents parks its last Q / dQ operand chunks in LDS instead of spilling (8-wave work-groups)."""
    k = kernels[_fwd(128, True, 8)]
    assert k["vgpr_spill_count"] == 0 and k["private_segment_fixed_size"] == 0, k


def test_lds_budgets(kernels):
    """Static LDS is not used by the tuned kernels (their tiles are dynamic LDS, opted in per launch) and nothing
    declares more than the 160 KB of a CU."""
    for n, k in kernels.items():
        assert k.get("group_segment_fixed_size", 0) <= 160 * 1024, (n, k)
