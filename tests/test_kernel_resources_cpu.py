"""What the compiler makes of the attention kernel, checked without a GPU: hipcc cross-compiles
csrc/verify_attention.hip with the library's own flags and reports every kernel's registers, scratch
memory and LDS (-Rpass-analysis=kernel-resource-usage).  The tile loop of that kernel lives at the
register limit, and a change that looks harmless in the source (an array instead of named
variables, a lambda that takes the accumulators by reference, a run-time block index) has more
than once moved accumulators or the tile ring into scratch memory, which costs the kernel a large
part of its speed and shares the memory counter of the tile loads."""
import os
import re
import shutil
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.join(ROOT, "ml-recurrent-drafter_amd"))
import build_hip  # noqa: E402

pytestmark = pytest.mark.skipif(shutil.which(build_hip.HIPCC) is None and not os.path.exists(build_hip.HIPCC),
                                reason="needs hipcc")


@pytest.fixture(scope="module")
def usage(tmp_path_factory):
    src = os.path.join(build_hip.CSRC, "verify_attention.hip")
    out = tmp_path_factory.mktemp("ru") / "verify_attention.o"
    cmd = [build_hip.HIPCC, "-x", "hip", *build_hip.FLAGS, "-Rpass-analysis=kernel-resource-usage", "-c", src, "-o", str(out)]
    r = subprocess.run(cmd, capture_output=True, text=True)
    assert r.returncode == 0, r.stderr[-2000:]
    kernels, name = {}, None
    for line in r.stderr.splitlines():
        m = re.search(r"remark: (?:Function Name: (\S+)|\s*([A-Za-z ]+?)(?: \[[^\]]*\])?: (\d+))", line)
        if not m:
            continue
        if m.group(1):
            name = m.group(1)
            kernels[name] = {}
        elif name is not None:
            kernels[name][m.group(2).strip()] = int(m.group(3))
    return kernels


def _attention(usage, rope):
    want = "Lb1E" if rope else "Lb0E"
    found = {k: v for k, v in usage.items() if "attn_mfma_kernel" in k and want in k}
    assert len(found) == 4, sorted(usage)  # one instantiation per wave layout
    return found


def test_plain_attention_kernels_keep_everything_in_registers(usage):
    for name, u in _attention(usage, rope=False).items():
        assert u["VGPRs"] <= 256 and u["VGPRs Spill"] == 0, (name, u)
        assert u["ScratchSize"] == 0, (name, u)
        assert u["SGPRs Spill"] == 0, (name, u)
        assert u["LDS Size"] == 93184, (name, u)
        assert u["Occupancy"] == 2, (name, u)


def test_fused_rotation_kernels_stay_out_of_scratch_in_the_loop(usage):
    for name, u in _attention(usage, rope=True).items():
        assert u["VGPRs"] <= 256 and u["VGPRs Spill"] <= 4, (name, u)
        assert u["ScratchSize"] <= 24, (name, u)
        assert u["LDS Size"] == 93184, (name, u)


def test_generic_kernel_is_small(usage):
    generic = {k: v for k, v in usage.items() if "attn_generic_kernel" in k}
    assert generic
    for name, u in generic.items():
        assert u["ScratchSize"] == 0 and u["VGPRs"] <= 128, (name, u)


@pytest.fixture(scope="module")
def assembly(tmp_path_factory):
    src = os.path.join(build_hip.CSRC, "verify_attention.hip")
    out = tmp_path_factory.mktemp("asm") / "verify_attention.s"
    cmd = [build_hip.HIPCC, "-x", "hip", *build_hip.FLAGS, "-S", "--cuda-device-only", src, "-o", str(out)]
    r = subprocess.run(cmd, capture_output=True, text=True)
    assert r.returncode == 0, r.stderr[-2000:]
    kernels, name = {}, None
    for line in out.read_text().splitlines():
        m = re.match(r"^(_Z\S*attn_mfma_kernel\S*):", line)
        if m:
            name = m.group(1)
            kernels[name] = []
        elif name is not None:
            kernels[name].append(line)
            if ".end_amdhsa_kernel" in line:
                name = None
    return kernels


def test_plain_attention_kernels_load_tiles_without_per_load_loops(assembly):
    """The tile loads are buffer loads with the non-temporal hint on a descriptor in scalar registers.
    A descriptor that the compiler takes for a per-lane value is legal but slow: every load is then
    wrapped in a loop over the descriptor's distinct values (one more loop per load)."""
    plain = {k: v for k, v in assembly.items() if "Lb0E" in k}
    assert len(plain) == 4
    for name, lines in plain.items():
        loads = [ln for ln in lines if "buffer_load_dwordx4" in ln]
        assert len(loads) == 24 and all(" nt" in ln for ln in loads), (name, len(loads))
        loops = sum("Loop Header" in ln for ln in lines)
        assert loops <= 4, (name, loops)  # the tile loop, the merge of split rows (two levels)
        # the loop's waits are counted ones: some wait with loads still in flight exists behind the loop header
        header = next(i for i, ln in enumerate(lines) if "Loop Header" in ln)
        assert any(re.search(r"s_waitcnt vmcnt\([1-9]", ln) for ln in lines[header:header + 1200]), name


def test_no_scalar_sign_extension_on_the_way_to_an_address(assembly):
    """A 32-bit half of an address that is widened as a signed number (an `int` OR-ed or added into a
    64-bit value) turns every address with bit 31 set into a wild one; in the scalar code of these
    kernels such a widening shows as s_bfe_i64, which their address arithmetic has no other use for."""
    for name, lines in assembly.items():
        assert not any("s_bfe_i64" in ln for ln in lines), name
