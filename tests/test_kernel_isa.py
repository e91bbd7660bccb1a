"""Static checks on the generated gfx950 code of the matrix-core mat-vec kernels (no GPU needed: hipcc cross-compiles).

The kernels' speed hangs on two properties that a source change can lose without any test failing:
  * the write that parks a register set in LDS must wait only for that set (s_waitcnt vmcnt(N) with N = the loads
    requested since), never for every outstanding load: vmcnt(0) there empties the weight stream in every stage;
  * the variants that are used must not spill registers (a private segment makes every wave set up scratch memory,
    measured at -17 %).
"""
import re
import shutil
import subprocess
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parents[1]
SRC = ROOT / "nntrain_amd" / "csrc" / "gemv_mfma_kernels.hip"
HIPCC = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"


@pytest.fixture(scope="module")
def isa(tmp_path_factory):
    if not Path(HIPCC).exists():
        pytest.skip("hipcc is not installed")
    out = tmp_path_factory.mktemp("isa") / "gemv_mfma.s"
    cmd = [HIPCC, "--offload-arch=gfx950", "-O3", "-std=c++17", "-ffp-contract=off", "-Xclang", "-target-feature", "-Xclang",
           "-packed-fp32-ops", "-S", "--cuda-device-only", "-o", str(out), str(SRC)]
    subprocess.run(cmd, check=True, capture_output=True, cwd=SRC.parent)
    return out.read_text()


def _kernels(isa_text):
    """name -> (lines of the kernel body, metadata dict)"""
    bodies, name = {}, None
    for line in isa_text.split("\n"):
        m = re.match(r"^(_ZN5nnhip\S*matvec_mfma\S*):", line)
        if m:
            name = m.group(1)
            bodies[name] = []
        elif name is not None:
            bodies[name].append(line)
            if "s_endpgm" in line:
                name = None
    meta = {}
    for m in re.finditer(r"\.name:\s+(\S+)\n(?:.*\n)*?\s+\.private_segment_fixed_size:\s+(\d+)(?:.*\n)*?\s+\.vgpr_spill_count:\s+(\d+)", isa_text):
        meta[m.group(1)] = {"private": int(m.group(2)), "vgpr_spills": int(m.group(3))}
    return bodies, meta


def _short(name):
    name = re.sub(r"_ZN5nnhip12_GLOBAL__N_1\d+", "", name)
    return re.sub(r"EEEvNS0_8(Wide|Mfma)ArgsE$", "", name)


# (task, stages per tile or tasks per wave, ...) of the variants the planners pick for the shapes of the benchmark and
# the tests: register form <Task, KC, M, LPW, one register set>, wide form <Task, M, LPW, R, one stage buffer, split>
USED = ["matvec_mfma_kernelINS0_7Q4KTaskELi1ELi2ELi5ELb0", "matvec_mfma_kernelINS0_7Q4KTaskELi2ELi1ELi3ELb0",
        "matvec_mfma_kernelINS0_7Q5KTaskELi2ELi1ELi3ELb0",
        "matvec_mfma_kernelINS0_7Q6KTaskELi2ELi1ELi4ELb0", "matvec_mfma_kernelINS0_7Q4KTaskELi1ELi1ELi3ELb0",
        "matvec_mfma_wide_kernelINS0_7Q4KTaskELi1ELi3ELi1ELb0ELb0", "matvec_mfma_wide_kernelINS0_7Q4KTaskELi1ELi3ELi4ELb0ELb0",
        "matvec_mfma_wide_kernelINS0_7Q5KTaskELi1ELi3ELi1ELb0ELb0", "matvec_mfma_wide_kernelINS0_7Q5KTaskELi1ELi3ELi4ELb0ELb0",
        "matvec_mfma_wide_kernelINS0_7Q6KTaskELi1ELi4ELi1ELb0ELb0", "matvec_mfma_wide_kernelINS0_7Q6KTaskELi1ELi4ELi4ELb0ELb0",
        "matvec_mfma_wide_kernelINS0_8IQ2STaskELi2ELi4ELi1ELb0ELb0", "matvec_mfma_wide_kernelINS0_8IQ2STaskELi1ELi2ELi4ELb0ELb0",
        "matvec_mfma_wide_kernelINS0_8Q8_0TaskELi1ELi5ELi1ELb0ELb0",
        "matvec_mfma_wide_kernelINS0_8Q8_0TaskELi2ELi8ELi1ELb1ELb0",
        "matvec_mfma_wide_kernelINS0_8Q8_0TaskELi1ELi5ELi4ELb0ELb0"]
# With one register set the last parking write of a stage rightly waits for everything: nothing else is on its way.
USED_ONE_SET = ["matvec_mfma_kernelINS0_7Q5KTaskELi1ELi2ELi6ELb1"]
# the split form of the shared pass (rows too long for four sets of planes in LDS)
USED_SPLIT = ["matvec_mfma_wide_kernelINS0_7Q4KTaskELi1ELi3ELi4ELb0ELb1", "matvec_mfma_wide_kernelINS0_7Q5KTaskELi1ELi3ELi4ELb0ELb1",
              "matvec_mfma_wide_kernelINS0_7Q6KTaskELi1ELi4ELi4ELb0ELb1", "matvec_mfma_wide_kernelINS0_8IQ2STaskELi1ELi2ELi4ELb0ELb1",
              "matvec_mfma_wide_kernelINS0_8IQ3STaskELi1ELi2ELi4ELb0ELb1",
              "matvec_mfma_wide_kernelINS0_7Q4KTaskELi1ELi3ELi1ELb0ELb1", "matvec_mfma_wide_kernelINS0_7Q5KTaskELi1ELi3ELi1ELb0ELb1",
              "matvec_mfma_wide_kernelINS0_7Q6KTaskELi1ELi4ELi1ELb0ELb1", "matvec_mfma_wide_kernelINS0_8IQ2STaskELi2ELi4ELi1ELb0ELb1",
              "matvec_mfma_wide_kernelINS0_8IQ3STaskELi2ELi4ELi1ELb0ELb1", "matvec_mfma_wide_kernelINS0_8Q8_0TaskELi1ELi5ELi1ELb0ELb1"]


def test_parking_writes_wait_only_for_their_own_register_set(isa):
    bodies, _ = _kernels(isa)
    by_short = {_short(k): v for k, v in bodies.items()}
    for name in USED + USED_SPLIT:
        assert name in by_short, f"{name} is no longer generated"
        last_wait, parks = None, []
        for line in by_short[name]:
            if "s_waitcnt vmcnt" in line:
                last_wait = int(re.search(r"vmcnt\((\d+)\)", line).group(1))
            elif "ds_write_b128" in line:
                parks.append(last_wait)
                last_wait = None
        waits = [w for w in parks if w is not None]
        assert len(waits) >= 6, (name, parks)                      # prologue and both stages of the loop park a set
        assert all(w > 0 for w in waits), f"{name}: a parking write drains the weight stream {parks}"


def test_variants_in_use_do_not_spill(isa):
    _, meta = _kernels(isa)
    by_short = {_short(k): v for k, v in meta.items()}
    for name in USED + USED_ONE_SET + USED_SPLIT:
        assert name in by_short, f"{name} has no metadata"
        assert by_short[name] == {"private": 0, "vgpr_spills": 0}, (name, by_short[name])
