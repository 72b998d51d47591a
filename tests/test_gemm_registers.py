"""The grouped GEMM's column-wave kernels keep their weight fragments in registers that the compiler does not know to be in
use (the asynchronous loads and the MFMAs name them in their assembly text).  That is only sound if the compiler itself never
touches those registers and never spills in the item loop (a reload from the stack waits for every copy in flight).  Checked
here on the code the build actually generates: megamoe.hip compiled to assembly with the build's own flags (no GPU needed)."""

import os
import re
import shutil
import subprocess

import pytest

from deepep_amd import build

SOURCE = os.path.join(build.CSRC, "megamoe.hip")


@pytest.fixture(scope="module")
def assembly(tmp_path_factory):
    hipcc = build._hipcc()
    if shutil.which(hipcc) is None and not os.path.exists(hipcc):
        pytest.skip("hipcc is not installed")
    out = tmp_path_factory.mktemp("isa") / "megamoe.s"
    flags = [f for f in build.FLAGS if f != "-fPIC"] + list(build.FILE_FLAGS.get("megamoe.hip", ()))
    proc = subprocess.run([hipcc, *flags, "--cuda-device-only", "-S", "-o", str(out), SOURCE], capture_output=True, text=True)
    assert proc.returncode == 0, proc.stderr[-2000:]
    return out.read_text().split("\n")


def _kernels(lines):
    """name -> (body lines, metadata) of every column-wave kernel."""
    text = "\n".join(lines)
    found = {}
    for match in re.finditer(r"\.amdhsa_kernel (\S*grouped_gemm_colwave_kernel\S*)(.*?)\.end_amdhsa_kernel", text, re.S):
        name, meta = match.group(1), match.group(2)
        start = next(i for i, line in enumerate(lines) if line.startswith(name + ":"))
        end = next(i for i in range(start, len(lines)) if lines[i].strip().startswith(".amdhsa_kernel"))
        scratch = int(re.search(r"\.amdhsa_private_segment_fixed_size\s+(\d+)", meta).group(1))
        found[name] = (lines[start:end], scratch)
    return found


def _numbers(text, file):
    singles = [int(x) for x in re.findall(r"\b" + file + r"(\d+)\b", text)]
    ranges = [int(v, 0) for pair in re.findall(r"\b" + file + r"\[(\w+):(\w+)\]", text) for v in pair]
    return singles + ranges


def test_weight_registers_belong_to_the_assembly_statements_alone(assembly):
    kernels = _kernels(assembly)
    assert len(kernels) == 6  # three tile heights x {first, second} GEMM
    for name, (body, scratch) in kernels.items():
        rows = int(re.search(r"kernelILi(\d)", name).group(1))
        # 64 / 128 rows: a64.. / a128.., right behind the accumulators; 192 rows: v192..v255
        file, first = ("v", 192) if rows == 3 else ("a", 64 * rows)
        in_statement, outside, in_loads, accumulators = False, [], set(), []
        for line in body:
            text = line.strip()
            if text.startswith(";;#ASMSTART"):
                in_statement = True
            elif text.startswith(";;#ASMEND"):
                in_statement = False
            elif in_statement:
                if text.startswith("global_load_dwordx4"):
                    in_loads.update(_numbers(text.split(",")[0], file))
                if text.startswith("v_mfma"):
                    accumulators += _numbers(text.split(",")[0], "a")
            elif any(first <= r < first + 64 for r in _numbers(text, file)):
                outside.append(text)
        assert not outside, f"{name}: the compiler uses weight registers itself: {outside[:3]}"
        assert in_loads and min(in_loads) == first and max(in_loads) == first + 63, (name, sorted(in_loads)[:4])
        assert max(accumulators) == 64 * rows - 1, f"{name}: accumulators reach a{max(accumulators)}"
        assert scratch == 0, f"{name}: {scratch} bytes of stack (a reload in the item loop waits for all copies in flight)"
