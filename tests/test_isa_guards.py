"""Checks on the gfx950 assembly hipcc generates for the MFMA kernels (no GPU needed: hipcc
cross-compiles).  Two code shapes gave wrong numbers on the device while this library was built,
both silently:

* an MFMA inside an EXEC-masked region.  MFMA instructions ignore EXEC, so a guard that the
  compiler turned into lane predication (because it could not prove the condition wave-uniform,
  e.g. one derived from ``threadIdx.x >> 6``) only holds while the compiler also keeps the
  ``s_cbranch_execz`` around the block; when it dropped one, clamped duplicate weight blocks were
  multiplied in and outputs came out 4x too large.  The kernels now derive such conditions from a
  ``readfirstlane`` wave id, which makes them scalar branches.
* a branch between an MFMA and the VALU instruction that reads its result.  hipcc 7.2 counts the
  required wait states along the fall-through path only; on the taken path the read saw stale
  accumulator values.

Both are properties of the generated code, so they are asserted on the generated code."""
import os
import re
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "ateniaengine_amd", "csrc")
HIPCC = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
FLAGS = ["--offload-arch=gfx950", "-O3", "-fPIC", "-std=c++17", "-w", "-Xclang", "-target-feature",
         "-Xclang", "-packed-fp32-ops", "--cuda-device-only", "-S"]

_EXEC_OPEN = ("s_and_saveexec", "s_andn2_saveexec", "s_or_saveexec", "s_and_b64 exec", "s_xor_b64 exec",
              "s_andn2_b64 exec")
_EXEC_CLOSE = ("s_or_b64 exec", "s_mov_b64 exec", "s_endpgm")


def _assembly(tmp_path_factory, name):
    out = tmp_path_factory.mktemp("isa") / (name + ".s")
    r = subprocess.run([HIPCC] + FLAGS + ["-o", str(out), os.path.join(CSRC, name)],
                       capture_output=True, text=True, timeout=900)
    assert r.returncode == 0, r.stderr[-2000:]
    return [ln.strip() for ln in open(out).read().split("\n")]


def _validated_release():
    """(Makefile, build.rs): the hipcc major.minor the generated code was validated with."""
    mk = open(os.path.join(CSRC, "Makefile")).read()
    rs = open(os.path.join(ROOT, "ffi", "atenia-moe-hip-sys", "build.rs")).read()
    return (re.search(r"^HIPCC_VALIDATED\s*:=\s*(\S+)", mk, flags=re.M).group(1),
            re.search(r'const HIPCC_VALIDATED: &str = "([^"]+)";', rs).group(1))


def test_hipcc_is_the_release_the_generated_code_was_validated_with():
    """The inline-assembly MFMAs of the nine-group tiles carry hand-counted wait states, and the
    checks below were read against one compiler release's assembly.  Another major.minor fails
    here, loudly, until somebody has read the new assembly and moved HIPCC_VALIDATED (Makefile and
    build.rs) on purpose."""
    if not os.path.exists(HIPCC):
        pytest.skip("hipcc not found")
    mk, rs = _validated_release()
    assert mk == rs, f"Makefile says {mk}, build.rs says {rs}"
    out = subprocess.run([HIPCC, "--version"], capture_output=True, text=True, timeout=120).stdout
    m = re.search(r"HIP version: (\d+)\.(\d+)", out)
    assert m, out[:300]
    assert f"{m.group(1)}.{m.group(2)}" == mk, (
        f"hipcc is release {m.group(1)}.{m.group(2)}, the kernels' assembly was validated with {mk}")


@pytest.fixture(scope="module", params=["ffn_stream.hip", "ffn_tiled.hip", "ffn_tiled_duo.hip", "ffn_f32.hip"])
def asm(request, tmp_path_factory):
    if not os.path.exists(HIPCC):
        pytest.skip("hipcc not found")
    return request.param, _assembly(tmp_path_factory, request.param)


def test_no_mfma_under_an_exec_mask(asm):
    name, lines = asm
    # A masked region is the code that follows an instruction narrowing EXEC, up to the
    # instruction restoring it -- or up to the next label that does not sit right behind the
    # opener and its branch: blocks are not laid out in execution order, so anything further
    # down the listing belongs to some other path.
    masked, since_open, hits, total = False, 0, [], 0
    for no, ln in enumerate(lines, 1):
        if not ln or ln.startswith(";"):
            continue
        if ln.startswith(_EXEC_OPEN):
            masked, since_open = True, 0
            continue
        since_open += 1
        if ln.startswith(_EXEC_CLOSE):
            masked = False
        elif ln.startswith(".LBB") and since_open > 2:
            masked = False
        elif ln.startswith("v_mfma"):
            total += 1
            if masked:
                hits.append((no, ln))
    assert total > (30 if name == "ffn_f32.hip" else 100), f"{name}: expected the MFMA kernels in the assembly, found {total} MFMAs"
    assert not hits, f"{name}: MFMA inside an EXEC-masked region (MFMA ignores EXEC): {hits[:5]}"


def _regs(operand):
    m = re.fullmatch(r"([va])\[(\d+):(\d+)\]", operand)
    if m:
        return {(m.group(1), i) for i in range(int(m.group(2)), int(m.group(3)) + 1)}
    m = re.fullmatch(r"([va])(\d+)", operand)
    return {(m.group(1), int(m.group(2)))} if m else set()


def test_no_branch_between_an_mfma_and_the_valu_read_of_its_result(asm):
    """For every branch that directly follows an MFMA: the first instructions at the branch
    target must not be plain VALU / LDS / memory reads of that MFMA's destination registers
    (an MFMA reading it as its own accumulator again is the hardware's back-to-back case)."""
    name, lines = asm
    labels = {ln[:-1]: i for i, ln in enumerate(lines) if ln.endswith(":") and ln.startswith(".LBB")}
    labels.update({ln.split(":")[0]: i for i, ln in enumerate(lines) if ln.startswith(".LBB") and ":" in ln})
    bad = []
    for i, ln in enumerate(lines):
        if not ln.startswith("v_mfma"):
            continue
        dst = _regs(ln.split()[1].rstrip(","))
        for j in range(i + 1, min(i + 3, len(lines))):
            if lines[j].startswith("v_mfma"):
                break
            if lines[j].startswith("s_cbranch") or lines[j].startswith("s_branch"):
                target = labels.get(lines[j].split()[-1])
                if target is None:
                    break
                waited = 0
                for t in lines[target + 1:target + 12]:
                    if not t or t.startswith(";") or t.endswith(":"):
                        continue
                    if t.startswith("s_nop"):
                        waited += int(t.split()[1]) + 1
                    if waited >= 8 or t.startswith(("s_waitcnt", "s_barrier", "s_cbranch", "s_branch")):
                        break
                    ops = [o.strip().rstrip(",") for o in t.replace(",", " ").split()[1:]]
                    reads = set().union(*[_regs(o) for o in ops[1:]]) if len(ops) > 1 else set()
                    if t.startswith("v_mfma"):
                        reads -= _regs(ops[-1]) if ops else set()   # accumulator operand
                    if reads & dst:
                        bad.append((i + 1, ln[:60], "->", target + 1, t[:60]))
                        break
                    waited += 1
                break
    assert not bad, f"{name}: result of an MFMA read right after a branch: {bad[:5]}"


def test_expert_kernels_use_no_scratch_memory(asm):
    """No expert kernel may keep anything in scratch (private) memory.  It happens silently: a
    reference that selects between the two by-value parameter structs of a launch (routed /
    shared expert) turned into a stack copy of the struct when an early return was placed in
    front of it, and the mid-batch kernels ran a third slower with every test still passing.
    The load-time repack kernel is the one exception (it runs once per layer)."""
    name, lines = asm
    if name == "ffn_tiled.hip":
        pytest.skip("the tiled kernels spill a few prologue values around their main loop by design "
                    "(512 registers per wave are all taken)")
    allowed = ("repack_blocks_kernel",)
    kernel, bad, seen = None, [], 0
    for ln in lines:
        if ln.startswith(".name:"):
            kernel = ln.split(":", 1)[1].strip()
        elif ln.startswith(".private_segment_fixed_size:"):
            size = int(ln.split(":")[1])
            seen += 1
            if size and kernel and not any(a in kernel for a in allowed):
                bad.append((kernel[:80], size))
    assert seen > 0, f"{name}: no kernel metadata found"
    assert not bad, f"{name}: kernels with scratch memory: {bad}"
