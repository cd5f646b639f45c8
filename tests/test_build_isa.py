"""Build-time checks on the compiled gfx950 ISA (hipcc cross-compiles here, no GPU needed).

The BPTT kernel issues its per-step global loads with inline assembly and waits for them with an
explicit s_waitcnt vmcnt(N), where N counts the vector-memory instructions (loads and stores alike:
one in-order counter on this target) issued after the loads being waited for.  The compiler does not know those destination registers are still being filled,
so this test proves on the emitted code that nothing reads or writes them between the load and the
wait that covers it, and that the hot loops use no scratch memory."""
import os
import re
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "rnn_train_ring_attractor_amd", "csrc")
from rnn_train_ring_attractor_amd.build import PER_SOURCE_FLAGS  # noqa: E402

HIPCC = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"

pytestmark = pytest.mark.skipif(not os.path.exists(HIPCC), reason="hipcc not available")


@pytest.fixture(scope="module")
def res256_asm(tmp_path_factory):
    out = tmp_path_factory.mktemp("isa") / "res256.s"
    cmd = [HIPCC, "--offload-arch=gfx950", "-O3", "-std=c++17", "-S", "--cuda-device-only", f"-I{ROOT}/include",
           f"-I{CSRC}", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
           *PER_SOURCE_FLAGS.get("ring_res256.hip", []),
           "-Rpass-analysis=kernel-resource-usage", os.path.join(CSRC, "ring_res256.hip"), "-o", str(out)]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    assert proc.returncode == 0, proc.stderr[-2000:]
    return out.read_text(), proc.stderr


def _regs(tok):
    out = set()
    for m in re.finditer(r"\bv\[(\d+):(\d+)\]", tok):
        out |= set(range(int(m.group(1)), int(m.group(2)) + 1))
    for m in re.finditer(r"\bv(\d+)\b", tok):
        out.add(int(m.group(1)))
    return out


def _kernel_body(asm, mangled):
    i = asm.index(mangled + ":")
    return asm[i:asm.index("s_endpgm", i)].split("\n")


@pytest.mark.parametrize("ga", [0, 1], ids=["weights_only", "with_grad_A"])
@pytest.mark.parametrize("merge", [0, 1], ids=["stores_per_step", "merged_pair_stores"])
@pytest.mark.parametrize("loss", [0, 1], ids=["grad_output", "fused_loss"])
def test_async_loads_are_not_touched_before_their_wait(res256_asm, loss, merge, ga):
    asm, _ = res256_asm
    depth = 2                           # input stages in flight (the launcher's choice)
    body = _kernel_body(asm, f"_Z23ring_bptt_res256_kernelILb1ELb{loss}ELb{merge}ELi{depth}ELb{ga}EEv12RingBpttArgs")
    fifo, loads, waits, tag = [], 0, 0, None
    for ln in body + body:                      # second pass models the loop back edge
        t = ln.strip()
        if t.startswith(".Lring_async_load_"):
            tag = "load"
            continue
        if t.startswith(".Lring_async_wait_"):
            tag = "wait"
            continue
        if not t or t[0] in ";.":
            continue
        if tag == "load":
            assert t.startswith(("global_load_dwordx4", "global_load_dwordx2")), t
            fifo.append(_regs(t.split()[1].rstrip(",")))
            loads += 1
            tag = None
            continue
        if tag == "wait":
            k = int(re.search(r"vmcnt\((\d+)\)", t).group(1))
            del fifo[:max(0, len(fifo) - k)]
            waits += 1
            tag = None
            continue
        if t.startswith("s_waitcnt") and "vmcnt(0)" in t:
            fifo = []
            continue
        # every other vector-memory instruction occupies a slot of the same in-order counter: stores define no
        # register, compiler-issued loads are waited for by the compiler itself
        if t.startswith(("global_store", "global_load", "buffer_store", "buffer_load", "scratch_")):
            fifo.append(set())
            continue
        pending = set().union(*fifo) if fifo else set()
        ops = t.split(None, 1)
        used = _regs(ops[1]) if len(ops) > 1 else set()
        assert not (used & pending), f"in-flight registers {sorted(used & pending)} touched by: {t}"
    assert loads >= 12 and waits >= 2           # the pattern is present at all


def test_hot_kernels_use_no_scratch(res256_asm):
    _, remarks = res256_asm
    blocks = re.split(r"remark: Function Name: ", remarks)
    seen = 0
    for b in blocks[1:]:
        name = b.split()[0]
        m = re.search(r"ScratchSize \[bytes/lane\]: (\d+)", b)
        full_fwd = re.match(r"_Z22ring_fwd_res256_kernelILi\dELb[01]ELb1ELb[01]EE", name)
        full_bptt = name.startswith("_Z23ring_bptt_res256_kernelILb1E")
        if full_fwd or full_bptt:
            seen += 1
            assert int(m.group(1)) == 0, f"{name} spills {m.group(1)} bytes per lane"
    assert seen >= 12


# ------------------------------------------------------------------------------------------------
# The N = 512 cluster forward issues its flag, gate, previous-state and operand loads with inline assembly as
# well and waits for them with counted s_waitcnt.  Same proof on its emitted code: between such a load and the first
# wait that covers it nothing reads or writes its destination registers (a copy "into place" ahead of the wait would
# copy a register that is still being filled), and no variant uses scratch memory.
# ------------------------------------------------------------------------------------------------
@pytest.fixture(scope="module")
def cluster_asm(tmp_path_factory):
    out = tmp_path_factory.mktemp("isa") / "cluster.s"
    cmd = [HIPCC, "--offload-arch=gfx950", "-O3", "-std=c++17", "-S", "--cuda-device-only", f"-I{ROOT}/include",
           f"-I{CSRC}", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
           *PER_SOURCE_FLAGS.get("ring_cluster.hip", []),
           "-Rpass-analysis=kernel-resource-usage", os.path.join(CSRC, "ring_cluster.hip"), "-o", str(out)]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    assert proc.returncode == 0, proc.stderr[-2000:]
    return out.read_text(), proc.stderr


def _sregs(tok):
    out = set()
    for m in re.finditer(r"\bs\[(\d+):(\d+)\]", tok):
        out |= set(range(int(m.group(1)), int(m.group(2)) + 1))
    for m in re.finditer(r"\bs(\d+)\b", tok):
        out.add(int(m.group(1)))
    return out


def _function_body(asm, name):
    i = asm.index(name + ":")
    return asm[i:asm.index(".Lfunc_end", i)].split("\n")


def _instructions(body):
    """(inside an asm statement?, instruction text) for every instruction of a function body."""
    in_asm = False
    for ln in body:
        t = ln.strip()
        if t.startswith(";;#ASMSTART"):
            in_asm = True
        elif t.startswith(";;#ASMEND"):
            in_asm = False
        elif t and t[0] not in ";.":
            yield in_asm, t


def _check_in_flight(body):
    """Asserts that nothing touches the destination of an asm-issued load before a wait covers it; returns the
    number of such loads seen (over two passes of the body: the second models the loop back edge)."""
    fifo, loads = [], 0
    for in_asm, t in list(_instructions(body)) * 2:
        if in_asm and t.startswith("global_load"):
            fifo.append(_regs(t.split()[1].rstrip(",")))
            loads += 1
            continue
        if t.startswith("s_waitcnt") and "vmcnt" in t:
            k = int(re.search(r"vmcnt\((\d+)\)", t).group(1))
            del fifo[:max(0, len(fifo) - k)]
            continue
        # every other vector-memory instruction occupies a slot of the same in-order counter
        if t.startswith(("global_store", "global_load", "buffer_", "scratch_")):
            fifo.append(set())
            continue
        pending = set().union(*fifo) if fifo else set()
        ops = t.split(None, 1)
        used = _regs(ops[1]) if len(ops) > 1 else set()
        assert not (used & pending), f"in-flight registers {sorted(used & pending)} touched by: {t}"
    return loads


CLUSTER_KERNELS = [f"_Z24ring_fwd_cluster8_kernelILi{act}ELb{save}EEv11RingFwdArgs15RingClusterArgs"
                   for act in range(4) for save in (0, 1)] + \
                  [f"_Z25ring_bptt_cluster8_kernelILb{gri}EEv12RingBpttArgs15RingClusterArgs" for gri in (0, 1)]


@pytest.mark.parametrize("save", [0, 1], ids=["history_only", "with_record"])
@pytest.mark.parametrize("act", [0, 1, 2, 3], ids=["relu", "gelu", "tanh", "silu"])
def test_cluster_forward_leaves_in_flight_registers_alone(cluster_asm, act, save):
    asm, _ = cluster_asm
    loads = _check_in_flight(_function_body(asm, f"_Z24ring_fwd_cluster8_kernelILi{act}ELb{save}EEv11RingFwdArgs15RingClusterArgs"))
    assert loads == 2 * 14          # early half: 2 previous-state, gates, flags, 4 operand; late half: gates, flags, 4 operand


@pytest.mark.parametrize("gri", [0, 1], ids=["weights_only", "with_grad_r_init"])
def test_cluster_bptt_leaves_in_flight_registers_alone(cluster_asm, gri):
    asm, _ = cluster_asm
    loads = _check_in_flight(_function_body(asm, f"_Z25ring_bptt_cluster8_kernelILb{gri}EEv12RingBpttArgs15RingClusterArgs"))
    assert loads == 2 * 20          # early half: 8 epilogue inputs, gates, flags, 4 operand; late half: gates, flags, 4 operand


@pytest.mark.parametrize("name", CLUSTER_KERNELS)
def test_cluster_asm_memory_instructions_keep_their_hazard_distances(cluster_asm, name):
    """The compiler's hazard recognizer does not look inside asm statements.  Two hazards of gfx950 concern the
    vector-memory instructions issued there: a store of more than 8 bytes per lane reads its data registers during
    the two wait states after it issues (a vector-ALU write to them in that window changes what is stored: the store
    carries its own s_nop 1), and a vector-ALU write of a scalar register (v_readfirstlane, v_cmp) needs five wait
    states before a vector-memory instruction reads it."""
    asm, _ = cluster_asm
    ins = list(_instructions(_function_body(asm, name)))
    wide = 0
    for k, (in_asm, t) in enumerate(ins):
        if not (in_asm and t.startswith(("global_load", "global_store"))):
            continue
        if t.startswith(("global_store_dwordx4", "global_store_dwordx3")):
            wide += 1
            assert ins[k + 1] == (True, "s_nop 1"), f"no wait states behind: {t}"
        need = _sregs(t)
        ws = 0
        for _, pt in reversed(ins[max(0, k - 8):k]):
            if ws >= 5:
                break
            op = pt.split()[0]
            if op.startswith("v_"):
                dst = pt.split(None, 1)[1].split(",")[0]
                assert not (_sregs(dst) & need), f"{pt} writes a scalar register {ws} wait states before: {t}"
            ws += int(pt.split()[1]) + 1 if op == "s_nop" else 1
    assert wide >= 4


def test_cluster_kernels_use_no_scratch(cluster_asm):
    _, remarks = cluster_asm
    seen = 0
    for b in re.split(r"remark: Function Name: ", remarks)[1:]:
        name = b.split()[0]
        if name.startswith(("_Z24ring_fwd_cluster8_kernel", "_Z25ring_bptt_cluster8_kernel")):
            seen += 1
            m = re.search(r"ScratchSize \[bytes/lane\]: (\d+)", b)
            assert int(m.group(1)) == 0, f"{name} spills {m.group(1)} bytes per lane"
    assert seen == 10
