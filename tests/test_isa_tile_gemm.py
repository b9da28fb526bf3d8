"""The tile GEMM states its own s_waitcnt counts for the weight prefetch and for the activation loads that go straight
into LDS; the counts assume the order in which a wavefront issues its vector-memory instructions in a k-step.  This
test compiles the kernel to assembly (no GPU needed) and checks, in every instantiation, that the k-loop issues its
loads in exactly that order with exactly those waits and no others.  "No others" matters twice: a wait the compiler
had to add would mean a stated count was too weak for a register dependency (the compiler tracks those), and a wait
for "all outstanding loads" anywhere in the loop would serialise the prefetch.  The dependency the compiler cannot see
(another wavefront reading what this one's loads wrote into LDS) is checked here by counting."""
import re
import subprocess
import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parents[1]
sys.path.insert(0, str(ROOT))
from onnxruntime_amd import build  # noqa: E402


@pytest.fixture(scope="module")
def kernels(tmp_path_factory):
    out = tmp_path_factory.mktemp("isa") / "mnb_gemm256.s"
    cmd = [build.hipcc(), *[f for f in build.HIPCC_FLAGS if f != "-fPIC"], "--cuda-device-only", "-S",
           str(build.CSRC / "mnb_gemm256.hip"), "-o", str(out)]
    subprocess.run(cmd, check=True, capture_output=True)
    found, name, lines = {}, None, []
    for line in out.read_text().splitlines():
        m = re.match(r"^(_Z\S+):\s", line)
        if m:
            if name:
                found[name] = lines
            name, lines = m.group(1), []
        elif name:
            lines.append(line)
    found[name] = lines
    return {k: v for k, v in found.items() if "mnb_gemm256_kernelILi" in k}


def _hot_loops(lines):
    """Token streams of the loops that hold matrix instructions: D = load into LDS, L = load into registers,
    BAR = barrier, wN = s_waitcnt vmcnt(N); from a label to the branch back to it."""
    loops, cur, label = [], [], None
    for line in lines:
        m = re.match(r"^(\.LBB\d+_\d+):", line)
        if m:
            cur, label = [], m.group(1)
        cur.append(line)
        if label and re.match(r"\s+s_cbranch_\w+\s+" + re.escape(label) + r"\b", line):
            loops.append(cur)
            cur, label = [], None
    out = []
    for body in loops:
        if sum("v_mfma" in x for x in body) < 16:
            continue
        toks = []
        for x in body:
            if re.match(r"\s+s_barrier", x):
                toks.append("BAR")
            elif re.match(r"\s+buffer_load_dwordx4 .* lds\b", x):
                toks.append("D")
            elif re.match(r"\s+(buffer_|global_|flat_|scratch_)(load|store|atomic)", x):
                toks.append("L")
            elif re.match(r"\s+s_waitcnt", x) and "vmcnt" in x:
                toks.append("w" + re.search(r"vmcnt\((\d+)\)", x).group(1))
        out.append(toks)
    return out


class Plan:
    """The issue order of a k-step, restated: slot 0 the activation loads, slots 1..3 the weight registers reloaded
    after the operands of slabs 1..3 were made, slot 4 those reloaded after slab 0's (behind the barrier)."""

    def __init__(self, bits, mps, a_loads, ct):
        """a_loads: activation loads per thread and k-step (tile rows x 8 / threads); ct: 32-column matrix-core tiles
        per wavefront = loads per weight vector and per meta entry."""
        self.bits, self.mps = bits, mps
        vps = 2 if bits == 4 else 4
        after = lambda kk: 4 if kk == 0 else kk  # noqa: E731
        self.vec_slot = [after(2 * v + 1 if bits == 4 else v) for v in range(vps)]
        self.meta_slot = [after(2 * e + 1 if bits == 4 else (e + 1) * 4 // mps - 1) for e in range(mps)]
        self.size = [a_loads] + [ct * self.vec_slot.count(q) + ct * self.meta_slot.count(q) for q in range(1, 5)]
        self.per_step = sum(self.size)

    def before(self, q):
        return sum(self.size[:q])

    def younger(self, q, steps, q_now):
        return steps * self.per_step + self.before(q_now) - self.before(q) - self.size[q]

    def wait_of_slab(self, kk):
        ahead, q_now = (1, 4) if kk == 0 else (0, kk)
        qv = self.vec_slot[kk >> 1 if self.bits == 4 else kk]
        qm = self.meta_slot[kk >> 1 if self.bits == 4 else kk * self.mps // 4]
        return min(self.younger(q, (3 if q == 4 else 2) - ahead, q_now) for q in (qv, qm))

    def wait_of_barrier(self):
        return min(self.younger(0, 1, 4), self.wait_of_slab(0))

    def step_tokens(self):
        toks = ["D"] * self.size[0]
        for kk in (1, 2, 3):
            if not (self.bits == 4 and kk & 1):
                toks.append(f"w{self.wait_of_slab(kk)}")
            toks += ["L"] * self.size[kk]
        bar = f"w{self.wait_of_barrier()}"
        return toks + [bar, "BAR", bar] + ["L"] * self.size[4]


def test_every_instantiation_issues_its_loads_and_waits_as_planned(kernels):
    # {4-bit, 8-bit with 2 or 4 entries} x {zp, none} x {128, 256 rows} x {fp16, bfloat16}, less the one that does not
    # fit the register file (bfloat16, four entries with zero points, 256 rows: never launched), plus fp16 on fp32
    # meta entries (zero points in the activation type: 4-bit with zero points) x {128, 256 rows}, plus the 128 x 128
    # tiles of four wavefronts for fp16 and bfloat16 models ({4-bit, 8-bit with 2 or 4 entries} x {zp, none} each)
    assert len(kernels) == 37
    for name, lines in kernels.items():
        bits, mps, tm, wm, nwv = (int(x) for x in re.search(
            r"kernelILi(\d)ELb[01]ELi(\d)ELi(\d)ELi(\d)ELi\dELi(\d)E", name).groups())
        # nwv wavefronts form wm x nwv/wm; 64 tm rows x 8 chunks are loaded by 64 nwv threads
        plan = Plan(bits, mps, a_loads=64 * tm * 8 // (64 * nwv), ct=wm)
        loops = _hot_loops(lines)
        assert len(loops) == 1, name
        assert loops[0] == plan.step_tokens() * 2, (name, " ".join(loops[0]))


def test_activation_loads_have_landed_before_the_barrier_that_publishes_them(kernels):
    """The loads into LDS of one step are read by other wavefronts after the barrier of the next step.  Counted on the
    instruction stream of two consecutive loop iterations: between such a load and that barrier's wait lie at least as
    many younger vector-memory instructions as the wait leaves outstanding."""
    for name, lines in kernels.items():
        toks = _hot_loops(lines)[0] * 2
        bars = [i for i, t in enumerate(toks) if t == "BAR"]
        assert len(bars) == 4
        for n in (2, 3):
            # the loads into LDS issued between barriers n-2 and n-1 are published by barrier n
            group = [i for i in range(bars[n - 2], bars[n - 1]) if toks[i] == "D"]
            assert group, name
            wait = toks[bars[n] - 1]
            assert wait.startswith("w"), (name, wait)
            younger = sum(t in ("D", "L") for t in toks[group[-1] + 1:bars[n]])
            assert younger >= int(wait[1:]), (name, younger, wait)


def test_no_register_spills(kernels):
    for name, lines in kernels.items():
        scratch = [x for x in lines if "ScratchSize:" in x]
        assert scratch and all(x.split(":")[1].strip() == "0" for x in scratch), (name, scratch)
