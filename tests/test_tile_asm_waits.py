"""Static check of the generated tile assembly (grouped_mm_bf16_amd/csrc/gen_tile_asm.py), no GPU needed.

LDS reads complete in the order they were issued, and the generator puts in front of every MFMA the
`s_waitcnt lgkmcnt(n)` that is meant to prove exactly its own operands.  This test replays the K loop of every
variant instruction by instruction with that rule -- a read is known complete only once a wait has left fewer
reads outstanding than were issued after it -- and fails if an MFMA could issue while one of its operand
registers is still the destination of a read in flight, or if a read overwrites a fragment register that a
later MFMA of the same step still wants with its old value.

Vector-memory operations (the global -> LDS copies and the prefetch touches) leave their counter in issue order
too; a second replay follows the prologue and the K loop through whole tiles of 1 to 13 K tiles and fails if a
barrier that releases a buffer to the fragment reads could be passed while a copy into that buffer is in flight."""
import importlib.util
import os
import re

import pytest

ROOT = os.path.abspath(os.path.join(os.path.dirname(__file__), ".."))
spec = importlib.util.spec_from_file_location("gen_tile_asm", os.path.join(ROOT, "grouped_mm_bf16_amd", "csrc", "gen_tile_asm.py"))
gen = importlib.util.module_from_spec(spec)
spec.loader.exec_module(gen)


def regs(token):
    """'v[4:7]' -> {4..7}, 'v12' -> {12}; anything else -> empty."""
    m = re.fullmatch(r"v\[(\d+):(\d+)\]", token)
    if m:
        return set(range(int(m.group(1)), int(m.group(2)) + 1))
    m = re.fullmatch(r"v(\d+)", token)
    return {int(m.group(1))} if m else set()


def loop_bodies(variant):
    """The K tile bodies of a variant as lists of instructions: {(buffer, interior?): [...]} and the prologue's tail."""
    e = gen.Emit()
    gen.gen_main(variant, e, "T")
    bodies, cur, pro = {}, None, []
    for line in e.lines:
        m = re.match(r"; ---- k tile on buffer (\d+)( \(interior\))?", line)
        if m:
            cur = (int(m.group(1)), bool(m.group(2)))
            bodies[cur] = []
            continue
        if cur is None:
            pro.append(line)
        elif line.startswith("s_branch L_join") or line.endswith(":") and line.startswith(("L_join", "L_slow", "L_done")):
            cur = None if not line.startswith("L_slow") else cur
            if line.startswith("L_slow"):
                cur = None
        elif line.startswith(("s_cmp", "s_cbranch")) and cur is not None and "L_nofix" not in line and bodies[cur] and \
                bodies[cur][-1].startswith("s_add_u32 s56"):
            cur = None          # the loop control after a body
        else:
            bodies[cur].append(line)
    return pro, bodies


class Lds:
    def __init__(self):
        self.queue = []           # destination register sets of the LDS operations in flight, oldest first

    def busy(self):
        return set().union(*self.queue) if self.queue else set()

    def step(self, ins):
        op, _, rest = ins.partition(" ")
        args = [a.strip() for a in rest.split(",")]
        if op.startswith("ds_read"):
            self.queue.append(regs(args[0]))
        elif op.startswith("ds_write"):
            self.queue.append(set())
        elif op == "s_waitcnt":
            m = re.search(r"lgkmcnt\((\d+)\)", rest)
            if m:
                keep = int(m.group(1))
                self.queue = self.queue[len(self.queue) - keep:] if keep else []
        elif op == "s_barrier":
            pass
        elif op.startswith("v_mfma"):
            srcs = regs(args[1]) | regs(args[2])
            pending = self.busy() & srcs
            assert not pending, f"{ins}: operand registers {sorted(pending)} may still be in flight"


VARIANTS = [(a, b, tm) for a in (0, 1) for b in (0, 1) for tm in (4, 2, 1) if tm == 4 or not a]


@pytest.mark.parametrize("a_tr,b_tr,tm", VARIANTS)
def test_every_mfma_waits_for_its_own_operands(a_tr, b_tr, tm):
    v = gen.Variant(a_tr, b_tr, 0, tm)
    pro, bodies = loop_bodies(v)
    stages = v.stages
    assert sorted(bodies) == sorted((b, f) for b in range(stages) for f in (False, True))
    for interior in (True, False):
        lds = Lds()
        # the prologue ends with the reads of step 0 of K tile 0; nothing before them matters here
        first = [i for i, l in enumerate(pro) if l.startswith("ds_read")]
        for ins in pro[first[0]:]:
            lds.step(ins)
        n_mfma = 0
        for trip in range(2):                      # twice round the buffers: the second trip starts from the first's state
            for buf in range(stages):
                for ins in bodies[(buf, interior)]:
                    lds.step(ins)
                    n_mfma += ins.startswith("v_mfma")
        assert n_mfma == 2 * stages * 32 * tm      # 8 tm MFMAs per step, four steps per K tile


@pytest.mark.parametrize("a_tr,b_tr,tm", VARIANTS)
def test_fragment_sets_alternate_so_that_no_read_lands_on_live_operands(a_tr, b_tr, tm):
    """A read issued in a step must not target a register that an MFMA later in the same step still reads (the
    hardware would be free to deliver it early)."""
    v = gen.Variant(a_tr, b_tr, 0, tm)
    _, bodies = loop_bodies(v)
    for key, body in bodies.items():
        # steps are delimited by the 8 tm MFMAs they hold
        idx = [i for i, l in enumerate(body) if l.startswith("v_mfma")]
        per = 8 * tm
        assert len(idx) == 4 * per
        for s in range(4):
            lo = idx[s * per]
            hi = idx[(s + 1) * per - 1]
            for i in range(lo, hi):
                if body[i].startswith("ds_read"):
                    dst = regs(body[i].split(" ", 1)[1].split(",")[0].strip())
                    for j in range(i + 1, hi + 1):
                        if body[j].startswith("v_mfma"):
                            a = [x.strip() for x in body[j].split(" ", 1)[1].split(",")]
                            assert not dst & (regs(a[1]) | regs(a[2])), (key, body[i], body[j])


def test_the_checker_catches_a_missing_wait():
    """Sanity of the test itself: drop the waits and the replay must object."""
    v = gen.Variant(0, 1, 0, 4)
    pro, bodies = loop_bodies(v)
    lds = Lds()
    first = [i for i, l in enumerate(pro) if l.startswith("ds_read")]
    with pytest.raises(AssertionError, match="may still be in flight"):
        for ins in pro[first[0]:] + bodies[(0, True)]:
            if not ins.startswith("s_waitcnt"):
                lds.step(ins)


class Vmem:
    """Vector-memory operations leave the counter in the order they were issued: `s_waitcnt vmcnt(n)` proves
    everything but the n youngest complete.  Tracks, for the copies (global -> LDS) in flight, the buffer each
    one fills: m0 is set to (wave base of A in s76 / of B in s77) + offset right before a copy."""

    def __init__(self, v):
        self.v = v
        self.flight = []          # oldest first: buffer index of a copy, None for a touch
        self.m0 = None

    def step(self, ins):
        op, _, rest = ins.partition(" ")
        if op == "s_add_u32" and rest.startswith("m0,"):
            base, off = [a.strip() for a in rest.split(",")][1:]
            is_a = base == "s%d" % (gen.S_T + 20)
            assert is_a or base == "s%d" % (gen.S_T + 21), ins
            stage = self.v.a_stage if is_a else self.v.b_stage
            self.m0 = (int(off) - (0 if is_a else self.v.b_base)) // stage
            assert 0 <= self.m0 < self.v.stages, ins
        elif op == "buffer_load_dwordx4":
            assert rest.rstrip().endswith("lds") or " lds" in rest, ins
            assert self.m0 is not None, "copy without a destination: " + ins
            self.flight.append(self.m0)
            self.m0 = None
        elif op.startswith("buffer_load"):
            self.flight.append(None)
        elif op == "s_waitcnt":
            m = re.search(r"vmcnt\((\d+)\)", rest)
            if m:
                keep = int(m.group(1))
                self.flight = self.flight[len(self.flight) - keep:] if keep else []

    def filling(self):
        return {b for b in self.flight if b is not None}


@pytest.mark.parametrize("a_tr,b_tr,tm", VARIANTS)
@pytest.mark.parametrize("nk", [1, 2, 3, 4, 5, 8, 13])
def test_a_k_tile_has_landed_before_its_buffer_is_read(a_tr, b_tr, tm, nk):
    """Replay of the prologue and of nk K tiles (the interior body where the generated branch takes it): at the
    barrier that ends the prologue no copy into buffer 0 may be in flight, and at the barrier inside K tile kt
    none into the buffer of K tile kt + 1 -- the fragment reads that follow each barrier take what is there."""
    v = gen.Variant(a_tr, b_tr, 0, tm)
    pro, bodies = loop_bodies(v)
    S = v.stages
    vm = Vmem(v)
    first_barrier = pro.index("s_barrier")
    for ins in pro[:first_barrier]:
        vm.step(ins)
    assert 0 not in vm.filling(), "K tile 0 may still be on its way when the prologue's barrier is passed"
    for ins in pro[first_barrier:]:
        vm.step(ins)
    for kt in range(nk):
        buf = kt % S
        interior = kt + S < nk - 1          # the branch in front of every body
        body = bodies[(buf, interior)]
        barrier = body.index("s_barrier")
        for ins in body[:barrier]:
            vm.step(ins)
        assert (buf + 1) % S not in vm.filling(), f"K tile {kt + 1} may still be on its way at the barrier of K tile {kt}"
        for ins in body[barrier:]:
            vm.step(ins)


def test_the_copy_checker_catches_a_wait_that_allows_too_much():
    v = gen.Variant(0, 1, 0, 4)
    pro, bodies = loop_bodies(v)
    vm = Vmem(v)
    for ins in pro:
        vm.step(ins)
    body = bodies[(0, True)]
    barrier = body.index("s_barrier")
    for ins in body[:barrier]:
        if ins.startswith("s_waitcnt vmcnt"):
            ins = re.sub(r"vmcnt\(\d+\)", "vmcnt(%d)" % (v.nt + 1), ins)   # one operation more than the touches
        vm.step(ins)
    assert 1 in vm.filling()


def read_buffer(v, ins):
    """(operand, buffer) a fragment read takes its data from, or None for any other instruction."""
    m = re.match(r"ds_read_b(?:128|64_tr_b16) \S+, v(\d+)(?: offset:(\d+))?", ins)
    if not m:
        return None
    reg, off = int(m.group(1)), int(m.group(2) or 0)
    if gen.V_TMP <= reg < gen.V_TMP + 12:
        return None     # the masking of a partial first / last k chunk: its own stretch between two barriers, no copies in it
    if v.stages == 2:
        is_a = reg in (gen.V_RA, gen.V_RA + 1)
        assert is_a or reg in (gen.V_RB, gen.V_RB + 1), ins
        return ("A" if is_a else "B", off // (v.a_stage if is_a else v.b_stage))
    is_a = gen.V_BUFA <= reg < gen.V_BUFA + 6
    assert is_a or gen.V_BUFB <= reg < gen.V_BUFB + 6, ins
    return ("A" if is_a else "B", (reg - (gen.V_BUFA if is_a else gen.V_BUFB)) // 2)


@pytest.mark.parametrize("a_tr,b_tr,tm", VARIANTS)
def test_no_buffer_is_copied_into_between_the_barriers_that_it_is_read_between(a_tr, b_tr, tm):
    """The four waves of a workgroup run the same code and meet at every barrier, so what one wave reads and what
    another one overwrites can only collide inside one stretch between two barriers: there, the buffers read and
    the buffers that copies are aimed at must differ."""
    v = gen.Variant(a_tr, b_tr, 0, tm)
    pro, bodies = loop_bodies(v)
    S = v.stages
    for nk in (1, 2, 3, 5, 9):
        stream = list(pro)
        for kt in range(nk):
            stream += bodies[(kt % S, kt + S < nk - 1)]
        check_stretches(v, stream)


def check_stretches(v, stream):
    read, written, m0 = set(), set(), None
    for ins in stream:
        if ins == "s_barrier":
            read, written = set(), set()
        elif ins.startswith("s_add_u32 m0,"):
            base, off = [a.strip() for a in ins.split(" ", 1)[1].split(",")][1:]
            is_a = base == "s%d" % (gen.S_T + 20)
            m0 = ("A" if is_a else "B", (int(off) - (0 if is_a else v.b_base)) // (v.a_stage if is_a else v.b_stage))
        elif ins.startswith("buffer_load_dwordx4"):
            written.add(m0)
        elif read_buffer(v, ins):
            read.add(read_buffer(v, ins))
        assert not read & written, (ins, sorted(read & written))


def test_the_stretch_checker_catches_a_copy_into_the_buffer_being_read():
    v = gen.Variant(0, 1, 0, 4)
    pro, bodies = loop_bodies(v)
    body = list(bodies[(0, True)])
    # step 3's copies (after the barrier) go into buffer 0; moved in front of the barrier they hit the buffer
    # that steps 0 to 2 read
    barrier = body.index("s_barrier")
    late = [i for i in range(barrier, len(body)) if body[i].startswith("s_add_u32 m0,")][0]
    moved = body[late:late + 3]
    assert any(x.startswith("buffer_load_dwordx4") for x in moved)
    with pytest.raises(AssertionError):
        check_stretches(v, pro + body[:barrier] + moved + body[barrier:])
