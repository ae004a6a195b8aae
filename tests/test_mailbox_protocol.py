"""The mailbox folded into the layer call, as a protocol: every interleaving of one level op (copy stream + polling host) with
three layer calls (device) is enumerated on a small model, and the reference's rules are checked on each
(threads/13-moe-layer-kernel/INTEGRATION.md:215-232, sm120/nqmoe.cu:908-923, sm120/levelswitch_mbox.py:33-65):

  (S) no launch reads a slot after the host was told that its row is gone (the host frees and overwrites it at once);
  (U) all parts of one call work from one reading of an expert's row (level, slot, sign vector);
  (V) the row a call used is the state the host believes in once that call has ended and it has polled;
  (L) an op that has landed is in use and published two calls later at the latest.

Device steps of one call, in the order the launches give them (nestquant_amd/csrc/nq_moe.hip):
  PUB    routing launch, workgroup 0: applied_host <- applied
  ROUTE  routing launch: header <- table[e]                      (every workgroup reads the same table: one observer)
  GU     gate|up launch: reads the planes the header names
  DN / APPLY  down launch: reads the planes the header names; its mailbox block reads seq and, if it moved, stage ->
         table, seq -> applied (the two are concurrent: both orders are enumerated)
The copy stream writes [slot bytes,] stage row, seq in order; the host polls after every step of anybody (the earliest
moment it could act) and, for a demotion it sees published, frees the slot and overwrites it.

A second model is the form this protocol replaced (every routing workgroup read seq for itself, the first projection launch
read it a third time and published at once); the same checker must reject it, which shows that the rules have teeth."""
import itertools

IMAGE, JUNK = "image", "junk"


class World:
    def __init__(s, op):
        s.op = op                                   # "demote": expert at level 4 in the slot -> 2; "promote": 2 -> 4
        old, new = ((4, "slot", "sc4"), (2, None, "sc2")) if op == "demote" else ((2, None, "sc2"), (4, "slot", "sc4"))
        s.table, s.new_row = old, new
        s.stage, s.seq, s.applied, s.applied_host, s.hseq = None, 0, 0, 0, 1
        s.slot = IMAGE if op == "demote" else JUNK
        s.host_level = old[0]                       # what the host believes; it moves when the host sees the op published
        s.errors = []

    # copy stream
    def c_slot(s): s.slot = IMAGE
    def c_row(s): s.stage = s.new_row
    def c_seq(s): s.seq = 1

    def host_poll(s):
        if s.host_level != s.new_row[0] and s.applied_host == s.hseq:
            s.host_level = s.new_row[0]
            if s.op == "demote":
                s.slot = JUNK                       # freed and overwritten at once (another expert's planes, or a scribble)

    def read_planes(s, hdr, who):
        if hdr[1] is not None and s.slot != IMAGE:
            s.errors.append(f"S: {who} decodes from a slot that does not hold the expert's planes")


def call_steps_new(w, used):
    """device steps of one call of the protocol in the library; `used` collects the row each call worked from"""
    st = {}
    def pub(): w.applied_host = w.applied
    def route(): st["hdr"] = w.table; used.append(w.table)
    def gu(): w.read_planes(st["hdr"], "gate|up")
    def dn(): w.read_planes(st["hdr"], "down")
    def apply():
        sq = w.seq
        if sq != w.applied:
            w.table, w.applied = w.stage, sq
    return [[pub, route, gu, dn, apply], [pub, route, gu, apply, dn]]


def call_steps_old(w, used):
    """the replaced form: two routing workgroups each read seq / stage for themselves, the gate|up launch's mailbox block reads
    seq again, writes the table and publishes immediately"""
    st = {}
    def look(): return w.stage if w.seq != w.applied else w.table
    def route_a(): st["hdr"] = look(); used.append(st["hdr"])
    def route_b():
        if look() != st["hdr"]:
            w.errors.append("U: two workgroups of one routing launch took different rows")
    def gu_apply():
        sq = w.seq
        if sq != w.applied:
            if w.stage != st["hdr"]:
                w.errors.append("U: the mailbox block applies a row this call did not route from")
            w.table, w.applied, w.applied_host = w.stage, sq, sq
    def gu(): w.read_planes(st["hdr"], "gate|up")
    def dn(): w.read_planes(st["hdr"], "down")
    return [[route_a, route_b, gu_apply, gu, dn]]


def run(op, call_steps, ncalls=3):
    """all interleavings; returns the set of rule violations found"""
    found = set()
    ncopy = 3 if op == "promote" else 2
    probe = call_steps(World(op), [])
    nsteps = len(probe[0])
    for variant in itertools.product(range(len(probe)), repeat=ncalls):
        total = nsteps * ncalls
        for places in itertools.combinations_with_replacement(range(total + 1), ncopy):   # copy step i goes before device step places[i]
            w, used = World(op), []
            device = []
            for c in range(ncalls):
                steps = call_steps(w, used)[variant[c]]
                device += [(c, f) for f in steps]
            copies = ([w.c_slot] if op == "promote" else []) + [w.c_row, w.c_seq]
            landed_before_call = None
            ci = 0
            for i in range(total + 1):
                while ci < ncopy and places[ci] == i:
                    copies[ci](); ci += 1
                    if ci == ncopy:
                        landed_before_call = (i + nsteps - 1) // nsteps        # first call that starts after the op has landed
                    w.host_poll()
                if i == total:
                    break
                c, f = device[i]
                f()
                w.host_poll()
                if i % nsteps == nsteps - 1 and used[c][0] != w.host_level:
                    w.errors.append(f"V: call {c} used level {used[c][0]}, the host believes {w.host_level}")
            if landed_before_call is not None and landed_before_call + 1 < ncalls:
                c = landed_before_call + 1                                     # two calls later at the latest: in use
                if used[c] != w.new_row:
                    w.errors.append("L: a landed op is still not in use two calls later")
            if landed_before_call is not None and landed_before_call + 1 < ncalls and w.host_level != w.new_row[0]:
                w.errors.append("L: a landed op is still not published two calls later")
            found |= set(w.errors)
    return found


def test_in_call_mailbox_protocol_holds_on_every_interleaving():
    for op in ("demote", "promote"):
        assert run(op, call_steps_new) == set(), op


def test_the_checker_rejects_the_multi_observer_form():
    bad = run("demote", call_steps_old)
    assert any(v.startswith("S:") for v in bad), bad                 # the slot is freed under the running launches
    assert any(v.startswith("U:") for v in bad), bad                 # and parts of one call disagree about the row
    assert any(v.startswith("U:") for v in run("promote", call_steps_old))
