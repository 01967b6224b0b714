#!/usr/bin/env python3
"""Generates rwkv_decode_back.inc: the weight-streaming ("back") waves of the single-token kernel,
written out instruction by instruction for each supported width.

    python gen_decode_back.py > rwkv_decode_back.inc

Why this is not C++: the ring of in-flight weight blocks has to live in a FIXED set of registers
that are reloaded in place, and the waits on it have to be counted by hand (loads of one wave return
in order).  Left to the register allocator every refill gets registers of its own, the ring needs
twice the space and spills; a spilled or copied in-flight register is silent corruption.  So the
whole back-wave program is one asm statement with its own register map; it talks to the compiled
front waves only through LDS and workgroup barriers.

Stream of one back wave (wave wb of 8) of workgroup g, in units of 1 KiB blocks ("positions"):
  per layer 13 jobs x KW blocks (job = one 16-column tile of a C-row matrix, or a quarter of the
  F-row ffn value tile; wave wb owns blocks wb, wb+8, ... of the job), padded to PP positions, a
  multiple of the ring size R, then the head tiles g, g+G, ... .  Position p lives in ring slot
  p % R.  At every position: wait until at most R-1 loads are outstanding (then the slot's block has
  landed), multiply, reload the slot with position p+R.  Every position issues exactly one load -
  padding positions and positions past the end of the head load a block that stays hot in L2 - so
  the wait count is the same everywhere.

Register map (VGPR; v0..v3 are left to the compiler): v4 A-operand address (C-row digit sets), v5
same for the F-row set, v6 park address, v7 abort-flag address, v8..v15 byte offset of block b
inside a job, v16..v23 two accumulators, v24..v35 three A-operand buffers, v[RB..NV-1] the ring (NV = the workgroup's VGPR budget).
SGPR: s36..s61 job base addresses of the current layer (13 pairs), s64..s89 of the next layer,
s90..s99 scalars, vcc as a scratch pair.
"""
import math
import sys

V_APC, V_APF, V_PARK, V_FLAG, V_OFF, V_D, V_A = 4, 5, 6, 7, 8, 16, 24
NA = 3            # A-operand buffers
S_CUR, S_NXT = 36, 64
S_L, S_T, S_JT, S_TILE, S_RT, S_RP, S_PAR = 90, 91, 92, 94, 95, 96, 99
PF = NA - 1       # A-operand reads run this many positions ahead
import os
WINDOW = int(os.environ.get("RWKV_BACK_WINDOW", "5"))
DEFER = int(os.environ.get("RWKV_BACK_DEFER", "1"))
# per-phase windows for the reloads that follow the barrier of the att k/v/r, att output, ffn key and ffn value phases
WINDOWS = [int(x) for x in os.environ.get("RWKV_BACK_WINDOWS", ",".join([str(WINDOW)] * 4)).split(",")]
BURST = int(os.environ.get("RWKV_BACK_BURST", "0"))      # the first BURST reloads after a phase's barrier go out back to back
PACE = int(os.environ.get("RWKV_BACK_PACE", "0"))        # s_sleep units (64 cycles) in front of every deferred reload: the reloads of a phase go out at a steady rate instead of as fast as the window allows
# RWKV_BACK_GATE="a,b,c,d": after the barrier of the att k/v/r, att output, ffn key and ffn value phases only the first
# a / b / c / d deferred reloads go out at once, so that the front waves' polls and gathers of the NEXT exchange do
# not queue behind a burst of weight loads.  The rest follow once every workgroup's results of that exchange have
# arrived: for the att k/v/r and ffn key phases a bounded spin on the LDS word FLAG_GO, for the att output and ffn
# value phases (BARGATE) simply after the first barrier of the LayerNorm phase that follows, which the front waves
# only reach with the statistics of all workgroups in hand.  Empty: no gate.
GATE = [int(x) for x in os.environ.get("RWKV_BACK_GATE", "8,2,12,6").split(",")] if os.environ.get("RWKV_BACK_GATE", "8,2,12,6") else None
WINDOW_WIDE = int(os.environ.get("RWKV_BACK_WINDOW_WIDE", "12"))
GATE_WIDE = [int(x) for x in os.environ.get("RWKV_BACK_GATE_WIDE", "16,8,16,12").split(",")]     # the same for two groups per workgroup (C = 5120)
BARGATE = int(os.environ.get("RWKV_BACK_BARGATE", "1"))   # reloads deferred past the att output and ffn value phases follow the next phase's first barrier
CARRYK = int(os.environ.get("RWKV_BACK_CARRYK", "0"))     # the carried reloads follow this barrier of the LayerNorm phase (0: statistics, 1: digits ready)
CARRYW = int(os.environ.get("RWKV_BACK_CARRYW", "0"))     # window of the carried reloads (0: the phase's)
# the same for workgroups whose ffn key tiles are streamed by helper workgroups (9 jobs per layer)
GATE_HELP = [int(x) for x in os.environ.get("RWKV_BACK_GATE_HELP", "8,2,12,6").split(",")]
WINDOW_HELP = int(os.environ.get("RWKV_BACK_WINDOW_HELP", "5"))
R_HELP = int(os.environ.get("RWKV_BACK_R_HELP", "23"))
GATE_SPINS = 1 << 16     # the gate gives way after this many looks (a few milliseconds): it only orders loads, it must never hold a wave
S_SEQ = 98        # phases finished by this wave (the front waves' exchange sequence number runs one ahead)
SLEEP = int(os.environ.get("RWKV_BACK_SLEEP", "0"))      # s_sleep units (64 cycles) between a phase's barrier and its reloads   # weight loads a wave keeps in flight while it reloads slots


S_FLAG = 100      # LDS address of the abort / go flag pair, where no register holds it (compact register map)


class Emit:
    def __init__(self, na=NA):
        self.lines = []
        self.issued = 0          # LDS operations issued since the last full drain
        self.ridx = [0] * na      # issue index of the read into A buffer k

    def __call__(self, s):
        self.lines.append(s)

    def drain_state(self):
        self.issued = 0


S_TMP = 62        # scratch pair for a block's address where block offsets are added on the scalar side


def gen(KW, R, NV, NSH, HELP=False):
    """HELP: the four ffn key tiles of a group are not this workgroup's (helper workgroups on the otherwise idle
    compute units own that matrix): 9 jobs per layer instead of 13, and the ffn receptance tile takes its digits
    from the first set of planes."""
    C = 512 * KW
    F = 4 * C
    PS, PSF = C + 64, F + 64
    NT = 2 if KW > 8 else 1          # groups of 16 channels (and their tiles) per workgroup
    SPG = 5                          # parked-tile slots per group
    NWG = 32 * KW // NT              # workgroups
    SADDR = KW > 8                   # no room for one offset register per block of a job: the block offset joins the base address in a scalar pair
    # Compact register map where block offsets travel on the scalar side: one offset register, two A-operand buffers
    # and no register for the flag address leave room for a ring of 26 blocks in 128 registers.
    V_OFF, V_D, V_A, NA = (7, 8, 16, 2) if SADDR else (globals()["V_OFF"], globals()["V_D"], globals()["V_A"], globals()["NA"])
    PF = NA - 1
    NJ = (9 if HELP else 13) * NT    # jobs per layer
    GATE = globals()["GATE"] if NT == 1 else GATE_WIDE
    WINDOW = globals()["WINDOW"] if NT == 1 else WINDOW_WIDE
    WINDOWS = globals()["WINDOWS"] if NT == 1 else [WINDOW_WIDE] * 4
    if HELP:
        GATE, WINDOW, WINDOWS = GATE_HELP, WINDOW_HELP, [WINDOW_HELP] * 4
    NREAL = NJ * KW
    PP = (NREAL + R - 1) // R * R
    RB = NV - 4 * R
    assert RB >= V_A + 4 * NA, "ring does not fit"
    assert R <= NREAL and R - 1 <= 63
    TB = 8 * KW * 1024
    DIG = max(12 * PS, 4 * PSF)
    RED = DIG                                 # byte offset of the parked tiles from the start of LDS
    RED_SLOTS = max(SPG * NT, 2 * NSH)
    FLAG = RED + RED_SLOTS * 2048 + 32 * 8 + NT * 32 * 8 + 2 * 4   # FLAG_ABORT word

    # Jobs of a layer in stream order.  ptr: index of the job's base address in the workgroup's table row (that of
    # its first group; the same tile of the next group lies `stride` bytes further), aset/aoff: digit planes the
    # A operand comes from, chain: jobs that add into one accumulator (the four quarters of an ffn value tile),
    # slot: where the finished tile is parked.
    jobs = []
    for gi in range(NT):
        for m in range(3):
            jobs.append(dict(ph=0, gi=gi, ptr=m, stride=TB, aset="C", aoff=m * 4 * PS, first=True, park=gi * SPG + m))
    for gi in range(NT):
        jobs.append(dict(ph=1, gi=gi, ptr=3, stride=TB, aset="C", aoff=0, first=True, park=gi * SPG))
    for gi in range(NT):
        jobs.append(dict(ph=2, gi=gi, ptr=4, stride=TB, aset="C", aoff=0 if HELP else 4 * PS, first=True, park=gi * SPG))
        for r in range(0 if HELP else 4):
            jobs.append(dict(ph=2, gi=gi, ptr=5 + r, stride=TB, aset="C", aoff=0, first=True, park=gi * SPG + 1 + r))
    for gi in range(NT):
        for q in range(4):
            jobs.append(dict(ph=3, gi=gi, ptr=9 + q, stride=4 * TB, aset="F", aoff=q * C, first=q == 0, park=gi * SPG if q == 3 else None))
    assert len(jobs) == NJ
    # accumulators alternate from one chain to the next, so that a parked tile is still being written while the next one starts
    acc_of, chain = [], -1
    for jb in jobs:
        if jb["first"]:
            chain += 1
        acc_of.append(chain % 2)

    def block_load(dst, sbase, extra, b, wh=False):
        """16-byte-per-lane load of block b of a job whose base address is in s[sbase:sbase+1] (+ extra bytes)."""
        if wh:
            e(f"global_load_dwordx4 {dst}, v{V_OFF}, %[wh]")
        elif SADDR:
            e(f"s_add_u32 s{S_TMP}, s{sbase}, {extra + 8192 * b}")
            e(f"s_addc_u32 s{S_TMP + 1}, s{sbase + 1}, 0")
            e(f"global_load_dwordx4 {dst}, v{V_OFF}, s[{S_TMP}:{S_TMP + 1}]")
        else:
            assert extra == 0
            e(f"global_load_dwordx4 {dst}, v{V_OFF + b}, s[{sbase}:{sbase + 1}]")
    LH = R * KW // math.gcd(R, KW)
    e = Emit(NA)

    def flag_addr():
        """Register that holds the LDS address of the flag pair (valid where no A-operand read is in flight)."""
        if not SADDR:
            return f"v{V_FLAG}"
        e(f"v_mov_b32 v{V_A + 2}, s{S_FLAG}")
        return f"v{V_A + 2}"

    def ring(slot):
        return f"v[{RB + 4 * slot}:{RB + 4 * slot + 3}]"

    def abuf(q):
        k = q % NA
        return f"v[{V_A + 4 * k}:{V_A + 4 * k + 3}]"

    def aread(q_layer_pos=None, head_b=None):
        """Issue the A-operand read of a layer position (or of block head_b of a head tile)."""
        if head_b is not None:
            base, off, k = V_APC, 512 * head_b, head_b % NA
        else:
            q = q_layer_pos
            j, b = divmod(q, KW)
            base, off = (V_APC if jobs[j]["aset"] == "C" else V_APF), jobs[j]["aoff"] + 512 * b
            k = q % NA
        assert off < 65536
        e(f"ds_read_b128 v[{V_A + 4 * k}:{V_A + 4 * k + 3}], v{base} offset:{off}")
        e.ridx[k] = e.issued
        e.issued += 1

    def bar_check():
        e("s_waitcnt lgkmcnt(0)")
        e("s_barrier")
        e(f"ds_read_b32 v{V_A}, {flag_addr()}")
        e("s_waitcnt lgkmcnt(0)")
        e(f"v_readfirstlane_b32 s{S_T}, v{V_A}")
        e(f"s_cmp_lg_u32 s{S_T}, 0")
        e("s_cbranch_scc1 9f")
        e.drain_state()

    def park_static(dreg, slot):
        e("s_nop 7"); e("s_nop 7"); e("s_nop 7")
        e("s_mov_b64 exec, 0xffff")
        e(f"ds_write_b128 v{V_PARK}, v[{dreg}:{dreg + 3}] offset:{slot * 2048}")
        e("s_mov_b64 exec, -1")
        e.issued += 1

    # ------------------------------------------------------------------ prologue
    e("s_mov_b64 exec, -1")
    e(f"v_mbcnt_lo_u32_b32 v{V_A}, -1, 0")
    e(f"v_mbcnt_hi_u32_b32 v{V_A}, -1, v{V_A}")                 # lane
    e(f"v_and_b32 v{V_A + 1}, 3, v{V_A}")                      # n & 3
    e(f"v_lshrrev_b32 v{V_A + 2}, 4, v{V_A}")
    e(f"v_lshlrev_b32 v{V_A + 2}, 4, v{V_A + 2}")              # 16 * g4
    e(f"s_lshl_b32 s{S_T}, %[wb], 6")
    e(f"s_add_u32 s{S_T}, s{S_T}, %[lds]")
    e(f"v_mov_b32 v{V_A + 3}, {PS}")
    e(f"v_mul_u32_u24 v{V_APC}, v{V_A + 1}, v{V_A + 3}")
    e(f"v_add3_u32 v{V_APC}, v{V_APC}, v{V_A + 2}, s{S_T}")
    e(f"v_mov_b32 v{V_A + 3}, {PSF}")
    e(f"v_mul_u32_u24 v{V_APF}, v{V_A + 1}, v{V_A + 3}")
    e(f"v_add3_u32 v{V_APF}, v{V_APF}, v{V_A + 2}, s{S_T}")
    e(f"s_lshl_b32 s{S_T}, %[wb], 8")
    e(f"s_add_u32 s{S_T}, s{S_T}, %[lds]")
    e(f"s_add_u32 s{S_T}, s{S_T}, {RED}")
    e(f"v_lshlrev_b32 v{V_PARK}, 4, v{V_A}")
    e(f"v_add_u32 v{V_PARK}, s{S_T}, v{V_PARK}")
    e(f"s_add_u32 s{S_T}, %[lds], {FLAG}")
    e(f"s_mov_b32 s{S_FLAG}, s{S_T}" if SADDR else f"v_mov_b32 v{V_FLAG}, s{S_T}")
    e(f"s_lshl_b32 s{S_T}, %[wb], 10")
    e(f"v_lshlrev_b32 v{V_OFF}, 4, v{V_A}")
    e(f"v_add_u32 v{V_OFF}, s{S_T}, v{V_OFF}")
    if not SADDR:
        for b in range(1, KW):
            e(f"v_add_u32 v{V_OFF + b}, {8192 * b}, v{V_OFF}")
    e(f"s_mov_b64 s[{S_JT}:{S_JT + 1}], %[jt]")
    e(f"s_mov_b32 s{S_L}, %[L]")
    e(f"s_mov_b32 s{S_SEQ}, 0")
    for base, off in ((S_CUR, 0), (S_NXT, 128)):
        e(f"s_load_dwordx16 s[{base}:{base + 15}], s[{S_JT}:{S_JT + 1}], {off}")
        e(f"s_load_dwordx8 s[{base + 16}:{base + 23}], s[{S_JT}:{S_JT + 1}], {off + 64}")
        e(f"s_load_dwordx2 s[{base + 24}:{base + 25}], s[{S_JT}:{S_JT + 1}], {off + 96}")
    e("s_waitcnt lgkmcnt(0)")
    # Which reloads follow a barrier instead of a spin gate: those deferred past a phase whose successor starts with
    # the statistics barrier (att output -> ffn key/receptance; ffn value -> next layer / head).  What the ffn value
    # phase carries over is issued at the top of the next layer, after that layer's first barrier - also in the
    # first layer, which is why the prologue leaves those positions out.
    phases = []                                # start, end, barriers before
    for ph in range(4):
        idx = [i for i, jb in enumerate(jobs) if jb["ph"] == ph]
        phases.append((idx[0] * KW, (idx[-1] + 1) * KW, 2 if ph in (0, 2) else 1))
    def deferred_of(ph):
        ps, pe, _ = phases[ph]
        d = [p for p in range(ps, pe) if not (p + R < pe and DEFER) and DEFER]
        if pe == NREAL:
            d += list(range(NREAL, PP))
        return d
    carry_d = deferred_of(3)[GATE[3]:] if (GATE is not None and BARGATE) else []
    assert all(p + R >= PP for p in carry_d)
    skip = set(p + R - PP for p in carry_d)
    for p in range(R):
        if p in skip:
            continue
        j, b = divmod(p, KW)
        block_load(ring(p), S_CUR + 2 * jobs[j]["ptr"], jobs[j]["gi"] * jobs[j]["stride"], b)

    # ------------------------------------------------------------------ layers
    # Loads are issued in position order; position q's load is the q-th load of the wave.  A slot
    # is reloaded right away only when its next position still belongs to the current phase;
    # otherwise the reload waits until the phase's tiles are parked and the barrier is passed, so
    # that pushing requests into a busy memory system never delays the phase's results.
    def throttle(window=WINDOW):
        # A burst of reloads would sit in the compute unit's memory pipeline in front of the front
        # waves' polls and stores; keeping a window in flight paces the requests to what HBM delivers.
        if window - 1 < R - 1:
            e(f"s_waitcnt vmcnt({window - 1})")

    def layer_reload(p, window=WINDOW, top=False):
        """Reload the slot of layer position p (0 <= p < PP) with position p + R.  top: issued at the top of the
        NEXT layer (or of the head), where that layer's addresses have already become the current ones."""
        throttle(window)
        slot = p % R
        q = p + R
        sset = S_CUR
        if q >= PP:
            q -= PP
            sset = S_CUR if top else S_NXT
        else:
            assert not top
        if q >= NREAL:
            block_load(ring(slot), 0, 0, 0, wh=True)
        else:
            jq, bq = divmod(q, KW)
            block_load(ring(slot), sset + 2 * jobs[jq]["ptr"], jobs[jq]["gi"] * jobs[jq]["stride"], bq)

    e("1:")
    carry = []
    for ph, (ps, pe, nbar) in enumerate(phases):
        for k in range(nbar):
            bar_check()
            if k == CARRYK and nbar == 2:
                # behind the statistics barrier: every exchange word of this phase has been fetched
                for p in (carry_d if ph == 0 else carry):
                    layer_reload(p, CARRYW or WINDOWS[ph], top=(ph == 0))
                carry = []
        for q in range(ps, min(ps + PF, pe)):
            aread(q)
        issued_loads = ps + R          # loads issued so far: positions < ps + R
        deferred = []
        for p in range(ps, pe):
            j, b = divmod(p, KW)
            if p + PF < pe:
                aread(p + PF)
            allow = e.issued - 1 - e.ridx[p % NA]
            assert 0 <= allow <= 15
            nvm = issued_loads - 1 - p
            assert 0 <= nvm <= 63, (KW, R, p, nvm)
            e(f"s_waitcnt vmcnt({nvm}) lgkmcnt({allow})")
            dreg = V_D + 4 * acc_of[j]
            first = (b == 0) and jobs[j]["first"]
            acc = "0" if first else f"v[{dreg}:{dreg + 3}]"
            e(f"v_mfma_i32_16x16x64_i8 v[{dreg}:{dreg + 3}], {abuf(p)}, {ring(p % R)}, {acc}")
            if p + R < pe or not DEFER:
                assert issued_loads == p + R
                layer_reload(p)
                issued_loads += 1
            else:
                deferred.append(p)
            if b == KW - 1 and jobs[j]["park"] is not None:
                park_static(dreg, jobs[j]["park"])
        e("s_waitcnt lgkmcnt(0)")
        e("s_barrier")
        e.drain_state()
        if pe == NREAL:
            deferred += list(range(NREAL, PP))     # padding positions: nothing to compute, only their turn to load
        if SLEEP and deferred:
            e(f"s_sleep {SLEEP}")
        e(f"s_add_u32 s{S_SEQ}, s{S_SEQ}, 1")
        assert deferred == deferred_of(ph)
        if GATE is not None and BARGATE and ph in (1, 3):
            carry = deferred[GATE[ph]:]
            deferred = deferred[:GATE[ph]]
        for i, p in enumerate(deferred):
            assert issued_loads == p + R
            if GATE is not None and i == GATE[ph]:
                # wait for FLAG_GO >= phases finished + 1 (or the abort flag: then the next barrier check leaves)
                e(f"s_add_u32 s{S_T}, s{S_SEQ}, 1")
                e(f"s_mov_b32 s{S_TILE}, {GATE_SPINS}")       # (free until the head)
                e(f"7{ph}:")
                e(f"ds_read_b64 v[{V_A}:{V_A + 1}], {flag_addr()}")
                e("s_waitcnt lgkmcnt(0)")
                e(f"v_readfirstlane_b32 vcc_lo, v{V_A}")
                e(f"v_readfirstlane_b32 vcc_hi, v{V_A + 1}")
                e("s_cmp_lg_u32 vcc_lo, 0")
                e(f"s_cbranch_scc1 6{ph}f")
                e(f"s_cmp_ge_i32 vcc_hi, s{S_T}")
                e(f"s_cbranch_scc1 6{ph}f")
                e(f"s_sub_u32 s{S_TILE}, s{S_TILE}, 1")
                e(f"s_cmp_eq_u32 s{S_TILE}, 0")
                e(f"s_cbranch_scc1 6{ph}f")
                e("s_sleep 1")
                e(f"s_branch 7{ph}b")
                e(f"6{ph}:")
            if PACE and i >= BURST:
                e(f"s_sleep {PACE}")
            layer_reload(p, max(BURST, WINDOWS[ph]) if i < BURST else WINDOWS[ph])
            issued_loads += 1
    # end of layer: next layer's addresses become current; fetch the layer after
    e(f"s_add_u32 s{S_JT}, s{S_JT}, 128")
    e(f"s_addc_u32 s{S_JT + 1}, s{S_JT + 1}, 0")
    for i in range(13):
        e(f"s_mov_b64 s[{S_CUR + 2 * i}:{S_CUR + 2 * i + 1}], s[{S_NXT + 2 * i}:{S_NXT + 2 * i + 1}]")
    e(f"s_sub_u32 s{S_L}, s{S_L}, 1")
    e(f"s_cmp_eq_u32 s{S_L}, 0")
    e("s_cbranch_scc1 2f")
    e(f"s_load_dwordx16 s[{S_NXT}:{S_NXT + 15}], s[{S_JT}:{S_JT + 1}], 128")
    e(f"s_load_dwordx8 s[{S_NXT + 16}:{S_NXT + 23}], s[{S_JT}:{S_JT + 1}], 192")
    e(f"s_load_dwordx2 s[{S_NXT + 24}:{S_NXT + 25}], s[{S_JT}:{S_JT + 1}], 224")
    e("s_branch 1b")

    # ------------------------------------------------------------------ head
    # Rounds of NSH tiles: multiply, park, barrier, then the round's reloads.  The body below covers
    # LH = lcm(R, KW) positions (a whole number of rounds), after which slots and blocks line up again.
    def head_ptr():
        """s[S_RP] = address of head tile g + G * s[S_RT], or of tile 0 when that is past the end."""
        e(f"s_mul_i32 vcc_lo, s{S_RT}, {NWG}")
        e(f"s_add_u32 vcc_lo, vcc_lo, %[g]")
        e(f"s_cmp_ge_u32 vcc_lo, %[vt]")
        e(f"s_cselect_b32 vcc_lo, 0, vcc_lo")
        e(f"s_mul_hi_u32 vcc_hi, vcc_lo, {TB}")
        e(f"s_mul_i32 vcc_lo, vcc_lo, {TB}")
        e(f"s_add_u32 s{S_RP}, %[whlo], vcc_lo")
        e(f"s_addc_u32 s{S_RP + 1}, %[whhi], vcc_hi")

    def head_reload(q):
        """Reload the slot of body position q with position q + R of the head stream."""
        throttle()
        rb = (q + R) % KW
        if rb == 0:
            e(f"s_add_u32 s{S_RT}, s{S_RT}, 1")
            head_ptr()
        block_load(ring(q % R), S_RP, 0, rb)

    tiles_per_body = LH // KW
    assert tiles_per_body % NSH == 0
    e("2:")
    bar_check()
    if CARRYK == 0:
        for p in carry_d:
            layer_reload(p, CARRYW or WINDOW, top=True)
    bar_check()
    if CARRYK == 1:
        for p in carry_d:
            layer_reload(p, CARRYW or WINDOW, top=True)
    e(f"s_mov_b32 s{S_TILE}, 0")
    e(f"s_mov_b32 s{S_PAR}, 0")
    e(f"s_mov_b32 s{S_RT}, {R // KW - (1 if R % KW == 0 else 0)}")
    head_ptr()
    e("3:")
    for r0 in range(0, tiles_per_body, NSH):
        ps, pe = r0 * KW, (r0 + NSH) * KW
        issued_loads = ps + R
        deferred = []
        for q in range(ps, pe):
            tq, b = divmod(q, KW)
            dreg = V_D + 4 * (tq % 2)
            if b == 0:
                # a round that starts past the end of the head is not started; one that ends past it
                # is cut short after the last tile (label 8)
                e(f"s_cmp_ge_u32 s{S_TILE}, %[hr]")
                e("s_cbranch_scc1 8f" if tq % NSH else "s_cbranch_scc1 9f")
                e("s_waitcnt lgkmcnt(0)")
                e.drain_state()
                for bb in range(min(PF, KW)):
                    aread(head_b=bb)
            if b + PF < KW:
                aread(head_b=b + PF)
            allow = e.issued - 1 - e.ridx[b % NA]
            assert 0 <= allow <= 15
            nvm = issued_loads - 1 - q
            assert 0 <= nvm <= 63
            e(f"s_waitcnt vmcnt({nvm}) lgkmcnt({allow})")
            acc = "0" if b == 0 else f"v[{dreg}:{dreg + 3}]"
            e(f"v_mfma_i32_16x16x64_i8 v[{dreg}:{dreg + 3}], v[{V_A + 4 * (b % NA)}:{V_A + 4 * (b % NA) + 3}], {ring(q % R)}, {acc}")
            if q + R < pe or not DEFER:
                assert issued_loads == q + R
                head_reload(q)
                issued_loads += 1
            else:
                deferred.append(q)
            if b == KW - 1:
                e("s_nop 7"); e("s_nop 7"); e("s_nop 7")
                e(f"s_add_u32 s{S_T}, s{S_PAR}, {tq % NSH}")
                e(f"s_lshl_b32 s{S_T}, s{S_T}, 11")
                e(f"v_add_u32 v{V_A}, s{S_T}, v{V_PARK}")
                e("s_mov_b64 exec, 0xffff")
                e(f"ds_write_b128 v{V_A}, v[{dreg}:{dreg + 3}]")
                e("s_mov_b64 exec, -1")
                e(f"s_add_u32 s{S_TILE}, s{S_TILE}, 1")
        e("s_waitcnt lgkmcnt(0)")
        e("s_barrier")
        e(f"s_xor_b32 s{S_PAR}, s{S_PAR}, {NSH}")
        for q in deferred:
            assert issued_loads == q + R
            head_reload(q)
            issued_loads += 1
    e("s_branch 3b")
    e("8:")                      # the head ended inside a round: its tiles are parked, release the finishers
    e("s_waitcnt lgkmcnt(0)")
    e("s_barrier")
    e("9:")
    return e.lines, dict(KW=KW, R=R, PP=PP, RB=RB, RED=RED, FLAG=FLAG, RED_SLOTS=RED_SLOTS, NS=NSH)


# (KW, front waves, ring size): 4 front waves -> 12 waves per workgroup, 168 VGPRs each;
# 8 front waves -> 16 waves, 128 VGPRs each.
CONFIGS = [(2, 4, 26), (4, 4, 26), (5, 4, 33), (8, 4, 26),
           (2, 8, 13), (4, 8, 13), (5, 8, 22), (8, 8, 13), (10, 8, int(os.environ.get("RWKV_BACK_R_WIDE", "26")))]


def main():
    out = []
    w = out.append
    w("// Generated by gen_decode_back.py - do not edit.  One asm statement per kernel width: the program")
    w("// of a weight-streaming wave of the single-token kernel (see the generator for the register map).")
    w("template <int KW, int FW> struct BackCfg;")
    w("template <int KW, int FW> struct BackCfgH;      // with helper workgroups: no ffn key tiles")
    for KW, FW, R, HELP in [c + (False,) for c in CONFIGS] + [(5, 8, R_HELP, True)]:
        NV = 168 if FW == 4 else 128
        clob = ", ".join(f'"v{i}"' for i in range(V_APC, NV)) + ", " + ", ".join(f'"s{i}"' for i in range(S_CUR, 102 if KW > 8 else 100))
        tiles_per_body = R // math.gcd(R, KW)
        NSH = max(d for d in range(1, 5) if tiles_per_body % d == 0)     # head tiles per barrier round
        lines, info = gen(KW, R, NV, NSH, HELP)
        w(f"template <> struct BackCfg{'H' if HELP else ''}<{KW}, {FW}> {{")
        w(f"    static constexpr int R = {R}, RED = {info['RED']}, FLAG = {info['FLAG']}, RED_SLOTS = {info['RED_SLOTS']}, NS = {info['NS']};")
        w("    static __device__ __forceinline__ void run(const unsigned long long *jt, const uint8_t *wh, int L, int hr, int vt,")
        w("                                                int g, int wb, unsigned lds) {")
        w("        const unsigned whlo = (unsigned)(unsigned long long)(uintptr_t)wh;")
        w("        const unsigned whhi = (unsigned)((unsigned long long)(uintptr_t)wh >> 32);")
        w("        asm volatile(")
        for ln in lines:
            w(f'            "{ln}\\n"')
        w('            :')
        w('            : [jt] "s"(jt), [wh] "s"(wh), [whlo] "s"(whlo), [whhi] "s"(whhi), [L] "s"(L), [hr] "s"(hr), [vt] "s"(vt),')
        w('              [g] "s"(g), [wb] "s"(wb), [lds] "s"(lds)')
        w(f'            : "memory", "scc", "vcc", {clob});')
        w("    }")
        w("};")
    sys.stdout.write("\n".join(out) + "\n")


if __name__ == "__main__":
    main()
