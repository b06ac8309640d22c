#!/usr/bin/env python3
"""Generates gemm256_loop.inc: the hand-scheduled main loop of the 256x256 GEMM
kernel for gfx950 as inline assembly with a fixed register map.

One workgroup = 4 waves (one per SIMD); each wave owns a 128x128 sub-tile =
4x4 v_mfma_f32_32x32x16 accumulators = all 256 AGPRs.  With a single wave per
SIMD nothing hides a stall except the wave's own instruction stream, so the
order of every instruction is fixed here instead of being left to the compiler.

K is consumed in stages of 32 (two k-steps of 16).  LDS holds a ring of five stage
buffers (32 KB each: A tile 16 KB, B tile 16 KB) that is filled by buffer loads
that write LDS directly (no staging registers, no LDS store instructions).
Fragments are read from LDS two k-steps (= one stage) before the MFMAs that use
them, into a rotation of four fragment register sets, so a wait for fragments
never follows their reads closely.  Stage t (buffer t % 5):

  k-step 0 : 16 MFMAs; reads of stage t+1 k-step 0 fragments;
             second half of the loads triggered by the previous stage's barrier
  wait: k-step 1 fragments there (= all own reads of buffer t % 5 done), own
        loads of stage t+2 landed;  workgroup barrier (buffer t % 5 is free)
  k-step 1 : 16 MFMAs; reads of stage t+1 k-step 1 fragments;
             first half of the loads this barrier triggers:
               operand with k as the slow axis: stage t+5 into buffer t % 5;
               operand with k contiguous, t even: stages t+4 AND t+5 together.
A stage of a k-contiguous operand is 64 bytes of each row = half a cache line; asking
for both halves in adjacent instructions fetches every line from L2 once instead of
twice (the L2 -> L1 fill path, 64 bytes per clock per CU, is what the loop is
short of).

Register map (VGPR):
  fragment set n (n = 0..3, k-step 2t+s uses set (2t+s) % 4):
      A fragments v[32n : 32n+15], B fragments v[32n+16 : 32n+31]
  v[192:203] A fragment read addresses, v[204:215] B fragment read addresses
      (k-contiguous operand: element 2h + s = k-step s, ring buffers 2h and 2h+1;
       other operand: element 4h + j = mn block j, ring buffers 2h and 2h+1)
  v216 / v217 A / B global byte offset of this thread's 16-byte chunk,
  v218 / v219 the same + 64 (second half line of a k-contiguous operand)
AGPR: accumulator (i, j) = a[16*(4*i+j) : +15]
SGPR: s[72:74] = 1..3 x A pass stride, s[76:78] = 1..3 x B pass stride, s80 = stage counter,
      s81 = caller's M0 (restored at the end)

An operand is either "K" (k is the contiguous axis in memory: stage tile stored
[256 rows][32 k], fragments read with ds_read_b128) or "MN" (k is the slow axis:
tile stored as it lies, [32 k][256 mn], fragments transposed on the way out with
ds_read_b64_tr_b16).

The family of tiles: B width 256 or 128 columns (rows are always 256) x ring depth 4, 5 or 6.
A member is emitted only when it passes the validity filter (`valid`): its ring fits the
160 KB of LDS of a compute unit, and accumulators plus fragment and address registers fit the
512 registers of a wave.  Ring depth D changes the prefetch distance (loads of stage t+D are
triggered by the barrier of stage t) and the unrolling (a multiple of D and of 2).  The
descriptions above are written for depth 5.

Run:  python3 gen_gemm256_loop.py > gemm256_loop.inc
      python3 gen_gemm256_loop.py two_set > gemm_twoset_loop.inc      (the members on two fragment sets, below)
"""
NST = 5               # ring stages (set per emitted function, like BW)
UNROLL = 10           # stages per loop body: lcm(ring, pair issue, fragment set rotation)
LDS_BYTES = 160 * 1024
WAVE_REGISTERS = 512
OPER = 16384          # bytes of the A tile (256 rows x 32 k); the B tile follows it in a stage buffer
# Set per emitted function: the B tile is 256 or 128 columns wide.  The narrow form gives a
# 256x128 workgroup tile (each wave 128x64 = 4x2 accumulators, 128 AGPRs) for problems
# whose 256x256 tiling leaves compute units idle.
BW = 256              # B tile width
NBF = 4               # B fragments (32 columns each) per wave = BW / 64
STAGE = 32768         # bytes per stage buffer = OPER + BW * 64


def configure(bw, ring=5):
    global BW, NBF, STAGE, NST, UNROLL
    BW, NBF, STAGE = bw, bw // 64, OPER + bw * 64
    NST = ring
    UNROLL = ring if ring % 2 == 0 else 2 * ring


def valid(bw, ring):
    """The validity filter of the tile family: LDS for the ring and for the epilogue's staging, which
    reuses it (four waves x 128 rows x (bw + 16) bytes), and registers (accumulators in AGPRs; four fragment sets, read addresses for up to six ring
    buffers, load offsets)."""
    lds = max(ring * (OPER + bw * 64), 4 * 128 * (bw + 16))     # the ring, or the epilogue's staging area in its place
    accumulators = 4 * (bw // 64) * 16
    vgprs = 4 * (16 + 4 * (bw // 64)) + 24 + 4
    return 2 <= ring <= 6 and lds <= LDS_BYTES and accumulators <= 256 and accumulators + vgprs <= WAVE_REGISTERS

SET = {n: (32 * n, 32 * n + 16) for n in range(4)}   # fragment set -> (A base vgpr, B base vgpr)
RA, RB = 192, 204
GOFF = {"A": 216, "B": 217}
GOFF2 = {"A": 218, "B": 219}
SP = {"A": 72, "B": 76}
ST = 80


def vr(base, n):
    return f"v[{base}:{base + n - 1}]"


def frag_reads(kind, which, g, s, fset):
    """LDS reads of the 4 fragments of k-step `s` of operand `which` from ring buffer `g`."""
    base = SET[fset][0 if which == "A" else 1]
    addr = RA if which == "A" else RB
    h, lo = g >> 1, (g & 1) * STAGE
    out = []
    rowb = 512 if which == "A" else 2 * BW      # bytes per k-row of an MN tile
    for j in range(4 if which == "A" else NBF):
        dst = base + 4 * j
        if kind == "K":
            out.append(f"ds_read_b128 {vr(dst, 4)}, v{addr + 2 * h + s} offset:{lo + j * 2048}")
        else:
            off = lo + s * 16 * rowb
            out.append(f"ds_read_b64_tr_b16 {vr(dst, 2)}, v{addr + 4 * h + j} offset:{off}")
            out.append(f"ds_read_b64_tr_b16 {vr(dst + 2, 2)}, v{addr + 4 * h + j} offset:{off + 4 * rowb}")
    return out


def all_frag_reads(kinds, g, s, fset):
    a, b = frag_reads(kinds["A"], "A", g, s, fset), frag_reads(kinds["B"], "B", g, s, fset)
    out = []
    for i in range(max(len(a), len(b))):
        out += a[i:i + 1] + b[i:i + 1]
    return out


def load_instr(which, stage, p, second_half=False):
    """One direct-to-LDS load (kept together with its M0 set-up) of pass `p` of `stage`:
    the wave's 1 KB LDS slot is M0 = wave base + buffer + operand + p * 4096."""
    g = stage % NST
    m0 = g * STAGE + (OPER if which == "B" else 0) + p * 4096
    so = "0" if p == 0 else f"s{SP[which] + p - 1}"
    voff = (GOFF2 if second_half else GOFF)[which]
    rs = "%[rsa]" if which == "A" else "%[rsb]"
    return dict(stage=stage, lines=[f"s_add_u32 m0, %[m0b], {m0}", "s_nop 0",
                                    f"buffer_load_dwordx4 v{voff}, {rs}, {so} offen lds"])


def trigger_group(kinds, t):
    """Loads triggered by the barrier of stage t (buffer t % 5 has just become free)."""
    grp = []
    for which in ("A", "B"):
        passes = 4 if which == "A" else NBF     # 4 KB (one 1 KB slot per wave) per pass
        if kinds[which] == "K":
            # stages 2m and 2m + 1 are the two halves of the same cache lines: the pair goes out
            # together, at the barrier that frees the buffer of its second stage
            if (t + NST - 1) % 2 == 0:
                for p in range(passes):
                    grp.append(load_instr(which, t + NST - 1, p))
                    grp.append(load_instr(which, t + NST, p, second_half=True))
                grp.append(dict(stage=None, lines=[f"v_add_u32 v{GOFF[which]}, 128, v{GOFF[which]}",
                                                   f"v_add_u32 v{GOFF2[which]}, 128, v{GOFF2[which]}"]))
        else:
            for p in range(passes):
                grp.append(load_instr(which, t + NST, p))
            step = "%[ta]" if which == "A" else "%[tb]"
            grp.append(dict(stage=None, lines=[f"v_add_u32 v{GOFF[which]}, {step}, v{GOFF[which]}"]))
    return grp


def halves(grp):
    n = (len(grp) + 1) // 2
    return grp[:n], grp[n:]


def mfmas(mnem, fset):
    a, b = SET[fset]
    out = []
    for i in range(4):
        # back and forth over the B fragments: consecutive MFMAs then always share one operand
        # (B when the row block changes), which leaves fewer operand lines toggling
        for j in (range(NBF) if i % 2 == 0 else reversed(range(NBF))):
            acc = 16 * (NBF * i + j)
            # (B, A): the accumulator tile comes out transposed (lane = row m)
            out.append(f"{mnem} a[{acc}:{acc + 15}], {vr(b + 4 * j, 4)}, {vr(a + 4 * i, 4)}, a[{acc}:{acc + 15}]")
    return out


def interleave(main, reads, loads):
    """Fragment reads behind the first four MFMAs of a k-step (they are not needed before
    the k-step after the next), loads spread evenly over the k-step.  `loads` are dicts
    whose lines stay together."""
    per = (len(reads) + 3) // 4
    every = max(1, len(main) // max(len(loads), 1))
    out, kl = [], 0
    for idx, m in enumerate(main):
        out.append(m)
        if idx < 4:
            out += reads[idx * per:(idx + 1) * per]
        if kl < len(loads) and idx % every == 0:
            out += loads[kl]["lines"]
            kl += 1
    for ld in loads[kl:]:
        out += ld["lines"]
    return out


class Tracker:
    """Program-order list of issued loads, to size the vmcnt waits: a wait in front of the
    barrier of stage t needs every load of stages <= t+2 landed, i.e. may leave
    outstanding only the loads issued after the last of those."""

    def __init__(self):
        self.order = []

    def issue(self, loads):
        for ld in loads:
            if ld["stage"] is not None:
                self.order.append(ld["stage"])

    def allowed(self, need_stage):
        last = max(i for i, s in enumerate(self.order) if s <= need_stage)
        return len(self.order) - 1 - last


def simulate(kinds):
    """vmcnt for the barrier of each body position (minimum over the first iterations and
    the steady state) and for the prologue."""
    tr = Tracker()
    for t in range(-NST, -1):
        tr.issue(trigger_group(kinds, t))
    first, second = halves(trigger_group(kinds, -1))
    tr.issue(first)
    pro = tr.allowed(1)
    pending = second
    counts = {}
    for t in range(4 * UNROLL):
        tr.issue(pending)                       # k-step 0
        c = tr.allowed(t + 2)
        counts[t % UNROLL] = min(counts.get(t % UNROLL, 63), c)
        first, pending = halves(trigger_group(kinds, t))
        tr.issue(first)                         # k-step 1
    return pro, counts


def stage_iteration(mnem, kinds, t, vmcnt, extra=(), extra_mid=()):
    g, nxt = t % NST, (t + 1) % NST
    r0 = all_frag_reads(kinds, nxt, 0, (2 * t + 2) % 4)
    r1 = all_frag_reads(kinds, nxt, 1, (2 * t + 3) % 4)
    _, prev_second = halves(trigger_group(kinds, t - 1))
    this_first, _ = halves(trigger_group(kinds, t))
    out = []
    # k-step 0: its fragments were read one stage ago; only the previous k-step's reads
    # (LDS operations retire in order) may still be outstanding
    out.append(f"s_waitcnt lgkmcnt({min(len(r1), 15)})")
    out += list(extra)      # older than every fragment read of this stage: the waits below cover them
    out += interleave(mfmas(mnem, (2 * t) % 4), r0, prev_second)
    # k-step 1
    out.append(f"s_waitcnt vmcnt({min(vmcnt, 63)}) lgkmcnt({min(len(r0), 15)})")
    out.append("s_barrier")
    out += list(extra_mid)
    out += interleave(mfmas(mnem, (2 * t + 1) % 4), r1, this_first)
    return out


def body(mnem, kinds):
    pro_vmcnt, vmcnts = simulate(kinds)
    out = []
    for r in range(64 * NBF):
        out.append(f"v_accvgpr_write_b32 a{r}, 0")
    for which, pin in (("A", "%[pa]"), ("B", "%[pb]")):
        for i in range(1, 4):
            out.append(f"s_mul_i32 s{SP[which] + i - 1}, {pin}, {i}")
    out.append(f"s_mov_b32 s{ST}, 0")
    out.append(f"s_mov_b32 s{ST + 1}, m0")
    # fragment read addresses of ring buffers 2..4 from those of buffers 0 and 1
    for which, base in (("A", RA), ("B", RB)):
        n = 2 if kinds[which] == "K" else 4
        for h in (1, 2):
            for e in range(n):
                out.append(f"v_add_u32 v{base + n * h + e}, {h * 2 * STAGE}, v{base + e}")
        out.append(f"v_add_u32 v{GOFF2[which]}, 64, v{GOFF[which]}")
    # the loads the barriers of stages -5 .. -1 would have triggered
    for t in range(-NST, -1):
        for ld in trigger_group(kinds, t):
            out += ld["lines"]
    first, _ = halves(trigger_group(kinds, -1))
    for ld in first:
        out += ld["lines"]
    out.append(f"s_waitcnt vmcnt({pro_vmcnt})")           # stages 0 and 1 landed
    out.append("s_barrier")
    out += all_frag_reads(kinds, 0, 0, 0)
    out += all_frag_reads(kinds, 0, 1, 1)
    out.append("s_waitcnt lgkmcnt(0)")
    out.append("L_gemm256_loop_%=:")
    for t in range(UNROLL):
        out += stage_iteration(mnem, kinds, t, vmcnts[t])
        out.append(f"s_add_u32 s{ST}, s{ST}, 1")
        if t < UNROLL - 1:
            out.append(f"s_cmp_ge_u32 s{ST}, %[kt]")
            out.append("s_cbranch_scc1 L_gemm256_done_%=")
        else:
            out.append(f"s_cmp_lt_u32 s{ST}, %[kt]")
            out.append("s_cbranch_scc1 L_gemm256_loop_%=")
    out.append("L_gemm256_done_%=:")
    # drain: loads of stages past the end still write LDS, which the caller reuses;
    # the last MFMA results must be readable by ordinary instructions
    out.append("s_waitcnt vmcnt(0) lgkmcnt(0)")
    out.append("s_barrier")
    out.append(f"s_mov_b32 m0, s{ST + 1}")
    out += ["s_nop 15", "s_nop 15"]
    return out


# ---- streamed tiles ------------------------------------------------------------------------------
# A persistent workgroup of the 256x128 kernel runs tile after tile.  From its second tile on, the
# loop below also stores the PREVIOUS tile, which the caller hands over as packed 16-bit values in
# v[128:191] (accumulator block i, 8-byte group c = 4 j + q at v[128 + 16 i + 2 c : +1]: row
# 32 i + (lane & 31), columns 8 c + 4 (lane >> 5) .. + 3 of the wave's 128x64 sub-tile).  The first
# 16 stages carry it, one 32-row block per four stages, through a 4 KB transposition area per wave:
#   stage 4i   : eight ds_write_b64 (row = 128 bytes, 16-byte chunk c at position c ^ ((row >> 1) & 7))
#   stage 4i+1 : four ds_read_b128, lane l <- row 8 p + l / 8, position l % 8
#   stage 4i+2 : four global_store_dwordx4 of 8 rows x 128 bytes each, right behind the barrier: an
#                even stage's wait is the tight one (it leaves only the youngest loads outstanding and
#                would have to sit out a store still in flight), and from there the next one is two
#                stages away
# The prologue (the loads of the first stages, and the tile's 128 bias values straight into LDS) is a
# function of its own, so that the caller can issue it BEFORE it converts the previous accumulators:
# the load latency then hides behind that conversion.  The caller must issue no vector memory
# instruction between the two functions (the waits below count the prologue's loads).
# Extra registers: v[220:235] chunk temporaries, v236 transposition write address (this lane's row,
# chunk 0), v237 read address, v238 / v239 byte offset into C of this lane's chunk for even / odd
# p, v[240:247] write addresses of the eight chunks, s[82:83] running row pointer into C.
STRAIGHT = 20         # stages emitted straight-line at the start of a streamed tile (2 x UNROLL)
XSTAGES = 16          # the first 16 of them carry the previous tile
PK, TMP, XA, WA, SC = 128, 220, 236, 240, 82


def stream_extras(t):
    """(lines in front of the stage's first MFMA, lines behind its barrier)"""
    i, ph = divmod(t, 4)
    first, mid = [], []
    if ph == 0:
        for c in range(8):
            r = PK + 16 * i + 2 * c
            first.append(f"ds_write_b64 v{WA + c}, v[{r}:{r + 1}]")
    elif ph == 1:
        for p in range(4):
            first.append(f"ds_read_b128 {vr(TMP + 4 * p, 4)}, v{XA + 1} offset:{p * 1024}")
    elif ph == 2:
        for p in range(4):
            # ordinary stores: with the streaming hint (nt) this kernel gained up to 7 %, but the next
            # kernel, which reads C, lost more than that (GPT-2 FFN-down after FFN-up: 54 -> 67 us)
            mid.append(f"global_store_dwordx4 v{XA + 2 + (p & 1)}, {vr(TMP + 4 * p, 4)}, s[{SC}:{SC + 1}]")
            mid.append(f"s_add_u32 s{SC}, s{SC}, %[srow]")
            mid.append(f"s_addc_u32 s{SC + 1}, s{SC + 1}, 0")
    return first, mid


def simulate_stream(kinds):
    """vmcnt of the prologue wait and of each straight-line stage of a streamed tile.  The stores
    of the previous tile are left out of the count on purpose: a store may be acknowledged before
    an older load has landed, so a wait that allowed for them could pass too early, while a wait
    that ignores them at worst also waits for a few younger loads."""
    tr = Tracker()
    tr.order.append(-100)                       # the bias load, first of the prologue
    for t in range(-NST, -1):
        tr.issue(trigger_group(kinds, t))
    first, pending = halves(trigger_group(kinds, -1))
    tr.issue(first)
    pro = tr.allowed(1)
    counts = []
    for t in range(STRAIGHT):
        tr.issue(pending)
        counts.append(tr.allowed(t + 2))
        first, pending = halves(trigger_group(kinds, t))
        tr.issue(first)
    return pro, counts


def stream_prologue(kinds):
    out = [f"s_mov_b32 s{ST + 1}, m0"]
    for which, pin in (("A", "%[pa]"), ("B", "%[pb]")):
        for i in range(1, 4):
            out.append(f"s_mul_i32 s{SP[which] + i - 1}, {pin}, {i}")
        out.append(f"v_add_u32 v{GOFF2[which]}, 64, v{GOFF[which]}")
    out += ["s_mov_b32 m0, %[m0bias]", "s_nop 0", "buffer_load_dword %[vbias], %[rsbias], 0 offen lds"]
    for t in range(-NST, -1):
        for ld in trigger_group(kinds, t):
            out += ld["lines"]
    first, _ = halves(trigger_group(kinds, -1))
    for ld in first:
        out += ld["lines"]
    out.append(f"s_mov_b32 m0, s{ST + 1}")
    return out


def stream_body(mnem, kinds):
    pro_vmcnt, straight = simulate_stream(kinds)
    _, vmcnts = simulate(kinds)
    out = [f"s_mov_b32 s{ST + 1}, m0"]
    for r in range(64 * NBF):
        out.append(f"v_accvgpr_write_b32 a{r}, 0")
    for which, pin in (("A", "%[pa]"), ("B", "%[pb]")):
        for i in range(1, 4):
            out.append(f"s_mul_i32 s{SP[which] + i - 1}, {pin}, {i}")
    for which, base in (("A", RA), ("B", RB)):
        n = 2 if kinds[which] == "K" else 4
        for h in (1, 2):
            for e in range(n):
                out.append(f"v_add_u32 v{base + n * h + e}, {h * 2 * STAGE}, v{base + e}")
        out.append(f"v_add_u32 v{GOFF2[which]}, 64, v{GOFF[which]}")
    for c in range(8):
        out.append(f"v_xor_b32 v{WA + c}, {16 * c}, v{XA}")
    out.append(f"s_mov_b64 s[{SC}:{SC + 1}], %[cptr]")
    out.append(f"s_waitcnt vmcnt({pro_vmcnt})")           # stages 0 and 1 landed
    out.append("s_barrier")
    out += all_frag_reads(kinds, 0, 0, 0)
    out += all_frag_reads(kinds, 0, 1, 1)
    out.append("s_waitcnt lgkmcnt(0)")
    for t in range(STRAIGHT):
        first, mid = stream_extras(t) if t < XSTAGES else ((), ())
        out += stage_iteration(mnem, kinds, t, straight[t], first, mid)
    out.append(f"s_mov_b32 s{ST}, {STRAIGHT}")
    out.append(f"s_cmp_ge_u32 s{ST}, %[kt]")
    out.append("s_cbranch_scc1 L_gemm256_done_%=")
    out.append("L_gemm256_loop_%=:")
    for t in range(UNROLL):
        out += stage_iteration(mnem, kinds, STRAIGHT + t, vmcnts[t])
        out.append(f"s_add_u32 s{ST}, s{ST}, 1")
        if t < UNROLL - 1:
            out.append(f"s_cmp_ge_u32 s{ST}, %[kt]")
            out.append("s_cbranch_scc1 L_gemm256_done_%=")
        else:
            out.append(f"s_cmp_lt_u32 s{ST}, %[kt]")
            out.append("s_cbranch_scc1 L_gemm256_loop_%=")
    out.append("L_gemm256_done_%=:")
    out.append("s_waitcnt vmcnt(0) lgkmcnt(0)")
    out.append("s_barrier")
    out.append(f"s_mov_b32 m0, s{ST + 1}")
    out += ["s_nop 15", "s_nop 15"]
    return out


def emit_stream(name, mnem, ka, kb):
    kinds = {"A": ka, "B": kb}
    print(f"// {name}_prologue: loads of the first stages of a streamed tile and its bias values")
    print(f"__device__ __forceinline__ void {name}_prologue(u32x2& goff, __amdgpu_buffer_rsrc_t rsa,")
    print("        __amdgpu_buffer_rsrc_t rsb, uint32_t pa, uint32_t pb, uint32_t ta, uint32_t tb, uint32_t m0b,")
    print("        __amdgpu_buffer_rsrc_t rsbias, uint32_t m0bias, uint32_t vbias) {")
    print("    asm volatile(")
    for ln in stream_prologue(kinds):
        print(f'        "{ln}\\n"')
    print(f'        : "+{{v[{GOFF["A"]}:{GOFF["B"]}]}}"(goff)')
    print('        : [rsa] "s"(rsa), [rsb] "s"(rsb), [pa] "s"(pa), [pb] "s"(pb), [ta] "s"(ta), [tb] "s"(tb),')
    print('          [m0b] "s"(m0b), [rsbias] "s"(rsbias), [m0bias] "s"(m0bias), [vbias] "v"(vbias)')
    clob = [f'"v{GOFF2["A"]}"', f'"v{GOFF2["B"]}"'] + [f'"s{i}"' for i in range(SP["A"], ST + 2)] + ['"scc"', '"memory"']
    print("        : " + ", ".join(clob) + ");")
    print("}\n")
    print(f"// {name}: main loop of a streamed tile ({mnem}); stores the previous tile on the way")
    print(f"__device__ __forceinline__ void {name}(f32x16 (&acc)[{4 * NBF}], u32x4& ra, u32x4& rb, u32x2& goff,")
    print("        __amdgpu_buffer_rsrc_t rsa, __amdgpu_buffer_rsrc_t rsb, uint32_t pa, uint32_t pb,")
    print("        uint32_t ta, uint32_t tb, uint32_t m0b, uint32_t kt, const u32x16 (&pk)[4], u32x4 xaddr,")
    print("        uint64_t cptr, uint32_t srow) {")
    print("    asm volatile(")
    for ln in stream_body(mnem, kinds):
        print(f'        "{ln}\\n"')
    outs = ", ".join(f'"={{a[{16 * i}:{16 * i + 15}]}}"(acc[{i}])' for i in range(4 * NBF))
    print(f"        : {outs},")
    print(f'          "+{{v[{GOFF["A"]}:{GOFF["B"]}]}}"(goff), "+{{v[{RA}:{RA + 3}]}}"(ra), "+{{v[{RB}:{RB + 3}]}}"(rb)')
    print('        : [rsa] "s"(rsa), [rsb] "s"(rsb), [pa] "s"(pa), [pb] "s"(pb), [ta] "s"(ta), [tb] "s"(tb),')
    print('          [m0b] "s"(m0b), [kt] "s"(kt),')
    pks = ", ".join(f'"{{v[{PK + 16 * i}:{PK + 16 * i + 15}]}}"(pk[{i}])' for i in range(4))
    print(f"          {pks},")
    print(f'          "{{v[{XA}:{XA + 3}]}}"(xaddr), [cptr] "s"(cptr), [srow] "s"(srow)')
    vclob = (list(range(128)) + list(range(RA + 4, RB)) + list(range(RB + 4, GOFF["A"])) + [GOFF2["A"], GOFF2["B"]]
             + list(range(TMP, TMP + 16)) + list(range(WA, WA + 8)))
    clob = ([f'"v{i}"' for i in vclob] + [f'"s{i}"' for i in range(SP["A"], ST + 2)] + [f'"s{SC}"', f'"s{SC + 1}"']
            + ['"scc"', '"memory"'])
    print("        : " + ", ".join(clob) + ");")
    print("}\n")


def emit(name, mnem, ka, kb):
    lines = body(mnem, {"A": ka, "B": kb})
    print(f"// {name}: A operand {ka}-major, B operand {kb}-major, {mnem}")
    print(f"__device__ __forceinline__ void {name}(f32x16 (&acc)[{4 * NBF}], u32x4& ra, u32x4& rb, u32x2& goff,")
    print("        __amdgpu_buffer_rsrc_t rsa, __amdgpu_buffer_rsrc_t rsb, uint32_t pa, uint32_t pb,")
    print("        uint32_t ta, uint32_t tb, uint32_t m0b, uint32_t kt) {")
    print("    asm volatile(")
    for ln in lines:
        print(f'        "{ln}\\n"')
    outs = ", ".join(f'"={{a[{16 * i}:{16 * i + 15}]}}"(acc[{i}])' for i in range(4 * NBF))
    print(f"        : {outs},")
    # ra / rb are written too: the addresses of the other ring buffers of a k-contiguous operand
    # are derived into their upper elements
    print(f'          "+{{v[{GOFF["A"]}:{GOFF["B"]}]}}"(goff), "+{{v[{RA}:{RA + 3}]}}"(ra), "+{{v[{RB}:{RB + 3}]}}"(rb)')
    print('        : [rsa] "s"(rsa), [rsb] "s"(rsb), [pa] "s"(pa), [pb] "s"(pb), [ta] "s"(ta), [tb] "s"(tb),')
    print('          [m0b] "s"(m0b), [kt] "s"(kt)')
    vclob = list(range(128)) + list(range(RA + 4, RB)) + list(range(RB + 4, GOFF["A"])) + [GOFF2["A"], GOFF2["B"]]
    clob = [f'"v{i}"' for i in vclob] + [f'"s{i}"' for i in range(SP["A"], ST + 2)] + ['"scc"', '"memory"']
    print("        : " + ", ".join(clob) + ");")
    print("}\n")


# ---- the 256x384 tile ----------------------------------------------------------------------------
# The widest member: 256 rows x 384 columns per workgroup, each wave 128 x 192 = 4 x 6 accumulator
# blocks = 384 registers, the first sixteen blocks in the AGPRs, the last eight in v[128:255].  It
# moves 17 % fewer bytes from the L2s to LDS per FLOP than the 256x256 tile, which is what a GEMM
# with short K whose operands come from memory is short of.  What it costs:
#   * two fragment sets instead of four (k-step s of every stage uses set s): the fragments of a
#     k-step are read during the k-step before it, 24 MFMAs = 768 cycles ahead;
#   * a stage is 40 KB -- [A 16 KB][B 16 KB][B2 8 KB] -- and the ring four stages deep (160 KB);
#     stage t+4 is asked for behind the barrier of stage t and must have landed at the barrier of
#     stage t+3 (the reads of buffer t+1 start behind the barrier of stage t).
# B is kept as the 256-column tile of the wide kernel followed by the 128-column tile of the narrow
# one (B2: columns 256..383 of the workgroup's 384), each in its own layout, so that loads, LDS
# layouts and fragment addresses are those of the two existing kernels; wave (wm, wn) owns columns
# 128 wn .. + 127 of B (blocks j = 0..3) and 64 wn .. + 63 of B2 (j = 4, 5).
#
# Register map (VGPR): fragment set n: A v[40n : 40n+15], B v[40n+16 : 40n+31], B2 v[40n+32 : 40n+39];
#   v[80:87] A read addresses, v[88:95] B, v[96:99] B2 (k-contiguous: element 2h + s; other: (blocks
#   per wave) h + j; ring buffers 2h and 2h+1); v100 / v101 / v102 global byte offsets of this thread's
#   chunk of A / B / B2, v103 / v104 / v105 the same + 64; v[128:255] accumulator blocks 16..23.
# AGPR: accumulator block b = 6 i + j < 16 at a[16 b : +15].
# SGPR: as above (s[72:74] A pass strides, s[76:78] B pass strides, s80 stage counter, s81 caller's M0).
#
# The same two-set schedule serves a second member, the 256x128 tile for two workgroups per compute
# unit: all of its registers below v64 and a[0:127] (256 registers per wave), a ring of three 24 KB
# stages (72 KB), so that two workgroups share a compute unit and one's prologue, epilogue and load
# latency run under the other's MFMAs.  Register map: fragment set n: A v[24n : 24n+15], B
# v[24n+16 : 24n+23]; v[48:55] A read addresses, v[56:59] B; v60 / v61 global offsets, v62 / v63 the
# same + 64; accumulator (i, j) at a[16 (2 i + j) : +15] as in the one-workgroup kernel.
# Two more members, described where they are defined: the 128x192 tile (`_x192`) and the 256x288
# tile (`_x288`).
class TwoSet:
    """One member of the two-fragment-set family: geometry and register map."""

    def __init__(self, name, nst, ops, region, sets, raddr, goff, goff2, blocks, passes, rowb, passmult,
                 acc_regs, grid, goff_span, clobber_to, stage=None, a_blocks=4, mn_fold=None):
        self.name, self.nst, self.ops = name, nst, ops
        # (`passes` of an operand: a number, or one per layout {"K": .., "MN": ..})
        self.stage = stage if stage else sum(passes[o] * 4096 for o in ops)
        self.a_blocks = a_blocks          # 32-row blocks of A per wave
        # An operand in the 256-column layout of which a wave reads more than four blocks: block j
        # uses the address register of block j % 4 and an offset of 256 bytes per four blocks (the
        # swizzle of that layout only touches the two low bits of the block index).
        self.mn_fold = mn_fold or {}
        self.unroll = nst if nst % 2 == 0 else 2 * nst
        self.region, self.sets, self.raddr, self.goff, self.goff2 = region, sets, raddr, goff, goff2
        self.blocks, self.passes, self.rowb, self.passmult = blocks, passes, rowb, passmult
        self.acc_regs = acc_regs          # block index -> register range text
        self.grid = grid                  # (accumulator block, B operand, its block, A block) per MFMA of a k-step
        self.goff_span = goff_span        # registers of the global-offset operand handed in by the caller
        self.clobber_to = clobber_to      # fragment registers v0 .. clobber_to - 1


def _x384():
    def acc(b):
        return f"a[{16 * b}:{16 * b + 15}]" if b < 16 else vr(128 + 16 * (b - 16), 16)
    # (back and forth over the B fragments, as in `mfmas`)
    grid = [(6 * i + j, "B" if j < 4 else "B2", j if j < 4 else j - 4, i)
            for i in range(4) for j in (range(6) if i % 2 == 0 else reversed(range(6)))]
    return TwoSet("384", 4, ("A", "B", "B2"), {"A": 0, "B": 16384, "B2": 32768},
                  {0: {"A": 0, "B": 16, "B2": 32}, 1: {"A": 40, "B": 56, "B2": 72}},
                  {"A": 80, "B": 88, "B2": 96}, {"A": 100, "B": 101, "B2": 102}, {"A": 103, "B": 104, "B2": 105},
                  {"A": 4, "B": 4, "B2": 2}, {"A": 4, "B": 4, "B2": 2}, {"A": 512, "B": 512, "B2": 256},
                  {"B2": 2}, [acc(b) for b in range(24)], grid, 4, 80)


def _xpair():
    grid = [(2 * i + j, "B", j, i) for i in range(4) for j in (range(2) if i % 2 == 0 else reversed(range(2)))]
    return TwoSet("pair", 3, ("A", "B"), {"A": 0, "B": 16384},
                  {0: {"A": 0, "B": 16}, 1: {"A": 24, "B": 40}},
                  {"A": 48, "B": 56}, {"A": 60, "B": 61}, {"A": 62, "B": 63},
                  {"A": 4, "B": 2}, {"A": 4, "B": 2}, {"A": 512, "B": 256},
                  {}, [f"a[{16 * b}:{16 * b + 15}]" for b in range(8)], grid, 2, 48)


def _x192():
    """128 x 192 tile: each wave 64 x 96 = 2 x 3 accumulator blocks in a[0:95]; A is 128 rows, B 192
    columns held in the 256-column layout of the wide kernel (its last quarter is never asked
    for); a stage is 24 KB, the ring six deep.  Register map: fragment set n: A v[20n : 20n+7], B
    v[20n+8 : 20n+19]; v[40:45] A read addresses, v[48:56] B; v60 / v61 global offsets, v62 / v63
    the same + 64."""
    grid = [(3 * i + j, "B", j, i) for i in range(2) for j in (range(3) if i % 2 == 0 else reversed(range(3)))]
    return TwoSet("x192", 6, ("A", "B"), {"A": 0, "B": 8192},
                  {0: {"A": 0, "B": 8}, 1: {"A": 20, "B": 28}},
                  {"A": 40, "B": 48}, {"A": 60, "B": 61}, {"A": 62, "B": 63},
                  {"A": 2, "B": 3}, {"A": 2, "B": {"K": 3, "MN": 4}}, {"A": 256, "B": 512},
                  {}, [f"a[{16 * b}:{16 * b + 15}]" for b in range(6)], grid, 2, 40, stage=24576, a_blocks=2)


def _x288():
    """256 x 288 tile: four waves one above the other, each 64 x 288 = 2 x 9 accumulator blocks, the
    first sixteen in a[0:255] and the last two in v[128:159].  Every wave reads all of B: its 256-column
    tile (eight blocks) and the first block of the 128-column tile behind it (columns 256..287; the
    rest of that tile is never loaded).  Register map: fragment set n: A v[44n : 44n+7], B
    v[44n+8 : 44n+39], B2 v[44n+40 : 44n+43]; v[88:91] A read addresses, v[92:99] B, v[100:103] B2;
    v104 / v105 / v106 global offsets, v107 / v108 / v109 the same + 64."""
    def acc(b):
        return f"a[{16 * b}:{16 * b + 15}]" if b < 16 else vr(128 + 16 * (b - 16), 16)
    grid = [(9 * i + j, "B" if j < 8 else "B2", j if j < 8 else 0, i)
            for i in range(2) for j in (range(9) if i % 2 == 0 else reversed(range(9)))]
    return TwoSet("x288", 4, ("A", "B", "B2"), {"A": 0, "B": 16384, "B2": 32768},
                  {0: {"A": 0, "B": 8, "B2": 40}, 1: {"A": 44, "B": 52, "B2": 84}},
                  {"A": 88, "B": 92, "B2": 100}, {"A": 104, "B": 105, "B2": 106}, {"A": 107, "B": 108, "B2": 109},
                  {"A": 2, "B": 8, "B2": 1}, {"A": 4, "B": 4, "B2": {"K": 1, "MN": 2}}, {"A": 512, "B": 512, "B2": 256},
                  {"B2": 2}, [acc(b) for b in range(18)], grid, 4, 88, stage=40960, a_blocks=2, mn_fold={"B": 4})


X = None      # the member being emitted


def x_addr_regs(kinds, which):
    """Fragment address registers of an operand per pair of ring buffers."""
    if x_kind(kinds, which) == "K":
        return 2
    return min(X.blocks[which], X.mn_fold.get(which, X.blocks[which]))


def x_passes(kinds, which):
    p = X.passes[which]
    return p[x_kind(kinds, which)] if isinstance(p, dict) else p


def x_kind(kinds, which):
    return kinds["B" if which == "B2" else which]


def x_frag_reads(kinds, g, s, fset):
    per = {}
    for which in X.ops:
        kind, base, addr = x_kind(kinds, which), X.sets[fset][which], X.raddr[which]
        h, lo = g >> 1, (g & 1) * X.stage
        out = []
        for j in range(X.blocks[which]):
            dst = base + 4 * j
            if kind == "K":
                out.append(f"ds_read_b128 {vr(dst, 4)}, v{addr + 2 * h + s} offset:{lo + j * 2048}")
            else:
                fold = X.mn_fold.get(which, X.blocks[which])
                off = lo + s * 16 * X.rowb[which] + (j // fold) * 256
                a = addr + min(X.blocks[which], fold) * h + j % fold
                out.append(f"ds_read_b64_tr_b16 {vr(dst, 2)}, v{a} offset:{off}")
                out.append(f"ds_read_b64_tr_b16 {vr(dst + 2, 2)}, v{a} offset:{off + 4 * X.rowb[which]}")
        per[which] = out
    out = []
    for i in range(max(len(v) for v in per.values())):
        for which in X.ops:
            out += per[which][i:i + 1]
    return out


def x_load(kinds, which, stage, p, second_half=False):
    g = stage % X.nst
    m0 = g * X.stage + X.region[which] + p * 4096
    sp = SP["A" if which == "A" else "B"]
    # (B2 with k as the slow axis packs four k-rows into a wave's 1 KB slot where B packs two: its
    # passes are twice as far apart)
    mult = p * (X.passmult.get(which, 1) if x_kind(kinds, which) == "MN" else 1)
    so = "0" if mult == 0 else f"s{sp + mult - 1}"
    voff = (X.goff2 if second_half else X.goff)[which]
    rs = "%[rsa]" if which == "A" else "%[rsb]"
    return dict(stage=stage, lines=[f"s_add_u32 m0, %[m0b], {m0}", "s_nop 0",
                                    f"buffer_load_dwordx4 v{voff}, {rs}, {so} offen lds"])


def x_trigger_group(kinds, t):
    """Loads triggered by the barrier of stage t (buffer t % ring has just become free)."""
    grp = []
    for which in X.ops:
        if x_kind(kinds, which) == "K":
            if (t + X.nst - 1) % 2 == 0:
                for p in range(x_passes(kinds, which)):
                    grp.append(x_load(kinds, which, t + X.nst - 1, p))
                    grp.append(x_load(kinds, which, t + X.nst, p, second_half=True))
                grp.append(dict(stage=None, lines=[f"v_add_u32 v{X.goff[which]}, 128, v{X.goff[which]}",
                                                   f"v_add_u32 v{X.goff2[which]}, 128, v{X.goff2[which]}"]))
        else:
            for p in range(x_passes(kinds, which)):
                grp.append(x_load(kinds, which, t + X.nst, p))
            step = "%[ta]" if which == "A" else "%[tb]"
            grp.append(dict(stage=None, lines=[f"v_add_u32 v{X.goff[which]}, {step}, v{X.goff[which]}"]))
    return grp


def x_mfmas(mnem, fset):
    out = []
    for acc_block, bop, bj, ai in X.grid:
        acc = X.acc_regs[acc_block]
        # (B, A): the accumulator tile comes out transposed (lane = row m)
        out.append(f"{mnem} {acc}, {vr(X.sets[fset][bop] + 4 * bj, 4)}, {vr(X.sets[fset]['A'] + 4 * ai, 4)}, {acc}")
    return out


def x_simulate(kinds):
    """vmcnt of the prologue wait (stage 0 landed) and of the barrier of each body position
    (stage t + 1 landed)."""
    tr = Tracker()
    for t in range(-X.nst, -1):
        tr.issue(x_trigger_group(kinds, t))
    first, pending = halves(x_trigger_group(kinds, -1))
    tr.issue(first)
    pro = tr.allowed(0)
    counts = {}
    for t in range(4 * X.unroll):
        tr.issue(pending)
        c = tr.allowed(t + 1)
        counts[t % X.unroll] = min(counts.get(t % X.unroll, 63), c)
        first, pending = halves(x_trigger_group(kinds, t))
        tr.issue(first)
    return pro, counts


def x_stage(mnem, kinds, t, vmcnt):
    g, nxt = t % X.nst, (t + 1) % X.nst
    r0 = x_frag_reads(kinds, g, 1, 1)          # this stage's second k-step
    r1 = x_frag_reads(kinds, nxt, 0, 0)        # the next stage's first
    _, prev_second = halves(x_trigger_group(kinds, t - 1))
    this_first, _ = halves(x_trigger_group(kinds, t))
    out = ["s_waitcnt lgkmcnt(0)"]             # set 0, read during the previous k-step
    out += interleave(x_mfmas(mnem, 0), r0, prev_second)
    # every read of buffer t % ring is back, the own loads of stage t + 1 have landed
    out.append(f"s_waitcnt vmcnt({min(vmcnt, 63)}) lgkmcnt(0)")
    out.append("s_barrier")
    out += interleave(x_mfmas(mnem, 1), r1, this_first)
    return out


def x_body(mnem, kinds):
    pro_vmcnt, vmcnts = x_simulate(kinds)
    out = []
    for regs in X.acc_regs:
        m = regs[2:-1].split(":")
        for r in range(int(m[0]), int(m[1]) + 1):
            out.append(f"v_accvgpr_write_b32 a{r}, 0" if regs[0] == "a" else f"v_mov_b32 v{r}, 0")
    for which, pin in (("A", "%[pa]"), ("B", "%[pb]")):
        for i in range(1, 4):
            out.append(f"s_mul_i32 s{SP[which] + i - 1}, {pin}, {i}")
    out.append(f"s_mov_b32 s{ST}, 0")
    out.append(f"s_mov_b32 s{ST + 1}, m0")
    # fragment read addresses of the ring's last buffer(s) from those of buffers 0 and 1
    for which in X.ops:
        n = x_addr_regs(kinds, which)
        for h in range(1, (X.nst + 1) // 2):
            for e in range(n):
                out.append(f"v_add_u32 v{X.raddr[which] + n * h + e}, {h * 2 * X.stage}, v{X.raddr[which] + e}")
        out.append(f"v_add_u32 v{X.goff2[which]}, 64, v{X.goff[which]}")
    for t in range(-X.nst, -1):
        for ld in x_trigger_group(kinds, t):
            out += ld["lines"]
    first, _ = halves(x_trigger_group(kinds, -1))
    for ld in first:
        out += ld["lines"]
    out.append(f"s_waitcnt vmcnt({pro_vmcnt})")           # stage 0 landed
    out.append("s_barrier")
    out += x_frag_reads(kinds, 0, 0, 0)
    out.append(f"L_gemm{X.name}_loop_%=:")
    for t in range(X.unroll):
        out += x_stage(mnem, kinds, t, vmcnts[t])
        out.append(f"s_add_u32 s{ST}, s{ST}, 1")
        if t < X.unroll - 1:
            out.append(f"s_cmp_ge_u32 s{ST}, %[kt]")
            out.append(f"s_cbranch_scc1 L_gemm{X.name}_done_%=")
        else:
            out.append(f"s_cmp_lt_u32 s{ST}, %[kt]")
            out.append(f"s_cbranch_scc1 L_gemm{X.name}_loop_%=")
    out.append(f"L_gemm{X.name}_done_%=:")
    out.append("s_waitcnt vmcnt(0) lgkmcnt(0)")
    out.append("s_barrier")
    out.append(f"s_mov_b32 m0, s{ST + 1}")
    out += ["s_nop 15", "s_nop 15"]
    return out


def emit_two_set(member, name, mnem, ka, kb):
    global X
    X = member
    kinds = {"A": ka, "B": kb}
    lines = x_body(mnem, kinds)
    nacc = len(X.acc_regs)
    print(f"// {name}: two fragment sets, ring of {X.nst}; A operand {ka}-major, B operand {kb}-major, {mnem}")
    args = [f"f32x16 (&acc)[{nacc}]"]
    for which in X.ops:
        args.append(("u32x4& r" if X.blocks[which] > 2 else "u32x2& r") + which.lower())
    args.append(("u32x4& " if X.goff_span == 4 else "u32x2& ") + "goff")
    print(f"__device__ __forceinline__ void {name}({', '.join(args)},")
    print("        __amdgpu_buffer_rsrc_t rsa, __amdgpu_buffer_rsrc_t rsb, uint32_t pa, uint32_t pb,")
    print("        uint32_t ta, uint32_t tb, uint32_t m0b, uint32_t kt) {")
    print("    asm volatile(")
    for ln in lines:
        print(f'        "{ln}\\n"')
    outs = ", ".join(f'"={{{X.acc_regs[b]}}}"(acc[{b}])' for b in range(nacc))
    print(f"        : {outs},")
    g0 = X.goff["A"]
    io = [f'"+{{v[{g0}:{g0 + X.goff_span - 1}]}}"(goff)']
    declared = set(range(g0, g0 + X.goff_span))
    for which in X.ops:
        base, n = X.raddr[which], (4 if X.blocks[which] > 2 else 2)
        io.append(f'"+{{v[{base}:{base + n - 1}]}}"(r{which.lower()})')
        declared |= set(range(base, base + n))
    print("          " + ", ".join(io))
    print('        : [rsa] "s"(rsa), [rsb] "s"(rsb), [pa] "s"(pa), [pb] "s"(pb), [ta] "s"(ta), [tb] "s"(tb),')
    print('          [m0b] "s"(m0b), [kt] "s"(kt)')
    # everything the block may write besides its operands: fragment sets, derived addresses, the
    # second-half offsets
    written = set(range(X.clobber_to))
    for which in X.ops:
        written |= set(range(X.raddr[which], X.raddr[which] + ((X.nst + 1) // 2) * max(2, x_addr_regs({"A": "MN", "B": "MN"}, which))))
        written.add(X.goff2[which])
    vclob = sorted(written - declared)
    clob = [f'"v{i}"' for i in vclob] + [f'"s{i}"' for i in range(SP["A"], ST + 2)] + ['"scc"', '"memory"']
    print("        : " + ", ".join(clob) + ");")
    print("}\n")


# The tile family: (B width, ring depth) -> stem of the emitted functions.  Every member that passes
# `valid` is emitted and becomes a kernel variant the tuner can time (gemm.hip lists the codes).
FAMILY = [(256, 5, "gemm256_loop"), (256, 4, "gemm256r4_loop"), (256, 6, "gemm256r6_loop"),
          (128, 5, "gemm256x128_loop"), (128, 4, "gemm256x128r4_loop"), (128, 6, "gemm256x128r6_loop")]


def main():
    """No argument: the four-set family and the streamed loops (gemm256_loop.inc).  `two_set`: the
    members on two fragment sets (gemm_twoset_loop.inc)."""
    import sys
    print("// Generated by gen_gemm256_loop.py -- do not edit by hand.")
    if sys.argv[1:] == ["two_set"]:
        print("// Main loops of the 256x384 GEMM kernel and of the 256x128 kernel for two workgroups per compute unit")
        print("// (the generator documents the schedule and the register maps).\n")
        print("#define MHIP_HAVE_GEMM256X384_LOOP 1\n")
        for member, stem in ((_x384(), "gemm256x384_loop"), (_xpair(), "gemm_pair_loop"), (_x192(), "gemm128x192_loop"),
                             (_x288(), "gemm256x288_loop")):
            for tname, mnem in (("bf16", "v_mfma_f32_32x32x16_bf16"), ("f16", "v_mfma_f32_32x32x16_f16")):
                for lname, ka, kb in (("nn", "K", "MN"), ("nt", "K", "K"), ("tn", "MN", "MN"), ("tt", "MN", "K")):
                    emit_two_set(member, f"{stem}_{lname}_{tname}", mnem, ka, kb)
        return
    print("// Main loops of the 256x256 and 256x128 GEMM kernels (the generator documents the schedule")
    print("// and the register map).\n")
    for bw, ring, stem in FAMILY:
        if not valid(bw, ring):
            print(f"// {stem}: 256x{bw} tile with a ring of {ring} stages fails the validity filter "
                  f"({ring * (OPER + bw * 64) // 1024} KB of LDS)\n")
            continue
        print(f"#define MHIP_HAVE_{stem.upper()} 1\n")
        configure(bw, ring)
        for tname, mnem in (("bf16", "v_mfma_f32_32x32x16_bf16"), ("f16", "v_mfma_f32_32x32x16_f16")):
            for lname, ka, kb in (("nn", "K", "MN"), ("nt", "K", "K"), ("tn", "MN", "MN"), ("tt", "MN", "K")):
                emit(f"{stem}_{lname}_{tname}", mnem, ka, kb)
    # streamed tiles: the 256x128 kernel as a persistent workgroup, for A with k contiguous
    configure(128, 5)
    for tname, mnem in (("bf16", "v_mfma_f32_32x32x16_bf16"), ("f16", "v_mfma_f32_32x32x16_f16")):
        for lname, ka, kb in (("nn", "K", "MN"), ("nt", "K", "K")):
            emit_stream(f"gemm_stream_loop_{lname}_{tname}", mnem, ka, kb)


if __name__ == "__main__":
    main()
