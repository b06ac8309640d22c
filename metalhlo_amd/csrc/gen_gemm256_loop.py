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

Run:  python3 gen_gemm256_loop.py > gemm256_loop.inc
"""
import os

EXP = os.environ.get("GEMM256_EXP", "")   # timing experiments only: noload, nomfma, noread, nobarrier

NST = 5               # ring stages
UNROLL = 10           # stages per loop body: lcm(ring, pair issue, fragment set rotation)
OPER = 16384          # bytes of the A tile (256 rows x 32 k); the B tile follows it in a stage buffer
# Set per emitted function: the B tile is 256 or 128 columns wide.  The narrow form gives a
# 256x128 workgroup tile (each wave 128x64 = 4x2 accumulators, 128 AGPRs) for problems
# whose 256x256 tiling leaves compute units idle.
BW = 256              # B tile width
NBF = 4               # B fragments (32 columns each) per wave = BW / 64
STAGE = 32768         # bytes per stage buffer = OPER + BW * 64


def configure(bw):
    global BW, NBF, STAGE
    BW, NBF, STAGE = bw, bw // 64, OPER + bw * 64

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
            if t % 2 == 0:
                for p in range(passes):
                    grp.append(load_instr(which, t + 4, p))
                    grp.append(load_instr(which, t + 5, p, second_half=True))
                grp.append(dict(stage=None, lines=[f"v_add_u32 v{GOFF[which]}, 128, v{GOFF[which]}",
                                                   f"v_add_u32 v{GOFF2[which]}, 128, v{GOFF2[which]}"]))
        else:
            for p in range(passes):
                grp.append(load_instr(which, t + 5, p))
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
        for j in range(NBF):
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


def drop(lines, prefix):
    return [l for l in lines if not l.startswith(prefix)]


def stage_iteration(mnem, kinds, t, vmcnt):
    g, nxt = t % NST, (t + 1) % NST
    r0 = all_frag_reads(kinds, nxt, 0, (2 * t + 2) % 4)
    r1 = all_frag_reads(kinds, nxt, 1, (2 * t + 3) % 4)
    _, prev_second = halves(trigger_group(kinds, t - 1))
    this_first, _ = halves(trigger_group(kinds, t))
    out = []
    # k-step 0: its fragments were read one stage ago; only the previous k-step's reads
    # (LDS operations retire in order) may still be outstanding
    out.append(f"s_waitcnt lgkmcnt({min(len(r1), 15)})")
    out += interleave(mfmas(mnem, (2 * t) % 4), r0, prev_second)
    # k-step 1
    out.append(f"s_waitcnt vmcnt({min(vmcnt, 63)}) lgkmcnt({min(len(r0), 15)})")
    out.append("s_barrier")
    out += interleave(mfmas(mnem, (2 * t + 1) % 4), r1, this_first)
    if "noload" in EXP:
        out = [l for l in drop(drop(out, "buffer_load"), "s_add_u32 m0") if l != "s_nop 0"]
    if "nomfma" in EXP:
        out = drop(out, "v_mfma")
    if "noread" in EXP:
        out = drop(out, "ds_read")
    if "nobarrier" in EXP:
        out = drop(out, "s_barrier")
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


def emit(name, mnem, ka, kb):
    lines = body(mnem, {"A": ka, "B": kb})
    print(f"// {name}: A operand {ka}-major, B operand {kb}-major, {mnem}")
    print(f"__device__ __forceinline__ void {name}(f32x16 (&acc)[{4 * NBF}], u32x4 ra, u32x4 rb, u32x2& goff,")
    print("        __amdgpu_buffer_rsrc_t rsa, __amdgpu_buffer_rsrc_t rsb, uint32_t pa, uint32_t pb,")
    print("        uint32_t ta, uint32_t tb, uint32_t m0b, uint32_t kt) {")
    print("    asm volatile(")
    for ln in lines:
        print(f'        "{ln}\\n"')
    outs = ", ".join(f'"={{a[{16 * i}:{16 * i + 15}]}}"(acc[{i}])' for i in range(4 * NBF))
    print(f"        : {outs},")
    print(f'          "+{{v[{GOFF["A"]}:{GOFF["B"]}]}}"(goff)')
    print(f'        : "{{v[{RA}:{RA + 3}]}}"(ra), "{{v[{RB}:{RB + 3}]}}"(rb),')
    print('          [rsa] "s"(rsa), [rsb] "s"(rsb), [pa] "s"(pa), [pb] "s"(pb), [ta] "s"(ta), [tb] "s"(tb),')
    print('          [m0b] "s"(m0b), [kt] "s"(kt)')
    vclob = list(range(128)) + list(range(RA + 4, RB)) + list(range(RB + 4, GOFF["A"])) + [GOFF2["A"], GOFF2["B"]]
    clob = [f'"v{i}"' for i in vclob] + [f'"s{i}"' for i in range(SP["A"], ST + 2)] + ['"scc"', '"memory"']
    print("        : " + ", ".join(clob) + ");")
    print("}\n")


def main():
    print("// Generated by gen_gemm256_loop.py -- do not edit by hand.")
    print("// Main loops of the 256x256 and 256x128 GEMM kernels (the generator documents the schedule")
    print("// and the register map).\n")
    for bw, stem in ((256, "gemm256_loop"), (128, "gemm256x128_loop")):
        configure(bw)
        for tname, mnem in (("bf16", "v_mfma_f32_32x32x16_bf16"), ("f16", "v_mfma_f32_32x32x16_f16")):
            for lname, ka, kb in (("nn", "K", "MN"), ("nt", "K", "K"), ("tn", "MN", "MN"), ("tt", "MN", "K")):
                emit(f"{stem}_{lname}_{tname}", mnem, ka, kb)


if __name__ == "__main__":
    main()
