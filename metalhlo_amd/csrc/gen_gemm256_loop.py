#!/usr/bin/env python3
"""Generates gemm256_loop.inc: the hand-scheduled main loop of the 256x256 GEMM
kernel for gfx950 as inline assembly with a fixed register map.

One workgroup = 4 waves (one per SIMD); each wave owns a 128x128 sub-tile =
4x4 v_mfma_f32_32x32x16 accumulators = all 256 AGPRs.  With a single wave per
SIMD nothing hides a stall except the wave's own instruction stream, so the
order of every instruction is fixed here instead of being left to the compiler.

K is consumed in stages of 32 (two k-steps of 16).  LDS holds a ring of four stage
buffers (32 KB each: A tile 16 KB, B tile 16 KB) that is filled by buffer loads
that write LDS directly (no staging registers, no LDS store instructions).
Fragments are read from LDS two k-steps (= one stage) before the MFMAs that use
them, into a rotation of four fragment register sets, so a wait for fragments
never follows their reads closely.  Stage t (buffer t % 4):

  k-step 0 : 16 MFMAs; reads of stage t+1 k-step 0 fragments;
             second half of the direct-to-LDS loads of stage t+3
  wait: k-step 1 fragments there (= all own reads of buffer t % 4 done), own
        loads of stage t+2 landed;  workgroup barrier
  k-step 1 : 16 MFMAs; reads of stage t+1 k-step 1 fragments;
             first half of the loads of stage t+4 into buffer t % 4

Register map (VGPR):
  fragment set n (n = 0..3, k-step 2t+s uses set (2t+s) % 4):
      A fragments v[32n : 32n+15], B fragments v[32n+16 : 32n+31]
  v[192:199] A fragment read addresses, v[200:207] B fragment read addresses
  v208 / v209 A / B global byte offsets of this thread's 16-byte chunk
AGPR: accumulator (i, j) = a[16*(4*i+j) : +15]
SGPR: s[72:74] = 1..3 x A pass stride, s[76:78] = 1..3 x B pass stride, s80 = stage counter,
      s81 = caller's M0 (restored at the end)

An operand is either "K" (k is the contiguous axis in memory: stage tile stored
[256 rows][32 k], fragments read with ds_read_b128) or "MN" (k is the slow axis:
tile stored as it lies, [32 k][256 mn], fragments transposed on the way out with
ds_read_b64_tr_b16).  Fragment read addresses: "K": element 2*h + s = k-step s in
ring half h (buffers 2h, 2h+1); "MN": element 4*h + j = mn block j in ring half h.

Run:  python3 gen_gemm256_loop.py > gemm256_loop.inc
"""
import os

EXP = os.environ.get("GEMM256_EXP", "")   # timing experiments only: noload, nomfma, noread

NST = 4               # ring stages
STAGE = 32768         # bytes per stage buffer
OPER = 16384          # bytes per operand tile
SET = {n: (32 * n, 32 * n + 16) for n in range(4)}   # fragment set -> (A base vgpr, B base vgpr)
RA, RB = 192, 200
GA, GB = 208, 209
SPA, SPB, ST = 72, 76, 80


def vr(base, n):
    return f"v[{base}:{base + n - 1}]"


def frag_reads(kind, which, g, s, fset):
    """LDS reads of the 4 fragments of k-step `s` of operand `which` from ring buffer `g`."""
    base = SET[fset][0 if which == "A" else 1]
    addr = RA if which == "A" else RB
    h, lo = g >> 1, (g & 1) * STAGE
    out = []
    for j in range(4):
        dst = base + 4 * j
        if kind == "K":
            out.append(f"ds_read_b128 {vr(dst, 4)}, v{addr + 2 * h + s} offset:{lo + j * 2048}")
        else:
            off = lo + s * 8192
            out.append(f"ds_read_b64_tr_b16 {vr(dst, 2)}, v{addr + 4 * h + j} offset:{off}")
            out.append(f"ds_read_b64_tr_b16 {vr(dst + 2, 2)}, v{addr + 4 * h + j} offset:{off + 2048}")
    return out


def all_frag_reads(ka, kb, g, s, fset):
    a, b = frag_reads(ka, "A", g, s, fset), frag_reads(kb, "B", g, s, fset)
    out = []
    for i in range(max(len(a), len(b))):
        out += a[i:i + 1] + b[i:i + 1]
    return out


def stage_loads(g, passes=range(4), advance=True):
    """Direct-to-LDS loads of one stage into ring buffer `g`: 4 passes per operand; the
    wave's 1 KB LDS slot of pass p is M0 = wave base + buffer + operand + p * 4096."""
    out = []
    for p in passes:
        so_a = "0" if p == 0 else f"s{SPA + p - 1}"
        so_b = "0" if p == 0 else f"s{SPB + p - 1}"
        out.append(f"s_add_u32 m0, %[m0b], {g * STAGE + p * 4096}")
        out.append("s_nop 0")
        out.append(f"buffer_load_dwordx4 v{GA}, %[rsa], {so_a} offen lds")
        out.append(f"s_add_u32 m0, %[m0b], {g * STAGE + OPER + p * 4096}")
        out.append("s_nop 0")
        out.append(f"buffer_load_dwordx4 v{GB}, %[rsb], {so_b} offen lds")
    if advance:
        out.append(f"v_add_u32 v{GA}, %[ta], v{GA}")
        out.append(f"v_add_u32 v{GB}, %[tb], v{GB}")
    return out


def group3(lines):
    """Keeps each (s_add m0, s_nop, buffer_load) triple together when interleaving."""
    out, i = [], 0
    while i < len(lines):
        if lines[i].startswith("s_add_u32 m0"):
            out.append(lines[i:i + 3])
            i += 3
        else:
            out.append([lines[i]])
            i += 1
    return out


def mfmas(mnem, fset):
    a, b = SET[fset]
    out = []
    for i in range(4):
        for j in range(4):
            acc = 16 * (4 * i + j)
            # (B, A): the accumulator tile comes out transposed (lane = row m)
            out.append(f"{mnem} a[{acc}:{acc + 15}], {vr(b + 4 * j, 4)}, {vr(a + 4 * i, 4)}, a[{acc}:{acc + 15}]")
    return out


def interleave(main, reads, loads, wave):
    """The four waves of a workgroup run in lockstep between barriers and share one
    LDS and one texture addresser, so each wave gets its own slots: wave w issues its
    fragment reads behind MFMAs 4w .. 4w+3 and its global loads behind MFMAs
    w, w+4, w+8, w+12 of a k-step.  A load group is a list of lines kept together."""
    loads = [[x] if isinstance(x, str) else x for x in loads]
    per = (len(reads) + 3) // 4
    out, kl = [], 0
    for idx, m in enumerate(main):
        out.append(m)
        rel = idx - 4 * wave
        if 0 <= rel < 4:
            out += reads[rel * per:(rel + 1) * per]
        if idx % 4 == wave and kl < len(loads):
            out += loads[kl]
            kl += 1
    for grp in loads[kl:]:
        out += grp
    return out


def drop(lines, prefix):
    return [l for l in lines if not l.startswith(prefix)]


def stage_iteration(mnem, ka, kb, g, wave):
    nxt, prv = (g + 1) % NST, (g - 1) % NST
    r0 = all_frag_reads(ka, kb, nxt, 0, (2 * g + 2) % 4)
    r1 = all_frag_reads(ka, kb, nxt, 1, (2 * g + 3) % 4)
    out = []
    # k-step 0: its fragments were read one stage ago; only the previous k-step's reads
    # (LDS operations retire in order) may still be outstanding
    out.append(f"s_waitcnt lgkmcnt({min(len(r1), 15)})")
    out += interleave(mfmas(mnem, (2 * g) % 4), r0, group3(stage_loads(prv, (2, 3))), wave)
    # k-step 1
    out.append(f"s_waitcnt vmcnt(8) lgkmcnt({min(len(r0), 15)})")
    out.append("s_barrier")
    out += interleave(mfmas(mnem, (2 * g + 1) % 4), r1, group3(stage_loads(g, (0, 1), advance=False)), wave)
    if "noload" in EXP:
        out = [l for l in drop(drop(out, "buffer_load"), "s_add_u32 m0") if l != "s_nop 0"]
    if "nomfma" in EXP:
        out = drop(out, "v_mfma")
    if "noread" in EXP:
        out = drop(out, "ds_read")
    if "nobarrier" in EXP:
        out = drop(out, "s_barrier")
    return out


def body(mnem, ka, kb):
    out = []
    for r in range(256):
        out.append(f"v_accvgpr_write_b32 a{r}, 0")
    for i in range(1, 4):
        out.append(f"s_mul_i32 s{SPA + i - 1}, %[pa], {i}")
        out.append(f"s_mul_i32 s{SPB + i - 1}, %[pb], {i}")
    out.append(f"s_mov_b32 s{ST}, 0")
    out.append(f"s_mov_b32 s{ST + 1}, m0")
    for g in range(NST - 1):
        out += stage_loads(g)
    out += stage_loads(NST - 1, (0, 1), advance=False)
    out.append("s_waitcnt vmcnt(12)")           # stages 0 and 1 landed
    out.append("s_barrier")
    out += all_frag_reads(ka, kb, 0, 0, 0)
    out += all_frag_reads(ka, kb, 0, 1, 1)
    out.append("s_waitcnt lgkmcnt(0)")
    # one copy of the loop per wave of the workgroup (different slot assignment)
    nvar = 1 if "nostagger" in EXP else 4
    for w in range(1, nvar):
        out.append(f"s_cmp_eq_u32 %[wv], {w}")
        out.append(f"s_cbranch_scc1 L_gemm256_loop{w}_%=")
    for w in range(nvar):
        out.append(f"L_gemm256_loop{w}_%=:")
        for g in range(NST):
            out += stage_iteration(mnem, ka, kb, g, w)
            out.append(f"s_add_u32 s{ST}, s{ST}, 1")
            if g < NST - 1:
                out.append(f"s_cmp_ge_u32 s{ST}, %[kt]")
                out.append("s_cbranch_scc1 L_gemm256_done_%=")
            else:
                out.append(f"s_cmp_lt_u32 s{ST}, %[kt]")
                out.append(f"s_cbranch_scc1 L_gemm256_loop{w}_%=")
        if w < nvar - 1:
            out.append("s_branch L_gemm256_done_%=")
    out.append("L_gemm256_done_%=:")
    # drain: loads of stages past the end still write LDS, which the caller reuses;
    # the last MFMA results must be readable by ordinary instructions
    out.append("s_waitcnt vmcnt(0) lgkmcnt(0)")
    out.append("s_barrier")
    out.append(f"s_mov_b32 m0, s{ST + 1}")
    out += ["s_nop 15", "s_nop 15"]
    return out


def emit(name, mnem, ka, kb):
    lines = body(mnem, ka, kb)
    print(f"// {name}: A operand {ka}-major, B operand {kb}-major, {mnem}")
    print(f"__device__ __forceinline__ void {name}(f32x16 (&acc)[16], u32x8 ra, u32x8 rb, u32x2& goff,")
    print("        __amdgpu_buffer_rsrc_t rsa, __amdgpu_buffer_rsrc_t rsb, uint32_t pa, uint32_t pb,")
    print("        uint32_t ta, uint32_t tb, uint32_t m0b, uint32_t kt, uint32_t wv) {")
    print("    asm volatile(")
    for ln in lines:
        print(f'        "{ln}\\n"')
    outs = ", ".join(f'"={{a[{16 * i}:{16 * i + 15}]}}"(acc[{i}])' for i in range(16))
    print(f"        : {outs},")
    print(f'          "+{{v[{GA}:{GB}]}}"(goff)')
    print(f'        : "{{v[{RA}:{RA + 7}]}}"(ra), "{{v[{RB}:{RB + 7}]}}"(rb),')
    print('          [rsa] "s"(rsa), [rsb] "s"(rsb), [pa] "s"(pa), [pb] "s"(pb), [ta] "s"(ta), [tb] "s"(tb),')
    print('          [m0b] "s"(m0b), [kt] "s"(kt), [wv] "s"(wv)')
    clob = [f'"v{i}"' for i in range(128)] + [f'"s{i}"' for i in range(SPA, ST + 2)] + ['"scc"', '"memory"']
    print("        : " + ", ".join(clob) + ");")
    print("}\n")


def main():
    print("// Generated by gen_gemm256_loop.py -- do not edit by hand.")
    print("// Main loops of the 256x256 GEMM kernel (the generator documents the schedule")
    print("// and the register map).\n")
    for tname, mnem in (("bf16", "v_mfma_f32_32x32x16_bf16"), ("f16", "v_mfma_f32_32x32x16_f16")):
        for lname, ka, kb in (("nn", "K", "MN"), ("nt", "K", "K"), ("tn", "MN", "MN"), ("tt", "MN", "K")):
            emit(f"gemm256_loop_{lname}_{tname}", mnem, ka, kb)


if __name__ == "__main__":
    main()
