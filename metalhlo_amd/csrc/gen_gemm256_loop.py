#!/usr/bin/env python3
"""Generates gemm256_loop.inc: the hand-scheduled main loop of the 256x256x64
GEMM kernel for gfx950 as inline assembly with a fixed register map.

One workgroup = 4 waves (one per SIMD); each wave owns a 128x128 sub-tile =
4x4 v_mfma_f32_32x32x16 accumulators = all 256 AGPRs.  With a single wave per
SIMD nothing hides a stall except the wave's own instruction stream, so the
order of every instruction is fixed here instead of being left to the compiler:

  * global -> register prefetch runs two K tiles ahead of the tile whose data
    is being written to LDS (two staging register sets, X and Y),
  * LDS -> register fragment reads of k-step s+1 are spread between the 16
    MFMAs of k-step s (two fragment register sets),
  * register -> LDS stores of tile t+1 are spread over k-steps 0 and 1, the
    global loads of tile t+3 over k-step 2,
  * one workgroup barrier per tile, in front of k-step 3, whose MFMAs cover the
    reads of the next tile's first fragments.

Register map (VGPR):
  v[0:15]  A fragments set 0     v[16:31] B fragments set 0
  v[32:47] A fragments set 1     v[48:63] B fragments set 1
  v[64:95] staging X (A)         v[96:127] staging X (B)
  v[128:159] staging Y (A)       v[160:191] staging Y (B)
  v[192:195] A fragment read addresses   v[196:199] B fragment read addresses
  v200 A LDS write address, v201 B LDS write address, v202 / v203 A / B global offsets
AGPR: accumulator (i, j) = a[16*(4*i+j) : +15]
SGPR: s[72:78] = 1..7 x A pass stride, s[80:86] = 1..7 x B pass stride, s88 = tile counter

An operand is either "K" (k is the contiguous axis in memory: tile stored
[256 rows][64 k], fragments read with ds_read_b128) or "MN" (k is the slow
axis: tile stored as it lies, [64 k][256 mn], fragments transposed on the way
out with ds_read_b64_tr_b16).

Run:  python3 gen_gemm256_loop.py > gemm256_loop.inc
"""
import os
import sys

EXP = os.environ.get('GEMM256_EXP', '')   # timing experiments: noload, nowrite, nomfma, noread

TILE = 32768          # bytes per operand tile in LDS
SET = {0: (0, 16), 1: (32, 48)}                 # fragment set -> (A base vgpr, B base vgpr)
STAGE = {"X": (64, 96), "Y": (128, 160)}        # staging set -> (A base vgpr, B base vgpr)
RA, RB = 192, 196
WA, WB, GA, GB = 200, 201, 202, 203
SPA, SPB, ST = 72, 80, 88


def vr(base, n):
    return f"v[{base}:{base + n - 1}]"


def frag_reads(kind, which, buf, s, fset):
    """LDS reads of the 4 fragments of k-step `s` of operand `which` from LDS buffer `buf`."""
    base = SET[fset][0 if which == "A" else 1]
    addr = RA if which == "A" else RB
    out = []
    for j in range(4):
        dst = base + 4 * j
        if kind == "K":
            out.append(f"ds_read_b128 {vr(dst, 4)}, v{addr + s} offset:{j * 4096 + buf * TILE}")
        else:
            off = s * 8192 + buf * TILE
            out.append(f"ds_read_b64_tr_b16 {vr(dst, 2)}, v{addr + j} offset:{off}")
            out.append(f"ds_read_b64_tr_b16 {vr(dst + 2, 2)}, v{addr + j} offset:{off + 2048}")
    return out


def all_frag_reads(ka, kb, buf, s, fset):
    a, b = frag_reads(ka, "A", buf, s, fset), frag_reads(kb, "B", buf, s, fset)
    # alternate A / B so the first MFMAs' operands arrive first
    out = []
    for i in range(max(len(a), len(b))):
        out += a[i:i + 1] + b[i:i + 1]
    return out


def lds_writes(stage, buf):
    sa, sb = STAGE[stage]
    out = []
    for i in range(8):
        out.append(f"ds_write_b128 v{WA}, {vr(sa + 4 * i, 4)} offset:{i * 4096 + buf * TILE}")
        out.append(f"ds_write_b128 v{WB}, {vr(sb + 4 * i, 4)} offset:{i * 4096 + buf * TILE}")
    return out


def global_loads(stage):
    sa, sb = STAGE[stage]
    out = []
    for i in range(8):
        so_a = "0" if i == 0 else f"s{SPA + i - 1}"
        so_b = "0" if i == 0 else f"s{SPB + i - 1}"
        out.append(f"buffer_load_dwordx4 {vr(sa + 4 * i, 4)}, v{GA}, %[rsa], {so_a} offen")
        out.append(f"buffer_load_dwordx4 {vr(sb + 4 * i, 4)}, v{GB}, %[rsb], {so_b} offen")
    out.append(f"v_add_u32 v{GA}, %[ta], v{GA}")
    out.append(f"v_add_u32 v{GB}, %[tb], v{GB}")
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


def interleave(main, first, rest=()):
    """One instruction of `first` behind each of the leading instructions of `main`
    (two while they outnumber the slots left), then `rest` spread evenly over the
    remaining instructions of `main`."""
    first, rest = list(first), list(rest)
    out = []
    n_first_slots = len(main) if not rest else min(len(main) // 2, len(first))
    per_f, extra_f = divmod(len(first), n_first_slots) if first else (0, 0)
    rest_slots = len(main) - n_first_slots
    per_r, extra_r = divmod(len(rest), rest_slots) if rest else (0, 0)
    kf = kr = 0
    for idx, m in enumerate(main):
        out.append(m)
        if idx < n_first_slots:
            n = per_f + (1 if idx < extra_f else 0)
            out += first[kf:kf + n]
            kf += n
        else:
            slot = idx - n_first_slots
            n = per_r + (1 if slot < extra_r else 0)
            out += rest[kr:kr + n]
            kr += n
    assert kf == len(first) and kr == len(rest), (kf, len(first), kr, len(rest))
    return out


def drop(lines, prefix):
    return [l for l in lines if not l.startswith(prefix)]


def tile_iteration(mnem, ka, kb, cur, stage):
    out = tile_iteration0(mnem, ka, kb, cur, stage)
    if 'noload' in EXP:
        out = drop(out, 'buffer_load')
        out = drop(out, 's_waitcnt vmcnt')
    if 'nowrite' in EXP:
        out = drop(out, 'ds_write')
    if 'nomfma' in EXP:
        out = drop(out, 'v_mfma')
    if 'noread' in EXP:
        out = drop(out, 'ds_read')
    return out


def tile_iteration0(mnem, ka, kb, cur, stage):
    """One K tile: consume LDS buffer `cur`; staging set `stage` holds tile t+1 and,
    once stored to the other LDS buffer, receives tile t+3.  Within a k-step the
    fragment reads go first and the LDS stores last, so the wait in front of the next
    k-step (LDS operations retire in order) covers the reads only."""
    nxt = cur ^ 1
    out = []
    w = lds_writes(stage, nxt)
    # k-step 0: fragments set 0 are ready (waited for at the end of the previous tile)
    out += interleave(mfmas(mnem, 0), all_frag_reads(ka, kb, cur, 1, 1), ["s_waitcnt vmcnt(16)"] + w[:8])
    out.append("s_waitcnt lgkmcnt(8)")
    # k-step 1
    out += interleave(mfmas(mnem, 1), all_frag_reads(ka, kb, cur, 2, 0), w[8:])
    out.append("s_waitcnt lgkmcnt(8)")
    # k-step 2
    # (the staging registers' last LDS stores have retired once only this k-step's
    # reads are outstanding)
    r3 = all_frag_reads(ka, kb, cur, 3, 1)
    out += interleave(mfmas(mnem, 0), r3, [f"s_waitcnt lgkmcnt({min(len(r3), 15)})"] + global_loads(stage))
    # k-step 3: everyone has read `cur` and written `nxt`
    out.append("s_waitcnt lgkmcnt(0)")
    out.append("s_barrier")
    out += interleave(mfmas(mnem, 1), all_frag_reads(ka, kb, nxt, 0, 0))
    out.append("s_waitcnt lgkmcnt(0)")
    return out


def body(mnem, ka, kb):
    out = []
    for r in range(256):
        out.append(f"v_accvgpr_write_b32 a{r}, 0")
    for i in range(1, 8):
        out.append(f"s_mul_i32 s{SPA + i - 1}, %[pa], {i}")
        out.append(f"s_mul_i32 s{SPB + i - 1}, %[pb], {i}")
    out.append(f"s_mov_b32 s{ST}, 0")
    out += global_loads("X")            # tile 0
    out += global_loads("Y")            # tile 1
    out.append("s_waitcnt vmcnt(16)")
    out += lds_writes("X", 0)
    out += global_loads("X")            # tile 2
    out.append("s_waitcnt lgkmcnt(0)")
    out.append("s_barrier")
    out += all_frag_reads(ka, kb, 0, 0, 0)
    out.append("s_waitcnt lgkmcnt(0)")
    out.append("L_gemm256_loop_%=:")
    out += tile_iteration(mnem, ka, kb, 0, "Y")
    out.append(f"s_add_u32 s{ST}, s{ST}, 1")
    out.append(f"s_cmp_ge_u32 s{ST}, %[kt]")
    out.append("s_cbranch_scc1 L_gemm256_done_%=")
    out += tile_iteration(mnem, ka, kb, 1, "X")
    out.append(f"s_add_u32 s{ST}, s{ST}, 1")
    out.append(f"s_cmp_lt_u32 s{ST}, %[kt]")
    out.append("s_cbranch_scc1 L_gemm256_loop_%=")
    out.append("L_gemm256_done_%=:")
    # drain: outstanding prefetches must land before the staging registers are reused,
    # and the last MFMA results must be readable by ordinary instructions
    out.append("s_waitcnt vmcnt(0)")
    out += ["s_nop 15", "s_nop 15"]
    return out


def emit(name, mnem, ka, kb):
    lines = body(mnem, ka, kb)
    print(f"// {name}: A operand {ka}-major, B operand {kb}-major, {mnem}")
    print(f"__device__ __forceinline__ void {name}(f32x16 (&acc)[16], u32x4 ra, u32x4 rb, u32x4& misc,")
    print("        __amdgpu_buffer_rsrc_t rsa, __amdgpu_buffer_rsrc_t rsb, uint32_t pa, uint32_t pb,")
    print("        uint32_t ta, uint32_t tb, uint32_t kt) {")
    print("    asm volatile(")
    for ln in lines:
        print(f'        "{ln}\\n"')
    outs = ", ".join(f'"={{a[{16 * i}:{16 * i + 15}]}}"(acc[{i}])' for i in range(16))
    print(f"        : {outs},")
    print(f'          "+{{v[{WA}:{WA + 3}]}}"(misc)')
    print(f'        : "{{v[{RA}:{RA + 3}]}}"(ra), "{{v[{RB}:{RB + 3}]}}"(rb),')
    print('          [rsa] "s"(rsa), [rsb] "s"(rsb), [pa] "s"(pa), [pb] "s"(pb), [ta] "s"(ta), [tb] "s"(tb), [kt] "s"(kt)')
    clob = [f'"v{i}"' for i in range(192)] + [f'"s{i}"' for i in range(SPA, ST + 1)] + ['"scc"', '"memory"']
    print("        : " + ", ".join(clob) + ");")
    print("}\n")


def main():
    print("// Generated by gen_gemm256_loop.py -- do not edit by hand.")
    print("// Main loops of the 256x256x64 GEMM kernel (see the generator for the schedule")
    print("// and the register map).\n")
    for tname, mnem in (("bf16", "v_mfma_f32_32x32x16_bf16"), ("f16", "v_mfma_f32_32x32x16_f16")):
        for lname, ka, kb in (("nn", "K", "MN"), ("nt", "K", "K"), ("tn", "MN", "MN"), ("tt", "MN", "K")):
            emit(f"gemm256_loop_{lname}_{tname}", mnem, ka, kb)


if __name__ == "__main__":
    main()
