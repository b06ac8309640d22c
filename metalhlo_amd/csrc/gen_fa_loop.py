#!/usr/bin/env python3
"""Generates fa_loop.inc: the hand-scheduled steady-state loop of the pipelined
flash-attention kernel (attention_pipe.hip) for gfx950 as inline assembly with a
fixed register map.  It covers key blocks that need no masking; the first block, the
blocks on the causal diagonal / past the last key and the final P.V product stay in
the C++ code around it.

One wave owns 64 query rows (two 32-row query blocks q0, q1) and walks key blocks of
64.  A wave that is alone on its SIMD issues one instruction every five cycles or so,
and a v_mfma_f32_32x32x16_bf16 keeps the matrix pipe busy for 32, so about six other
instructions fit behind every MFMA and nothing else is free: the loop is laid out so
that EVERY MFMA has softmax arithmetic behind it.  Body for block j (entered with the
raw scores S(j) and the finished P(j-1)):

  phase B   O += V(j-1)^T . P(j-1)^T        32 MFMAs, 16 V fragments (2 transposing
            || first half of softmax(j)     reads each); row maxima, reference update,
                                            alpha(j), the first exponentials
  end of B  O *= alpha(j) where a row's reference maximum moved (rare, see below);
            wait for this wave's loads of the next blocks, workgroup barrier,
            8 direct-to-LDS loads: K(j+4), V(j+3) into the buffers just released
  phase A   S(j+1) = K(j+1) . Q^T           32 MFMAs, 16 K fragments (ds_read_b128) into
            || second half of softmax(j)    the other S buffer; remaining exponentials,
                                            row sums, conversion to P(j)

Softmax keeps a REFERENCE maximum per row that only moves when the block maximum exceeds
it by more than 8 (log2 domain): probabilities are exp2(s - ref) <= 2^8, accumulated in
fp32, and the final normalisation divides by the sum taken with the same reference, so
the result is the same function; what it saves is the rescaling of the 128 accumulator
registers, which a strict running maximum triggers in almost every block when 64 rows
share a wave.

Register map:
  a[0:63]    Q^T fragments: query block qi, k-step st at a[4*(8*qi+st) : +3]
  a[128:255] O accumulators: (qi, dt) at a[128 + 16*(4*qi+dt) : +15]
  v[0:63]    S buffer 0, v[192:255] S buffer 1: (qi, t) at base + 16*(2*qi+t); bodies
             alternate (even: softmax reads buffer 0, the MFMAs fill buffer 1);
             exponentials overwrite the scores in place
  v[64:95]   P set X, v[160:191] P set Y: (qi, u) at base + 4*(4*qi+u); bodies
             alternate (even: read Y, write X)
  v[96:111]  fragment ring (4 x 4): K fragments in phase A, V fragments in phase B;
             v[112:127] are left to the compiler
  v[128:135] K fragment addresses per k-step, v[136:139] V fragment addresses per d block
  v[140:143] reference maximum q0, q1, running sum q0, q1
  v[144:145] byte offsets of this thread's chunk in the K / V blocks loaded next
  v[146:159] alpha q0, q1 and six temporaries per query block
  s[72:74] = 4096, 8192, 12288 (row-group offsets of the loads), s76 = body counter,
  s77 = caller's M0, s[78:79] / s[80:81] = compare results of q0 / q1,
  s[82:83] / s[84:85] = lanes of q0 / q1 whose reference maximum moved
"""
NQ = 2
SBUF = (0, 192)
PX, PY = 64, 160
KF = VF = 96       # one fragment ring: phase A holds K fragments in it, phase B V fragments
KADDR, VADDR = 128, 136
MREF, LSUM = 140, 142
GK, GV = 144, 145
ALPHA = 146
T0 = 148          # temporaries: six per query block
KTILE = 16384
VRING = 65536
MN = "v_mfma_f32_32x32x16_bf16"     # main() sets both per element type
CVT = "v_cvt_pk_bf16_f32"


def v(i, n=1):
    return f"v{i}" if n == 1 else f"v[{i}:{i + n - 1}]"


def a(i, n=1):
    return f"a{i}" if n == 1 else f"a[{i}:{i + n - 1}]"


def softmax_stream(qi, sbase, pnew):
    """VALU instructions turning S(qi) (32 registers) into packed P and updating the row state.
    The two query blocks' streams are interleaved instruction by instruction by the caller,
    so each has its own temporaries and its own condition register pair."""
    S = [sbase + 32 * qi + i for i in range(32)]
    t0, t1, mc, thr, mnew, acc = (T0 + 6 * qi + i for i in range(6))
    cond = f"s[{78 + 2 * qi}:{79 + 2 * qi}]"
    al = ALPHA + qi
    out = []
    # maximum: two chains
    out.append(f"v_max3_f32 {v(t0)}, {v(S[0])}, {v(S[1])}, {v(S[2])}")
    out.append(f"v_max3_f32 {v(t1)}, {v(S[3])}, {v(S[4])}, {v(S[5])}")
    i, k = 6, 0
    while i < 32:
        t = (t0, t1)[k % 2]
        out.append(f"v_max3_f32 {v(t)}, {v(t)}, {v(S[i])}, {v(S[i + 1])}")
        i += 2
        k += 1
    out.append(f"v_max_f32 {v(t0)}, {v(t0)}, {v(t1)}")
    out.append(f"v_mov_b32 {v(t1)}, {v(t0)}")
    out.append("s_nop 1")
    out.append(f"v_permlane32_swap_b32 {v(t0)}, {v(t1)}")        # the other 32-lane half's maximum
    out.append("s_nop 1")
    out.append(f"v_max_f32 {v(t0)}, {v(t0)}, {v(t1)}")
    out.append(f"v_mul_f32 {v(mc)}, %[c], {v(t0)}")              # block maximum in the log2 domain
    out.append(f"v_add_f32 {v(thr)}, 0x41000000, {v(MREF + qi)}")   # reference + 8
    out.append(f"v_cmp_gt_f32 {cond}, {v(mc)}, {v(thr)}")
    out.append(f"v_cndmask_b32 {v(mnew)}, {v(MREF + qi)}, {v(mc)}, {cond}")
    out.append(f"v_sub_f32 {v(thr)}, {v(MREF + qi)}, {v(mnew)}")
    out.append(f"v_exp_f32 {v(al)}, {v(thr)}")                   # alpha = 2^(old ref - new ref)
    out.append(f"v_mov_b32 {v(MREF + qi)}, {v(mnew)}")
    out.append(f"v_cmp_neq_f32 s[{82 + 2 * qi}:{83 + 2 * qi}], 1.0, {v(al)}")      # lanes whose reference moved
    # exponentials: the fma of element i+2 sits between the fma and the exp of element i
    for r in S[:2]:
        out.append(f"v_fma_f32 {v(r)}, {v(r)}, %[c], -{v(mnew)}")
    for i, r in enumerate(S):
        if i + 2 < 32:
            out.append(f"v_fma_f32 {v(S[i + 2])}, {v(S[i + 2])}, %[c], -{v(mnew)}")
        out.append(f"v_exp_f32 {v(r)}, {v(r)}")
    # row sum: two chains (v_dot2c on the packed pairs would halve the count, but it costs
    # more than two adds next to the MFMAs)
    out.append(f"v_add_f32 {v(acc)}, {v(S[0])}, {v(S[1])}")
    out.append(f"v_add_f32 {v(t0)}, {v(S[2])}, {v(S[3])}")
    for i in range(4, 32):
        t = (acc, t0)[i % 2]
        out.append(f"v_add_f32 {v(t)}, {v(t)}, {v(S[i])}")
    out.append(f"v_add_f32 {v(acc)}, {v(acc)}, {v(t0)}")
    for p in range(8):
        out.append(f"{CVT} {v(pnew + 16 * qi + p)}, {v(S[2 * p])}, {v(S[2 * p + 1])}")
    out.append(f"v_fma_f32 {v(LSUM + qi)}, {v(LSUM + qi)}, {v(al)}, {v(acc)}")
    for p in range(8, 16):
        out.append(f"{CVT} {v(pnew + 16 * qi + p)}, {v(S[2 * p])}, {v(S[2 * p + 1])}")
    return out


def interleave(x, y):
    out = []
    for i in range(max(len(x), len(y))):
        if i < len(x):
            out.append(x[i])
        if i < len(y):
            out.append(y[i])
    return out


def chunks(lst, n):
    """lst cut into n consecutive pieces of nearly equal length."""
    out, pos = [], 0
    for i in range(n):
        end = (len(lst) * (i + 1)) // n
        out.append(lst[pos:end])
        pos = end
    return out


def rescale_block(tag):
    """O *= alpha when some lane's alpha is not 1 (the accumulators live in AGPRs); lanes
    whose alpha is 1 multiply by 1.  The compares sit in the softmax streams."""
    out = ["s_or_b64 s[82:83], s[82:83], s[84:85]", "s_cmp_eq_u64 s[82:83], 0", f"s_cbranch_scc1 L_fa_keep_{tag}_%=",
           "s_nop 15", "s_nop 15"]          # the last MFMAs' results must be readable
    for qi in range(NQ):
        for r in range(64):
            reg = 128 + 64 * qi + r
            out.append(f"v_accvgpr_read_b32 {v(T0)}, {a(reg)}")
            out.append(f"v_mul_f32 {v(T0)}, {v(T0)}, {v(ALPHA + qi)}")
            out.append(f"v_accvgpr_write_b32 {a(reg)}, {v(T0)}")
    out.append("s_nop 4")
    out.append(f"L_fa_keep_{tag}_%=:")
    return out


RING = 8           # fragment ring slots (v[96:127]); a slot holds one K or one V fragment
VAHEAD = 6         # V fragments (two reads each) in flight at most: the LDS counter holds 15 operations


def k_read(f, slot, ring=4):
    st, t = f // 2, f % 2
    return f"ds_read_b128 {v(KF + 4 * (f % ring), 4)}, {v(KADDR + st)} offset:{slot * KTILE + t * 8192}"


def v_reads(g, slot, ring=4):
    u, dt = g // 4, g % 4
    base = VF + 4 * (g % ring)
    off = slot * KTILE + u * 4096
    return [f"ds_read_b64_tr_b16 {v(base, 2)}, {v(VADDR + dt)} offset:{off}",
            f"ds_read_b64_tr_b16 {v(base + 2, 2)}, {v(VADDR + dt)} offset:{off + 2048}"]


def v_prefetch(slot):
    out = []
    for g in range(4):
        out += v_reads(g, slot)
    return out


class LdsOrder:
    """LDS reads in program order, to size the lgkmcnt waits: a wait for fragment X may leave
    outstanding exactly the reads issued after X's last one (they return in order)."""

    def __init__(self):
        self.tags = []

    def issue(self, tag, lines):
        self.tags += [tag] * len(lines)
        return lines

    def wait_for(self, tags):
        last = max(i for i, t in enumerate(self.tags) if t in tags)
        return f"s_waitcnt lgkmcnt({min(len(self.tags) - 1 - last, 15)})"


def loop_prefetch(order, body_no, slot):
    """The first VAHEAD V fragments of body `body_no` (ring buffer `slot`)."""
    out = []
    for g in range(VAHEAD):
        out += order.issue(("V", body_no, g), v_reads(g, slot, RING))
    return out


def body(n, order, uid):
    """Body n of the unrolled loop handles block j = n (mod 4).  `uid` numbers the bodies in
    emission order (tags of the fragment reads, which run ahead across bodies).

    Fragments go through a ring of eight register slots (fragment i of a phase in slot i % 8).
    V fragments are read up to six ahead; the K fragments of phase A are read from the last
    iterations of phase B on, i.e. BEFORE this step's barrier: the wait in front of the barrier
    leaves only the youngest pair of loads in flight, so K(j+1) landed, for every wave, with the
    barrier of the step before.  Phase A then starts with its first fragments in registers
    instead of behind a full LDS latency."""
    slot_v = (n + 3) % 4             # V(j-1)
    slot_k = (n + 1) % 4             # K(j+1)
    load_k, load_v = n % 4, (n + 3) % 4          # K(j+4) replaces K(j), V(j+3) replaces V(j-1)
    s_in, s_out = (SBUF[0], SBUF[1]) if n % 2 == 0 else (SBUF[1], SBUF[0])
    pprev, pnew = (PY, PX) if n % 2 == 0 else (PX, PY)
    valu = interleave(softmax_stream(0, s_in, pnew), softmax_stream(1, s_in, pnew))
    half = len(valu) // 2
    # the scores were written by the MFMAs just before this body: the first two MFMAs of
    # phase B (64 cycles) stand between them and the first instruction that reads them
    head = [[], []] + chunks(valu[:half], 30)
    tail = chunks(valu[half:], 32)
    out = []
    # ---- phase B: O += V^T . P^T  ||  first half of the softmax
    k = 0
    for g2 in range(8):
        out.append(order.wait_for({("V", uid, 2 * g2), ("V", uid, 2 * g2 + 1)}))
        for g in (2 * g2, 2 * g2 + 1):
            u, dt = g // 4, g % 4
            for qi in range(NQ):
                acc = a(128 + 16 * (4 * qi + dt), 16)
                out.append(f"{MN} {acc}, {v(VF + 4 * (g % RING), 4)}, {v(pprev + 4 * (4 * qi + u), 4)}, {acc}")
                out += head[k]
                k += 1
        for g in (2 * g2 + VAHEAD, 2 * g2 + VAHEAD + 1):
            if g < 16:
                out += order.issue(("V", uid, g), v_reads(g, slot_v, RING))
        # slots freed by the V fragments take the first eight K fragments of phase A
        first_k = {5: range(0, 4), 6: range(4, 6), 7: range(6, 8)}.get(g2, ())
        for f in first_k:
            out += order.issue(("K", uid, f), [k_read(f, slot_k, RING)])
    # ---- end of B
    out += rescale_block(f"{uid}")
    out.append("s_waitcnt vmcnt(8)")
    out.append("s_barrier")
    # the eight loads of K(j+4), V(j+3): M0 (the LDS target) is written one MFMA ahead of its load
    loads = []
    for i in range(4):
        so = "0" if i == 0 else f"s{72 + i - 1}"
        loads.append((f"s_add_u32 m0, %[m0b], {load_k * KTILE + i * 4096}", f"buffer_load_dwordx4 {v(GK)}, %[rk], {so} offen lds"))
        loads.append((f"s_add_u32 m0, %[m0b], {VRING + load_v * KTILE + i * 4096}", f"buffer_load_dwordx4 {v(GV)}, %[rv], {so} offen lds"))
    # ---- phase A: S(j+1) = K . Q^T  ||  second half of the softmax
    k = 0
    for f2 in range(8):
        out.append(order.wait_for({("K", uid, 2 * f2), ("K", uid, 2 * f2 + 1)}))
        for f in (2 * f2, 2 * f2 + 1):
            st, t = f // 2, f % 2
            for qi in range(NQ):
                if k < len(loads):
                    out.append(loads[k][0])
                d = v(s_out + 16 * (2 * qi + t), 16)
                c = "0" if st == 0 else d
                out.append(f"{MN} {d}, {v(KF + 4 * (f % RING), 4)}, {a(4 * (8 * qi + st), 4)}, {c}")
                out += tail[k]
                if k < len(loads):
                    out.append(loads[k][1])
                if k == len(loads) - 1:
                    out.append(f"v_add_u32 {v(GK)}, {KTILE}, {v(GK)}")
                    out.append(f"v_add_u32 {v(GV)}, {KTILE}, {v(GV)}")
                k += 1
        for f in (2 * f2 + 8, 2 * f2 + 9):
            if f < 16:
                out += order.issue(("K", uid, f), [k_read(f, slot_k, RING)])
        # V(j): the first fragments of the next body, into the slots the K fragments leave
        nxt = {4: (0, 1), 5: (2, 3), 6: (4, 5)}.get(f2, ())
        for g in nxt:
            out += order.issue(("V", uid + 1, g), v_reads(g, n % 4, RING))
    return out


def loop():
    out = ["s_mov_b32 s72, 4096", "s_mov_b32 s73, 8192", "s_mov_b32 s74, 12288", "s_mov_b32 s76, 0", "s_mov_b32 s77, m0"]
    # the waits are those of the steady state: a first trip through the four bodies sets up the order
    # of the reads in flight, the second one is emitted (on entry fewer reads are in flight than the
    # waits allow for, which only makes them stricter)
    order = LdsOrder()
    warm = loop_prefetch(order, 0, 3)
    for n in range(4):
        body(n, order, n)
    out += warm
    out.append("L_fa_loop_%=:")
    for n in range(4):
        out += body(n, order, 4 + n)
        out.append("s_add_u32 s76, s76, 1")
        if n < 3:
            out.append("s_cmp_ge_u32 s76, %[count]")
            out.append("s_cbranch_scc1 L_fa_done_%=")
        else:
            out.append("s_cmp_lt_u32 s76, %[count]")
            out.append("s_cbranch_scc1 L_fa_loop_%=")
    out.append("L_fa_done_%=:")
    out.append("s_waitcnt lgkmcnt(0)")       # the prefetched fragments land in registers the caller owns again
    out.append("s_mov_b32 m0, s77")
    out += ["s_nop 15", "s_nop 15"]          # the last scores must be readable by what follows
    return out


def scores0():
    """S(0) = K(0) . Q^T into S buffer 0 (no other work to pair it with)."""
    out = [k_read(f, 0) for f in range(4)]
    for f in range(16):
        st, t = f // 2, f % 2
        out.append(f"s_waitcnt lgkmcnt({min(3, 15 - f)})")
        for qi in range(NQ):
            d = v(SBUF[0] + 16 * (2 * qi + t), 16)
            c = "0" if st == 0 else d
            out.append(f"{MN} {d}, {v(KF + 4 * (f % 4), 4)}, {a(4 * (8 * qi + st), 4)}, {c}")
        if f + 4 < 16:
            out.append(k_read(f + 4, 0))
    out += ["s_nop 15", "s_nop 15"]
    return out


NEGINF, LIM = 112, 114


def mask_stream(qi, sbase):
    """Scores of keys past a lane's limit become -inf.  Register i of a query block holds key
    32*(i/16) + 8*((i%16)/4) + i%4 (+ 4 for the upper 32 lanes, folded into the limit)."""
    cond = f"s[{78 + 2 * qi}:{79 + 2 * qi}]"
    out = []
    for i in range(32):
        key = 32 * (i // 16) + 8 * ((i % 16) // 4) + i % 4
        r = sbase + 32 * qi + i
        out.append(f"v_cmp_gt_i32 {cond}, {key}, {v(LIM + qi)}")
        out.append(f"v_cndmask_b32 {v(r)}, {v(r)}, {v(NEGINF)}, {cond}")
    return out


def final():
    """Last block j of a wave, which may need masking: O += V(j-1)^T . P(j-1)^T next to the
    whole softmax of S(j) (in S buffer 0; P(j-1) in set Y, P(j) to set X), then the rescale.
    The V fragment addresses already include the ring slot."""
    valu = [f"v_mov_b32 {v(NEGINF)}, 0xff800000"]
    valu += interleave(mask_stream(0, SBUF[0]) + softmax_stream(0, SBUF[0], PX),
                       mask_stream(1, SBUF[0]) + softmax_stream(1, SBUF[0], PX))
    parts = [[], []] + chunks(valu, 30)
    out = v_prefetch(0)
    k = 0
    for g in range(16):
        u, dt = g // 4, g % 4
        out.append(f"s_waitcnt lgkmcnt({min(6, 2 * (15 - g))})")
        for qi in range(NQ):
            acc = a(128 + 16 * (4 * qi + dt), 16)
            out.append(f"{MN} {acc}, {v(VF + 4 * (g % 4), 4)}, {v(PY + 4 * (4 * qi + u), 4)}, {acc}")
            out += parts[k]
            k += 1
        if g + 4 < 16:
            out += v_reads(g + 4, 0)
    out += rescale_block("f")
    out += ["s_nop 4"]
    return out


def pv_tail():
    """O += V(j)^T . P(j)^T for the last block (P in set X)."""
    out = v_prefetch(0)
    for g in range(16):
        u, dt = g // 4, g % 4
        out.append(f"s_waitcnt lgkmcnt({min(6, 2 * (15 - g))})")
        for qi in range(NQ):
            acc = a(128 + 16 * (4 * qi + dt), 16)
            out.append(f"{MN} {acc}, {v(VF + 4 * (g % 4), 4)}, {v(PX + 4 * (4 * qi + u), 4)}, {acc}")
        if g + 4 < 16:
            out += v_reads(g + 4, 0)
    out += ["s_nop 15", "s_nop 15"]
    return out


def emit(lines):
    print("    asm volatile(")
    for ln in lines:
        print(f'        "{ln}\\n"')


def clobbers(vregs, sregs=()):
    return ", ".join([f'"v{i}"' for i in vregs] + [f'"s{i}"' for i in sregs] + ['"vcc"', '"scc"', '"memory"'])


O_OPS = '"+{a[128:159]}"(o0), "+{a[160:191]}"(o1), "+{a[192:223]}"(o2), "+{a[224:255]}"(o3)'
FRAGS = list(range(KF, KF + 16))
RING_FRAGS = list(range(KF, KF + 4 * RING))
TEMPS = list(range(ALPHA, ALPHA + 14))


def emit_all(dt):
    # ---- scores of block 0
    print("// S(0) = K(0) . Q^T into (s0, s1).")
    print(f"__device__ __forceinline__ void fa_pipe_scores0_{dt}(f32x32& s0, f32x32& s1, u32x32 q0, u32x32 q1, u32x8 kaddr) {{")
    emit(scores0())
    print(f'        : "={{v[{SBUF[0]}:{SBUF[0] + 31}]}}"(s0), "={{v[{SBUF[0] + 32}:{SBUF[0] + 63}]}}"(s1)')
    print(f'        : "{{a[0:31]}}"(q0), "{{a[32:63]}}"(q1), "{{v[{KADDR}:{KADDR + 7}]}}"(kaddr)')
    print("        : " + clobbers(FRAGS) + ");")
    print("}\n")
    # ---- steady state
    print("// Blocks 0 .. count-1, none of which needs masking.  Entered with the raw scores of block 0")
    print("// in (s0, s1) and zeros in py; after `count` bodies the raw scores of block `count` are in")
    print("// (s0, s1) when count is even, else in (s2, s3), and the probabilities of block count-1 in")
    print("// py when count is even, else in px.")
    print(f"__device__ __forceinline__ void fa_pipe_loop_{dt}(f32x32& o0, f32x32& o1, f32x32& o2, f32x32& o3,")
    print("        f32x32& s0, f32x32& s1, f32x32& s2, f32x32& s3, u32x32& px, u32x32& py, f32x4& state, u32x2& goff,")
    print("        u32x32 q0, u32x32 q1, u32x8 kaddr, u32x4 vaddr,")
    print("        __amdgpu_buffer_rsrc_t rk, __amdgpu_buffer_rsrc_t rv, float c, uint32_t m0b, uint32_t count) {")
    emit(loop())
    print("        : " + O_OPS + ",")
    print(f'          "+{{v[{SBUF[0]}:{SBUF[0] + 31}]}}"(s0), "+{{v[{SBUF[0] + 32}:{SBUF[0] + 63}]}}"(s1),')
    print(f'          "={{v[{SBUF[1]}:{SBUF[1] + 31}]}}"(s2), "={{v[{SBUF[1] + 32}:{SBUF[1] + 63}]}}"(s3),')
    print(f'          "={{v[{PX}:{PX + 31}]}}"(px), "+{{v[{PY}:{PY + 31}]}}"(py), "+{{v[{MREF}:{MREF + 3}]}}"(state),')
    print(f'          "+{{v[{GK}:{GV}]}}"(goff)')
    print(f'        : "{{a[0:31]}}"(q0), "{{a[32:63]}}"(q1), "{{v[{KADDR}:{KADDR + 7}]}}"(kaddr), "{{v[{VADDR}:{VADDR + 3}]}}"(vaddr),')
    print('          [rk] "s"(rk), [rv] "s"(rv), [c] "s"(c), [m0b] "s"(m0b), [count] "s"(count)')
    print("        : " + clobbers(RING_FRAGS + TEMPS, range(72, 86)) + ");")
    print("}\n")
    # ---- last block
    print("// Last block of a wave: raw scores in (s0, s1), probabilities of the block before it in py,")
    print("// lim = per-lane index of the last key of the block that is kept (minus 4 in the upper 32")
    print("// lanes), vaddr = V fragment addresses of the block before it.  Leaves P in px.")
    print(f"__device__ __forceinline__ void fa_pipe_final_{dt}(f32x32& o0, f32x32& o1, f32x32& o2, f32x32& o3,")
    print("        f32x32& s0, f32x32& s1, u32x32& px, u32x32 py, f32x4& state, u32x4 vaddr, u32x2 lim, float c) {")
    emit(final())
    print("        : " + O_OPS + ",")
    print(f'          "+{{v[{SBUF[0]}:{SBUF[0] + 31}]}}"(s0), "+{{v[{SBUF[0] + 32}:{SBUF[0] + 63}]}}"(s1),')
    print(f'          "={{v[{PX}:{PX + 31}]}}"(px), "+{{v[{MREF}:{MREF + 3}]}}"(state)')
    print(f'        : "{{v[{PY}:{PY + 31}]}}"(py), "{{v[{VADDR}:{VADDR + 3}]}}"(vaddr), "{{v[{LIM}:{LIM + 1}]}}"(lim), [c] "s"(c)')
    print("        : " + clobbers(FRAGS + TEMPS + [NEGINF], range(78, 86)) + ");")
    print("}\n")
    # ---- last product
    print("// O += V(j)^T . P(j)^T for the last block: P in px, vaddr = V fragment addresses of block j.")
    print(f"__device__ __forceinline__ void fa_pipe_pv_{dt}(f32x32& o0, f32x32& o1, f32x32& o2, f32x32& o3, u32x32 px, u32x4 vaddr) {{")
    emit(pv_tail())
    print("        : " + O_OPS)
    print(f'        : "{{v[{PX}:{PX + 31}]}}"(px), "{{v[{VADDR}:{VADDR + 3}]}}"(vaddr)')
    print("        : " + clobbers(FRAGS) + ");")
    print("}")



def main():
    global MN, CVT
    print("// Generated by gen_fa_loop.py -- do not edit by hand.")
    print("// Hand-scheduled pieces of the pipelined flash-attention kernel; the generator documents")
    print("// the schedule and the register map.\n")
    for dt in ("bf16", "f16"):
        MN = f"v_mfma_f32_32x32x16_{dt}"
        CVT = f"v_cvt_pk_{dt}_f32"
        print(f"// ---- {dt} ----\n")
        emit_all(dt)


if __name__ == "__main__":
    main()
