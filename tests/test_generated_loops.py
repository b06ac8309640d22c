"""Host-side check of the generated inline-assembly loops (gemm256_loop.inc, gemm_twoset_loop.inc, fa_loop.inc): every register an
assembly block writes must be declared to the compiler as an output, an in/out operand or a
clobber.  A persistent kernel calls these blocks several times and keeps values live across them,
so one undeclared write lets the compiler reuse a register the block has changed (seen once: a
fragment address input whose upper elements the loop derives was taken for a known zero)."""
import os
import re

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(os.path.dirname(HERE), "metalhlo_amd", "csrc")
INCS = [os.path.join(CSRC, "gemm256_loop.inc"), os.path.join(CSRC, "gemm_twoset_loop.inc"), os.path.join(CSRC, "fa_loop.inc")]

NO_DEST = ("s_waitcnt", "s_barrier", "s_nop", "s_cbranch", "s_cmp", "s_branch", "buffer_load", "global_store",
           "ds_write")


def _regs(tok):
    tok = tok.strip()
    m = re.fullmatch(r"([vas])\[(\d+):(\d+)\]", tok)
    if m:
        return {f"{m.group(1)}{i}" for i in range(int(m.group(2)), int(m.group(3)) + 1)}
    return {tok} if re.fullmatch(r"[vas]\d+", tok) else set()


def _blocks():
    for inc in INCS:
        yield from _blocks_of(open(inc).read())


def _blocks_of(src):
    for f in re.split(r"\n(?=__device__ __forceinline__ void )", src)[1:]:
        name = re.match(r"__device__ __forceinline__ void (\w+)", f).group(1)
        lines = re.findall(r'^\s+"(.*?)\\n"$', f, re.M)
        outs, ins, clob = f[f.index("        : "):].split("\n        : ")[:3]
        declared = set()
        for m in re.finditer(r'"[=+]\{([vas])\[(\d+):(\d+)\]\}"', outs):
            declared |= {f"{m.group(1)}{i}" for i in range(int(m.group(2)), int(m.group(3)) + 1)}
        declared |= set(re.findall(r'"([vas]\d+)"', clob))
        yield name, lines, declared


def test_every_written_register_is_declared():
    names = []
    for name, lines, declared in _blocks():
        names.append(name)
        written = set()
        for line in lines:
            op, _, rest = line.partition(" ")
            if op.endswith(":") or op.startswith(NO_DEST):
                continue
            dst = rest.split(",")[0].strip()
            if dst in ("m0", "exec"):
                continue                      # m0 is saved and restored by every block; exec is never written
            regs = _regs(dst)
            assert regs, f"{name}: destination of '{line}' not understood"
            written |= regs
        assert written, name
        assert not (written - declared), f"{name} writes undeclared registers {sorted(written - declared)}"
    for stem in ("gemm_stream_loop_", "gemm256_loop_", "gemm256x128_loop_", "gemm256x384_loop_", "gemm_pair_loop_", "gemm128x192_loop_", "gemm256x288_loop_", "fa_pipe_loop_"):
        assert any(n.startswith(stem) for n in names), stem


def test_m0_is_restored_and_exec_untouched():
    for name, lines, _ in _blocks():
        assert not any(re.match(r"s_\w+ exec", l) for l in lines), name
        writes_m0 = [i for i, l in enumerate(lines) if re.match(r"s_\w+ m0,", l)]
        if writes_m0:
            save = [i for i, l in enumerate(lines) if re.match(r"s_mov_b32 s\d+, m0", l)]
            assert save and save[0] < writes_m0[0], f"{name}: m0 written before it is saved"
            assert re.match(r"s_mov_b32 m0, s\d+", lines[writes_m0[-1]]), f"{name}: m0 not restored last"
