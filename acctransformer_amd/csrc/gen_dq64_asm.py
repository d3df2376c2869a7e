#!/usr/bin/env python3
"""Writes fa_bwd_dq64_asm.inc: the hand-scheduled tile loop of the dQ kernel that gives every wave 64 query rows
(one wave per SIMD, 512 registers).  Run by hand after editing (python3 gen_dq64_asm.py); the output is committed.

The work on one 32-key chunk i of the key axis (two chunks per 64-key tile), for the wave's 32-row groups A and B:

    SP(i):   S^T  = K Q^T        (A operand: K fragments from LDS, 16-byte reads; B: the Q fragments, resident in AGPRs)
             dP^T = V dO^T       (A: V fragments from LDS; B: the dO fragments, resident in AGPRs)         32 MFMAs
    VALU(i): dS^T = P^T o (dP^T - D),  P^T = exp2(S^T * scale*log2e - LSE*log2e), packed to the I/O type   ~150 vector ops
    DQ(i):   dQ^T += K^T dS^T    (A: K^T fragments by transposed LDS reads; B: dS^T; C/D: AGPRs)           16 MFMAs

Every LDS fragment feeds two MFMAs (groups A and B): half the LDS bytes per flop of the 32-rows-per-wave kernel.
A lone wave per SIMD has nobody to overlap with, so the loop is software-pipelined by hand, three chunks deep:
one step issues the MFMAs of SP(i+1) and DQ(i-1) with VALU(i) spread evenly behind them (about three vector
instructions per MFMA, which the matrix pipe hides).  An iteration of the loop is two such steps (tile j):

    step 1:  SP(2j+1)  [tile j]    DQ(2j-1) [tile j-1]   VALU(2j)
    wait for the DMA of tile j+1, workgroup barrier (everybody is done with tile j-1), request tile j+2 into its buffer
    step 2:  SP(2j+2)  [tile j+1]  DQ(2j)   [tile j]     VALU(2j+1)

with three K/V tile buffers in LDS.  Before the loop SP(0) runs alone and the dS^T registers of chunk -1 are zeroed
(its DQ step then adds nothing; it reads K^T of tile 0 so that the other operand is finite).  A wave's last tile
(the one with its diagonal under the causal mask, else the last of the workgroup) runs a closing body: step 2
without SP, then DQ of the last chunk.  After it the wave only keeps its share of the DMA and the barriers going.

LDS fragments go through a ring of eight 4-register slots, requested DIST fragments ahead of their MFMAs, across
steps and across the loop's back edge.  The reads of tile j+1 may not start before the barrier: every step's
fragment stream therefore opens with DIST fragments of DQ (tile j, long landed).

Fixed register map (the kernel pins its operands to these registers with physical-register constraints):
    a[0:127]    dQ^T accumulators: group g, 32-column block db of the head dim at a[64 g + 16 db : +15]
    a[128:191]  Q fragments  (group g, k-step t at a[128 + 32 g + 4 t : +3])
    a[192:255]  dO fragments (group g, k-step t at a[192 + 32 g + 4 t : +3])
    v[96:103]   byte offsets of the row-major fragment of k-step t inside a tile (lane = key row)
    v[104:107]  byte offsets of the transposed fragment of block db inside a tile
    v108, v109  -LSE*log2e (+ shift) of the lane's row, groups A and B;  v110, v111  D of that row
    v[116:119], v[120:123]  per-lane byte offsets of this wave's four DMA instructions of a K tile, of a V tile
    v124, v125  row of the lane in groups A and B, minus the lane's first key inside a 32-key chunk
    scratch inside the loop: v[16:23] addresses of the SP tile's fragments, v[24:27] of the DQ tile's,
    v[28:43] / v[44:59] dS^T fragments of even / odd chunks, v[60:91] fragment ring,
    v[112:115] last visible key per [group][chunk] (diagonal tile), v[128:191] / v[192:255] S and dP of even / odd chunks
Scalar registers of the loop: s80 tile j, s81 / s92 LDS address of the buffers of tiles j, j+1, s91 of the buffer
    that tile j+2 streams into (tile j-1's), s[82:83] / s[84:85] global address of the K / V rows of tile j+2
    (clamped to the last tile), s87 first key of tile j, s88 / s90 scratch.
"""
import argparse
import os

# Classes of instructions left out of the tile body (--leave-out): for timing builds only, the results are wrong.
# What a class costs the kernel is the time of the complete build minus the time of the build without it.
LEAVE_OUT = set()

NSLOT, DIST = 8, 6        # fragment ring: slots of four registers at v[60:91]; fragments in flight ahead of their MFMAs
TILEB = 64 * 256          # bytes of a 64-key tile (256-byte rows); a buffer is a K tile followed by a V tile
PITCH = 256
VALU_NAMES = ("v_fma_f32", "v_exp_f32_e32", "v_sub_f32_e32", "v_mul_f32_e32", "v_cmp_gt_i32_e32", "v_cndmask_b32_e64",
              "v_cvt_pk_f16_f32", "v_cvt_pk_bf16_f32")


def tr_hi(db):
    return 8 * PITCH + (-128 if (db >> 1) & 1 else 128)


# ---- fragments: what to read from LDS and the two MFMAs (groups A, B) it feeds -------------------------------------
class Frag:
    def __init__(self, reads, mfmas):
        self.reads, self.mfmas = reads, mfmas       # both: functions of the ring slot's first register


def frag_sp(mfma, c, idx):
    """fragment idx (0..7 K for the S product, 8..15 V for the dP product) of the score products of a chunk of parity c"""
    t, is_v = idx % 8, idx >= 8
    off = (TILEB if is_v else 0) + c * 32 * PITCH

    def reads(sl):
        return [f"ds_read_b128 v[{sl}:{sl + 3}], v{16 + t} offset:{off}"]

    def mfmas(sl):
        out = []
        for g in range(2):
            acc = 128 + 64 * c + (32 if is_v else 0) + 16 * g
            b = (192 if is_v else 128) + 32 * g + 4 * t
            cin = "0" if t == 0 else f"v[{acc}:{acc + 15}]"
            out.append(f"{mfma} v[{acc}:{acc + 15}], v[{sl}:{sl + 3}], a[{b}:{b + 3}], {cin}")
        return out
    return Frag(reads, mfmas)


def frag_dq(mfma, c, idx):
    """fragment idx = 4 hh + db (16-key half hh of the chunk, 32-column block db) of the dQ product of a chunk of parity c"""
    hh, db = divmod(idx, 4)
    off = 16 * (2 * c + hh) * PITCH

    def reads(sl):
        return [f"ds_read_b64_tr_b16 v[{sl}:{sl + 1}], v{24 + db} offset:{off}",
                f"ds_read_b64_tr_b16 v[{sl + 2}:{sl + 3}], v{24 + db} offset:{off + tr_hi(db)}"]

    def mfmas(sl):
        out = []
        for g in range(2):
            acc = 64 * g + 16 * db
            ds = 28 + 16 * c + 8 * g + 4 * hh
            out.append(f"{mfma} a[{acc}:{acc + 15}], v[{sl}:{sl + 3}], v[{ds}:{ds + 3}], a[{acc}:{acc + 15}]")
        return out
    return Frag(reads, mfmas)


def step_stream(mfma, c_sp, c_dq):
    """fragment order of one step: DIST fragments of DQ first (see the module text), the rest threaded into SP"""
    dq = [frag_dq(mfma, c_dq, i) for i in range(8)]
    sp = [frag_sp(mfma, c_sp, i) for i in range(16)]
    assert DIST == 6
    return dq[:6] + sp[0:2] + dq[6:7] + sp[2:4] + dq[7:8] + sp[4:]


def valu_ops(cvt, c, edge):
    """vector work of a chunk of parity c: dS^T fragments from the score and dP accumulators"""
    ops = []
    S = lambda g, r: 128 + 64 * c + 16 * g + r
    P = lambda g, r: 128 + 64 * c + 32 + 16 * g + r
    for g in range(2):
        for r in range(16):
            ops.append(f"v_fma_f32 v{S(g, r)}, v{S(g, r)}, %[scale], v{108 + g}")
    for g in range(2):
        for r in range(16):
            ops.append(f"v_exp_f32_e32 v{S(g, r)}, v{S(g, r)}")
    if edge:
        for g in range(2):
            for r in range(16):
                k = 8 * (r >> 2) + (r & 3)
                ops.append(f"v_cmp_gt_i32_e32 vcc, {k}, v{112 + 2 * g + c}")
                ops.append(f"v_cndmask_b32_e64 v{S(g, r)}, v{S(g, r)}, 0, vcc")
    for g in range(2):
        for r in range(16):
            ops.append(f"v_sub_f32_e32 v{P(g, r)}, v{P(g, r)}, v{110 + g}")
    for g in range(2):
        for r in range(16):
            ops.append(f"v_mul_f32_e32 v{S(g, r)}, v{S(g, r)}, v{P(g, r)}")
    for g in range(2):
        for hh in range(2):
            for i in range(4):
                d = 28 + 16 * c + 8 * g + 4 * hh + i
                ops.append(f"{cvt} v{d}, v{S(g, 8 * hh + 2 * i)}, v{S(g, 8 * hh + 2 * i + 1)}")
    return ops


class Code:
    """Instruction list with an LDS read counter: the LDS returns data in order, so a wait names how many reads
    issued after the wanted one may still be in flight."""

    def __init__(self, outstanding):
        self.lines = []
        self.issued = 0
        self.tickets = {}
        # fragments requested by the code that runs before this one (stream positions 0 .. outstanding-1, all DQ)
        for i in range(outstanding):
            self.issued += 2
            self.tickets[i] = self.issued

    def emit(self, s):
        op = s.split()[0]
        if "dma" in LEAVE_OUT and (op == "global_load_lds_dwordx4" or s.startswith("s_mov_b32 m0")):
            return
        if "valu" in LEAVE_OUT and op in VALU_NAMES:
            return
        if "exp" in LEAVE_OUT and op == "v_exp_f32_e32":
            return
        if "lds" in LEAVE_OUT and (op.startswith("ds_read") or s.startswith("s_waitcnt lgkmcnt")):
            return
        if "mfma" in LEAVE_OUT and op.startswith("v_mfma"):
            return
        self.lines.append(s)

    def read(self, pos, frag):
        for r in frag.reads(60 + 4 * (pos % NSLOT)):
            self.emit(r)
            self.issued += 1
        self.tickets[pos] = self.issued

    def wait_for(self, pos):
        assert self.issued - self.tickets[pos] <= 15
        self.emit(f"s_waitcnt lgkmcnt({self.issued - self.tickets[pos]})")


def dma(code, n):
    """instruction n (0..7) of this wave's share of the DMA of tile j+2: K rows 0..3, V rows 4..7"""
    e = code.emit
    if n == 0:
        e("s_add_u32 s88, s91, %[lds0]")
    elif n == 4:
        e(f"s_add_u32 s88, s88, {TILEB - 4096}")
    e("s_mov_b32 m0, s88")
    e("s_add_u32 s88, s88, 1024")
    e(f"global_load_lds_dwordx4 v{(116 if n < 4 else 120) + n % 4}, s[{82 if n < 4 else 84}:{83 if n < 4 else 85}]")


def run_stream(code, stream, first_pos, following, pending, hooks, dma_from=None):
    """Issue the MFMAs of `stream` (ring positions first_pos ..) with the vector instructions in `pending` spread
    evenly behind them; once the stream's own fragments are all requested the ring goes on with `following`'s.
    hooks[k]: code emitted before fragment k of the stream is consumed.  dma_from: stream index from which the eight
    DMA instructions follow every second fragment."""
    e = code.emit
    n = len(stream)
    total = 2 * n
    done = 0
    n_dma = 0
    for k, frag in enumerate(stream):
        for h in hooks.get(k, []):
            h()
        pos = first_pos + k
        code.wait_for(pos)
        for m in frag.mfmas(60 + 4 * (pos % NSLOT)):
            e(m)
            done += 1
            left = total - done + 1
            for _ in range(min(len(pending), -(-len(pending) // left))):
                e(pending.pop(0))
        if dma_from is not None and k >= dma_from and (k - dma_from) % 2 == 0 and n_dma < 8:
            dma(code, n_dma)
            n_dma += 1
        # request the fragment DIST positions ahead (its slot was read by the MFMAs two fragments back)
        ahead = k + DIST
        if ahead < n:
            code.read(first_pos + ahead, stream[ahead])
        elif following is not None and ahead - n < len(following):
            code.read(first_pos + ahead, following[ahead - n])
    while dma_from is not None and n_dma < 8:
        dma(code, n_dma)
        n_dma += 1
    while pending:
        e(pending.pop(0))


def addr_sp(code, base):
    for t in range(8):
        code.emit(f"v_add_u32_e32 v{16 + t}, {base}, v{96 + t}")


def addr_dq(code, base):
    for db in range(4):
        code.emit(f"v_add_u32_e32 v{24 + db}, {base}, v{104 + db}")


def barrier(code):
    # the tile requested one iteration ago has landed for every wave; every wave is done with tile j-1
    code.emit("s_waitcnt vmcnt(0)")
    code.emit("s_barrier")


def body(mfma, cvt, edge, closing):
    """one iteration of the loop (tile j).  closing: the wave's last tile."""
    code = Code(DIST)
    e = code.emit
    s1 = step_stream(mfma, 1, 1)            # SP(2j+1), DQ(2j-1)
    s2 = step_stream(mfma, 0, 0)            # SP(2j+2), DQ(2j)
    if edge:
        # last visible key of the lane's row relative to the lane's first key of the chunk: [group][chunk]
        e("v_subrev_u32_e32 v112, s87, v124")
        e("v_subrev_u32_e32 v113, 32, v112")
        e("v_subrev_u32_e32 v114, s87, v125")
        e("v_subrev_u32_e32 v115, 32, v114")
    e("s_nop 1")                            # (the last conversions of the step before wrote B operands of the MFMAs that follow)
    # the DQ addresses move to tile j before step 2's first fragment is requested (while fragment 24 - DIST of step 1
    # is consumed); the SP addresses move to tile j+1 at the barrier, before its first read
    hooks1 = {len(s1) - DIST: [lambda: addr_dq(code, "s81")]}
    if not closing:
        run_stream(code, s1, 0, s2, valu_ops(cvt, 0, edge), hooks1)
        e("s_nop 1")
        hooks2 = {0: [lambda: barrier(code), lambda: addr_sp(code, "s92")]}
        run_stream(code, s2, len(s1), s1, valu_ops(cvt, 1, edge), hooks2, dma_from=0)
    else:
        dq0 = [frag_dq(mfma, 0, i) for i in range(8)]
        dq1 = [frag_dq(mfma, 1, i) for i in range(8)]
        run_stream(code, s1, 0, dq0, valu_ops(cvt, 0, edge), hooks1)
        e("s_nop 1")
        hooks2 = {0: [lambda: barrier(code)]}
        run_stream(code, dq0, len(s1), dq1, valu_ops(cvt, 1, edge), hooks2, dma_from=0)
        e("s_nop 1")                        # chunk 2j+1's dS^T fragments are complete before its products start
        run_stream(code, dq1, len(s1) + 8, None, [], {})
    return code.lines


def first_step(mfma):
    """before the loop: SP(0) alone; leaves the first DIST fragments of the loop's stream requested"""
    code = Code(0)
    e = code.emit
    e("s_waitcnt lgkmcnt(0)")               # nothing foreign in the LDS / scalar-load queue: the waits count this code's reads
    addr_sp(code, "s81")
    addr_dq(code, "s81")
    for r in range(44, 60):
        e(f"v_mov_b32_e32 v{r}, 0")
    sp0 = [frag_sp(mfma, 0, i) for i in range(16)]
    s1 = step_stream(mfma, 1, 1)
    for i in range(DIST):
        code.read(i, sp0[i])
    run_stream(code, sp0, 0, s1, [], {})
    return code.lines


def idle():
    code = Code(0)
    barrier(code)
    for n in range(8):
        dma(code, n)
    return code.lines


def clobbers():
    regs = list(range(16, 92)) + list(range(112, 116)) + list(range(128, 256))
    sregs = [80, 81, 82, 83, 84, 85, 87, 88, 90, 91, 92]
    return ", ".join(f'"v{r}"' for r in regs) + ", " + ", ".join(f'"s{r}"' for r in sregs) + ', "vcc", "scc", "memory"'


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--leave-out", default="", help="comma list of dma, valu, exp, lds, mfma: a timing build without them")
    ap.add_argument("--out", default=os.path.join(os.path.dirname(os.path.abspath(__file__)), "fa_bwd_dq64_asm.inc"))
    args = ap.parse_args()
    LEAVE_OUT.update(filter(None, args.leave_out.split(",")))
    assert LEAVE_OUT <= {"dma", "valu", "exp", "lds", "mfma"}, LEAVE_OUT
    out = ["// Generated by gen_dq64_asm.py -- do not edit.  Tile loop of fa_bwd_dq64_kernel: see the generator for the",
           "// schedule and the register map.", ""]
    variants = [("F16", "v_mfma_f32_32x32x16_f16", "v_cvt_pk_f16_f32"), ("BF16", "v_mfma_f32_32x32x16_bf16", "v_cvt_pk_bf16_f32")]
    # One asm statement per element type holds the whole loop, so that the pinned operands are set up once.
    for name, mfma, cvt in variants:
        out.append(f"#define DQ64_LOOP_{name} \\")
        L = []
        # tiles 0 and 1 are in the first two buffers; the first iteration's DQ step reads tile 0 (see the module text)
        L += ["s_mov_b32 s80, 0", "s_mov_b32 s81, %[kbuf0]", f"s_add_u32 s92, %[kbuf0], {2 * TILEB}", f"s_add_u32 s91, %[kbuf0], {4 * TILEB}",
              "s_mov_b64 s[82:83], %[kptr]", "s_mov_b64 s[84:85], %[vptr]", "s_mov_b32 s87, 0"]
        L += first_step(mfma)
        L += [".Ldq64_loop_%=:"]
        # what the wave does with tile j: past its last tile nothing, on it a closing body, before it the interior body
        L += ["s_cmp_gt_u32 s80, %[jlast]", "s_cbranch_scc1 .Ldq64_idle_%=",
              "s_cmp_lt_u32 s80, %[jlast]", "s_cbranch_scc1 .Ldq64_interior_%=",
              "s_cmp_eq_u32 %[lastedge], 0", "s_cbranch_scc1 .Ldq64_close_%="]
        L += body(mfma, cvt, True, True)
        L += ["s_branch .Ldq64_end_%=", ".Ldq64_close_%=:"]
        L += body(mfma, cvt, False, True)
        L += ["s_branch .Ldq64_end_%=", ".Ldq64_idle_%=:"]
        L += idle()
        L += ["s_branch .Ldq64_end_%=", ".Ldq64_interior_%=:"]
        L += body(mfma, cvt, False, False)
        L += [".Ldq64_end_%=:"]
        L += ["s_add_u32 s80, s80, 1", "s_add_u32 s87, s87, 64",
              # buffers of tiles j, j+1 and the DMA target <- those of j+1, j+2 (where the DMA just went), and tile j's
              "s_mov_b32 s88, s91", "s_mov_b32 s91, s81", "s_mov_b32 s81, s92", "s_mov_b32 s92, s88",
              # advance the DMA source to tile j+2 (of the new j) unless it already points at the last tile
              "s_add_u32 s88, s80, 1", "s_cmp_lt_u32 s88, %[jhi]", "s_cselect_b32 s88, %[kstep], 0", "s_cselect_b32 s90, %[vstep], 0",
              "s_add_u32 s82, s82, s88", "s_addc_u32 s83, s83, 0", "s_add_u32 s84, s84, s90", "s_addc_u32 s85, s85, 0",
              "s_cmp_le_u32 s80, %[jhi]", "s_cbranch_scc1 .Ldq64_loop_%="]
        # the LDS is the caller's again once every wave's DMA has landed; the caller reads the accumulators, and an
        # MFMA result is not interlocked against vector reads
        L += ["s_waitcnt vmcnt(0)", "s_barrier", "s_nop 15", "s_nop 7"]
        for ln in L:
            out.append(f'  "{ln}\\n\\t" \\')
        out.append('  ""')
        out.append("")
    out.append(f"#define DQ64_CLOBBERS {clobbers()}")
    out.append("")
    with open(args.out, "w") as f:
        f.write("\n".join(out))
    n_mfma = sum(1 for ln in body(variants[0][1], variants[0][2], False, False) if ln.startswith("v_mfma"))
    print(f"wrote {args.out}: {n_mfma} MFMAs per tile")


if __name__ == "__main__":
    main()
