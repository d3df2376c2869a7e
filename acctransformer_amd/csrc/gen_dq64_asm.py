#!/usr/bin/env python3
"""Writes fa_bwd_dq64_asm.inc: the hand-scheduled tile body of the dQ kernel that gives every wave 64 query rows
(one wave per SIMD, 512 registers).  Run by hand after editing (python3 gen_dq64_asm.py); the output is committed.

One call of the block processes one K/V tile of 64 keys for the wave's two 32-row groups A and B:

    S^T  = K Q^T        (A operand: K fragments from LDS, 16-byte reads; B: the Q fragments, resident in AGPRs)
    dP^T = V dO^T       (A: V fragments from LDS; B: the dO fragments, resident in AGPRs)
    dS^T = P^T o (dP^T - D),  P^T = exp2(S^T * scale*log2e - LSE*log2e)
    dQ^T += K^T dS^T    (A: K^T fragments by transposed LDS reads; B: dS^T packed to the I/O type; C/D: AGPRs)

Every LDS fragment feeds two MFMAs (groups A and B): half the LDS bytes per flop of the 32-rows-per-wave kernel.
A lone wave per SIMD has nobody to overlap with, so the block is software-pipelined by hand over the tile's two
32-key chunks: the vector work of chunk c (exp2, products, conversions) is issued between the MFMAs of the score
products of chunk c+1 and of the dQ product of chunk c-1 ... a few vector instructions after every MFMA.

Fixed register map (the kernel pins its operands to these registers with physical-register constraints):
    a[0:127]    dQ^T accumulators: group g, 32-column block db of the head dim at a[64 g + 16 db : +15]
    a[128:191]  Q fragments  (group g, k-step t at a[128 + 32 g + 4 t : +3])
    a[192:255]  dO fragments (group g, k-step t at a[192 + 32 g + 4 t : +3])
    v[96:103]   byte offsets of the row-major fragment of k-step t inside a tile (lane = key row)
    v[104:107]  byte offsets of the transposed fragment of block db inside a tile
    v108, v109  -LSE*log2e (+ shift) of the lane's row, groups A and B;  v110, v111  D of that row
    v[116:119], v[120:123]  per-lane byte offsets of this wave's four DMA instructions of a K tile, of a V tile
    v124, v125  row of the lane in groups A and B, minus the lane's first key inside a 32-key chunk
    scratch inside the block: v[16:27] addresses, v[28:59] dS^T fragments, v[60:91] fragment ring,
    v[112:115] last visible key per [group][chunk] (edge tiles), v[128:255] score / dP accumulators of the two chunks
"""
import argparse
import os

# Classes of instructions left out of the tile body (--leave-out): for timing builds only, the results are wrong.
# What a class costs the kernel is the time of the complete build minus the time of the build without it.
LEAVE_OUT = set()

NSLOT, DIST = 8, 6          # fragment ring: slots of four registers at v[60:91]; fragments in flight ahead of their MFMAs
TILEB = 64 * 256          # bytes of a 64-key tile (256-byte rows)
PITCH = 256


def tr_hi(db):
    return 8 * PITCH + (-128 if (db >> 1) & 1 else 128)


class Block:
    def __init__(self, mfma, cvt, edge):
        self.mfma, self.cvt, self.edge = mfma, cvt, edge
        self.lines = []
        self.issued = 0          # LDS reads issued so far (in order)
        self.tickets = {}        # fragment -> number of reads issued when its last read was

    def emit(self, s):
        if "dma" in LEAVE_OUT and (s.startswith("global_load_lds") or s.startswith("s_mov_b32 m0")):
            return
        if "valu" in LEAVE_OUT and s.split()[0] in ("v_fma_f32", "v_exp_f32_e32", "v_sub_f32_e32", "v_mul_f32_e32", "v_cmp_gt_i32_e32",
                                                   "v_cndmask_b32_e64", "v_cvt_pk_f16_f32", "v_cvt_pk_bf16_f32"):
            return
        if "exp" in LEAVE_OUT and s.startswith("v_exp_f32"):
            return
        if "lds" in LEAVE_OUT and (s.startswith("ds_read") or s.startswith("s_waitcnt lgkmcnt")):
            return
        if "mfma" in LEAVE_OUT and s.startswith("v_mfma"):
            return
        self.lines.append(s)

    # ---- LDS reads, tracked so that waits can be exact (the LDS returns data in order) ----
    # One stream of 48 fragments per tile: 0..31 row-major (chunk c = i // 16: K fragments of the S product for
    # i % 16 < 8, then V fragments of the dP product), 32..47 transposed K^T fragments (chunk, half hh, block db).
    def slot(self, i):
        return 60 + 4 * (i % NSLOT)

    def read(self, i):
        sl = self.slot(i)
        if i < 32:
            c, w = divmod(i, 16)
            t, is_v = w % 8, w >= 8
            self.emit(f"ds_read_b128 v[{sl}:{sl + 3}], v{16 + t} offset:{(TILEB if is_v else 0) + c * 32 * PITCH}")
            self.issued += 1
        else:
            c, w = divmod(i - 32, 8)
            hh, db = divmod(w, 4)
            off = 16 * (2 * c + hh) * PITCH
            self.emit(f"ds_read_b64_tr_b16 v[{sl}:{sl + 1}], v{24 + db} offset:{off}")
            self.emit(f"ds_read_b64_tr_b16 v[{sl + 2}:{sl + 3}], v{24 + db} offset:{off + tr_hi(db)}")
            self.issued += 2
        self.tickets[i] = self.issued

    def wait_for(self, i):
        self.emit(f"s_waitcnt lgkmcnt({self.issued - self.tickets[i]})")

    # ---- vector work of chunk c: dS^T fragments from the score and dP accumulators ----
    def valu_ops(self, c):
        ops = []
        S = lambda g, r: 128 + 64 * c + 16 * g + r
        P = lambda g, r: 128 + 64 * c + 32 + 16 * g + r
        for g in range(2):
            for r in range(16):
                ops.append(f"v_fma_f32 v{S(g, r)}, v{S(g, r)}, %[scale], v{108 + g}")
        for g in range(2):
            for r in range(16):
                ops.append(f"v_exp_f32_e32 v{S(g, r)}, v{S(g, r)}")
        if self.edge:
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
                    ops.append(f"{self.cvt} v{d}, v{S(g, 8 * hh + 2 * i)}, v{S(g, 8 * hh + 2 * i + 1)}")
        return ops

    def dma(self, n):
        """instruction n (0..7) of this wave's share of the next tile's DMA: K rows 0..3, V rows 4..7"""
        e = self.emit
        if n == 0:
            e("s_sub_u32 s88, %[ldssum], s81")
            e("s_add_u32 s88, s88, %[lds0]")
        elif n == 4:
            e(f"s_add_u32 s88, s88, {TILEB - 4096}")
        e("s_mov_b32 m0, s88")
        e("s_add_u32 s88, s88, 1024")
        e(f"global_load_lds_dwordx4 v{(116 if n < 4 else 120) + n % 4}, s[{82 if n < 4 else 84}:{83 if n < 4 else 85}]")

    def build(self):
        e = self.emit
        e("s_waitcnt lgkmcnt(0)")          # nothing foreign in the LDS / scalar-load queue: the waits below count this block's reads
        for t in range(8):
            e(f"v_add_u32_e32 v{16 + t}, s81, v{96 + t}")
        for db in range(4):
            e(f"v_add_u32_e32 v{24 + db}, s81, v{104 + db}")
        for i in range(DIST):
            self.read(i)
        nxt = DIST
        pending = []                      # vector instructions waiting for a slot behind an MFMA

        def drain(n):
            for _ in range(min(n, len(pending))):
                e(pending.pop(0))

        def prefetch():
            nonlocal nxt
            if nxt < 48:
                self.read(nxt)
                nxt += 1

        # ---- phases 1 and 2: score and dP products of chunks 0 and 1.  Phase 1 carries the next tile's DMA
        # instructions, one behind every fourth MFMA; the vector work of chunk 0 rides on chunk 1's MFMAs.
        for i in range(32):
            c, w = divmod(i, 16)
            t, is_v = w % 8, w >= 8
            if i == 16:
                pending.extend(self.valu_ops(0))
            sl = self.slot(i)
            self.wait_for(i)
            for g in range(2):
                acc = 128 + 64 * c + (32 if is_v else 0) + 16 * g
                b = (192 if is_v else 128) + 32 * g + 4 * t
                cin = "0" if t == 0 else f"v[{acc}:{acc + 15}]"
                e(f"{self.mfma} v[{acc}:{acc + 15}], v[{sl}:{sl + 3}], a[{b}:{b + 3}], {cin}")
                if c == 0 and g == 1 and i % 2 == 1:
                    self.dma(i // 2)
                if c == 1:
                    left = 2 * (32 - i) - g             # MFMAs left in this phase, this one included
                    drain(-(-len(pending) // left))
                if g == 1:
                    prefetch()                          # (the slot it fills was read by the MFMAs two fragments back)
        drain(len(pending))
        # ---- phases 3 and 4: dQ products of chunks 0 and 1; the vector work of chunk 1 rides on chunk 0's MFMAs
        e("s_nop 1")                       # (the last conversions wrote B operands of the MFMAs that follow)
        pending.extend(self.valu_ops(1))
        for i in range(32, 48):
            c, w = divmod(i - 32, 8)
            hh, db = divmod(w, 4)
            sl = self.slot(i)
            if i == 40:
                drain(len(pending))               # chunk 1's dS^T fragments are complete before its products start
                e("s_nop 1")
            self.wait_for(i)
            for g in range(2):
                acc = 64 * g + 16 * db
                ds = 28 + 16 * c + 8 * g + 4 * hh
                e(f"{self.mfma} a[{acc}:{acc + 15}], v[{sl}:{sl + 3}], v[{ds}:{ds + 3}], a[{acc}:{acc + 15}]")
                if c == 0:
                    left = 2 * (40 - i) - g
                    drain(-(-len(pending) // left))
                if g == 1:
                    prefetch()
        # the code after the block may read the accumulators: an MFMA result is not interlocked against vector reads
        e("s_nop 15")
        e("s_nop 7")
        return self.lines


def clobbers():
    regs = list(range(16, 92)) + list(range(112, 116)) + list(range(128, 256))
    sregs = [80, 81, 82, 83, 84, 85, 87, 88, 89, 90]
    return ", ".join(f'"v{r}"' for r in regs) + ", " + ", ".join(f'"s{r}"' for r in sregs) + ', "vcc", "scc", "memory"'


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--leave-out", default="", help="comma list of dma, valu, exp, lds, mfma: a timing build without them")
    ap.add_argument("--out", default=os.path.join(os.path.dirname(os.path.abspath(__file__)), "fa_bwd_dq64_asm.inc"))
    args = ap.parse_args()
    LEAVE_OUT.update(filter(None, args.leave_out.split(",")))
    assert LEAVE_OUT <= {"dma", "valu", "exp", "lds", "mfma"}, LEAVE_OUT
    out = ["// Generated by gen_dq64_asm.py -- do not edit.  Tile body of fa_bwd_dq64_kernel: see the generator for the",
           "// schedule and the register map.", ""]
    variants = [("F16", "v_mfma_f32_32x32x16_f16", "v_cvt_pk_f16_f32"), ("BF16", "v_mfma_f32_32x32x16_bf16", "v_cvt_pk_bf16_f32")]
    # One asm statement per element type holds the whole tile loop, so that the pinned operands are set up once:
    # DMA of the next tile, what the wave does with the current one (nothing / interior body / edge body), the
    # body, the wait for the DMA and the workgroup barrier.  Scalar registers of the loop: s80 tile index j, s81 LDS
    # address of the current K tile (V follows it), s[82:83] / s[84:85] global address of the next K / V tile,
    # s87 first key of the current tile, s88 scratch, s89 mode.
    for name, mfma, cvt in variants:
        out.append(f"#define DQ64_LOOP_{name} \\")
        L = []
        L += ["s_mov_b32 s80, 0", "s_mov_b32 s81, %[kbuf0]", "s_mov_b64 s[82:83], %[kptr]", "s_mov_b64 s[84:85], %[vptr]",
              "s_mov_b32 s87, 0", ".Ldq64_loop_%=:"]
        # s[82:85]: rows of the tile that streams into the other buffer while this one is worked on -- tile j + 1, or
        # the last tile once more (into a buffer nobody reads again) so that the bodies need no branch around their DMA
        # mode: 1 interior; causal: 2 when keys of the tile come after rows of the wave, 0 when all of them do
        L += ["s_mov_b32 s89, 1", "s_cmp_eq_u32 %[causal], 0", "s_cbranch_scc1 .Ldq64_mode_%=",
              "s_add_u32 s88, s87, 63", "s_cmp_gt_i32 s88, %[wq0]", "s_cselect_b32 s89, 2, 1",
              "s_cmp_gt_i32 s87, %[wq0p63]", "s_cselect_b32 s89, 0, s89", ".Ldq64_mode_%=:"]
        # last visible key of the lane's row relative to the lane's first key of the chunk: [group][chunk]
        L += ["v_subrev_u32_e32 v112, s87, v124", "v_subrev_u32_e32 v113, 32, v112",
              "v_subrev_u32_e32 v114, s87, v125", "v_subrev_u32_e32 v115, 32, v114"]
        L += ["s_cmp_lt_u32 s89, 2", "s_cbranch_scc0 .Ldq64_edge_%=", "s_cmp_eq_u32 s89, 0", "s_cbranch_scc1 .Ldq64_idle_%="]
        L += Block(mfma, cvt, False).build()
        L += ["s_branch .Ldq64_end_%=", ".Ldq64_edge_%=:"]
        L += Block(mfma, cvt, True).build()
        L += ["s_branch .Ldq64_end_%=", ".Ldq64_idle_%=:"]
        idle = Block(mfma, cvt, False)
        for n in range(8):
            idle.dma(n)
        L += idle.lines
        L += [".Ldq64_end_%=:"]
        # the tile requested above has landed; every wave is done with the current one
        L += ["s_waitcnt vmcnt(0)", "s_barrier", "s_add_u32 s80, s80, 1", "s_add_u32 s87, s87, 64", "s_sub_u32 s81, %[ldssum], s81",
              # advance the DMA source unless it already points at the last tile
              "s_cmp_lt_u32 s80, %[jhi]", "s_cselect_b32 s88, %[kstep], 0", "s_cselect_b32 s90, %[vstep], 0",
              "s_add_u32 s82, s82, s88", "s_addc_u32 s83, s83, 0", "s_add_u32 s84, s84, s90", "s_addc_u32 s85, s85, 0",
              "s_cmp_le_u32 s80, %[jhi]", "s_cbranch_scc1 .Ldq64_loop_%="]
        for ln in L:
            out.append(f'  "{ln}\\n\\t" \\')
        out.append('  ""')
        out.append("")
    out.append(f"#define DQ64_CLOBBERS {clobbers()}")
    out.append("")
    path = args.out
    with open(path, "w") as f:
        f.write("\n".join(out))
    n_mfma = sum(1 for ln in Block(variants[0][1], variants[0][2], False).build() if ln.startswith("v_mfma"))
    print(f"wrote {path}: {n_mfma} MFMAs per tile")


if __name__ == "__main__":
    main()
