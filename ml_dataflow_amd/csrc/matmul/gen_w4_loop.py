#!/usr/bin/env python3
"""Writes gemm_w4_loop.inc: the k-loop of the four-wave GEMM kernel (gemm_bf16_w4_kernel in gemm_w4_kernel.h) as
inline-assembly text, one macro per variant.  Run by the Makefile; the output is a build product.

The kernel: 256 threads, one wave per SIMD, work-group tile 256 (m) x BN (n) x 64 (k), wave w owns rows
[64 w, 64 w + 64) of the m side and all BN columns: 4 x NB blocks of 16 x 16 (NB = BN / 16 = 16 or 18), accumulated with
v_mfma_f32_16x16x32_bf16.  Accumulators of column blocks 0..15 live in a[0:255], those of blocks 16, 17 in v[0:31].

One asm statement multiplies all k-tiles of one output tile.  Operands reach the LDS through registers: k-tile g+2 is
requested from global memory (buffer_load_dwordx4 into register set g & 1) at the start of step g, k-tile g+1 -- requested
a step earlier into the other set -- is written to the LDS stage (g + 1) & 1 with ds_write_b128 during the second half
of step g, and the barrier near the end of the step publishes it.  A load so has almost two k-tiles of multiplies to
arrive, where a load that goes straight into a free LDS stage (two stages fill the LDS) has one.

State across statements (tile to tile): LDS stage 0 holds k-tile 0 of the tile and is visible to all waves, register
set 1 (in/out operand) holds k-tile 1, landed.  The statement loads the next tile's first two k-tiles the same way while
it multiplies its own last two; k-tile counts are even.

Step g (stage p = g & 1), MFMA m = 0 .. 8 NB - 1 in the order k-step, column block j, row block i:
  * fragment of Q for column block b (counted over both k-steps) goes to ring slot b % 4, read right after the last
    MFMA of block b - 4;
  * the four P fragments of k-step 1 are read during k-step 0 into the second P buffer, those of k-step 0 of the next
    k-tile behind the barrier;
  * load q of k-tile g+2 goes out behind column q of k-step 0, the cursor arithmetic (scalar) behind the last load;
  * write q of k-tile g+1 is spread over k-step 1, each behind the s_waitcnt vmcnt that covers exactly its load;
  * after MFMA 8 NB - 9: s_waitcnt lgkmcnt(0), s_barrier, then the first reads of stage 1 - p.
s_waitcnt lgkmcnt values come from a simulation of the in-order LDS queue.
"""
import os
import sys

P_STAGE = 32768          # bytes of one P stage (256 rows x 64 k)

# schedule parameters (W4_OPTS="key=value,..." overrides them for experiments; ablations give wrong results, timing only)
OPTS = {"loads_per_column": 1, "write_start": 0.0, "abl": ""}
for kv in os.environ.get("W4_OPTS", "").split(","):
    if "=" in kv:
        k_, v_ = kv.split("=", 1)
        OPTS[k_] = type(OPTS[k_])(v_)
ABL = set(OPTS["abl"].split("+")) if OPTS["abl"] else set()


class Variant:
    def __init__(self, NB, PKM, GATHER):
        self.NB, self.PKM, self.GATHER = NB, PKM, GATHER
        self.BN = NB * 16
        self.Q_STAGE = self.BN * 128
        self.NLD_P = 8
        self.NLD_Q = self.BN * 8 // 256
        self.NLD = self.NLD_P + self.NLD_Q
        base = 32 if NB == 18 else 0
        self.SET = [base, base + 4 * self.NLD]
        self.AF = base + 8 * self.NLD
        self.BF = self.AF + 32
        self.VOFFP = self.BF + 16
        self.VOFFQ = self.VOFFP + 8
        self.ARD = self.VOFFQ + 9
        self.BRD = self.ARD + 4
        self.WRP = self.BRD + 4
        self.WRQ = self.WRP + 1
        self.MAPA = self.WRQ + 2
        self.KCH = self.MAPA + 1
        self.TMP = self.KCH + 1
        self.LANE_BLOCK = self.VOFFP                 # 32 registers from here are the lane-constant in/out operands
        assert self.TMP < self.LANE_BLOCK + 32
        self.LAST_VGPR = self.LANE_BLOCK + 31
        assert self.LAST_VGPR <= 247
        self.name = "W4_LOOP_NB%d_%s_%s" % (NB, "PKM" if PKM else "PKC", "GATHER" if GATHER else "PACKED")
        self.L = []
        # LDS queue simulation
        self.issued = 0
        self.prod = {}
        self.known_done = -1

    # ---------------------------------------------------------------- helpers
    def e(self, x):
        if "oob" in ABL and x.startswith("s_cselect_b32 s66,"):
            x = "s_mov_b32 s66, 0"
        if "oob" in ABL and x.startswith("s_cselect_b32 s70,"):
            x = "s_mov_b32 s70, 0"
        if ("noloads" in ABL and x.startswith("buffer_load")) or ("nowrites" in ABL and x.startswith("ds_write")) or \
           ("nobar" in ABL and x == "s_barrier") or ("nomfma" in ABL and x.startswith("v_mfma")) or \
           ("noreads" in ABL and x.startswith("ds_read_b") and "b32" not in x) or ("novm" in ABL and x.startswith("s_waitcnt vmcnt") and "lgkm" not in x) or \
           ("nolgkm" in ABL and x.startswith("s_waitcnt lgkmcnt")):
            return
        self.L.append(x)

    def vr(self, lo, n):
        return "v%d" % lo if n == 1 else "v[%d:%d]" % (lo, lo + n - 1)

    def acc(self, i, j):
        if j < 16:
            lo = (j * 4 + i) * 4
            return "a[%d:%d]" % (lo, lo + 3)
        lo = (j - 16) * 16 + i * 4
        return "v[%d:%d]" % (lo, lo + 3)

    def lds(self, text, key=None):
        self.e(text)
        if key is not None:
            self.prod[key] = self.issued
        self.issued += 1

    def need(self, *keys):
        n = max(self.prod.get(k, -1) for k in keys)
        if n > self.known_done:
            after = self.issued - 1 - n
            assert 0 <= after <= 15, after
            self.e("s_waitcnt lgkmcnt(%d)" % after)
            self.known_done = n

    def lds_drain(self):
        self.e("s_waitcnt lgkmcnt(0)")
        self.known_done = self.issued - 1

    # ---------------------------------------------------------------- LDS traffic
    def read_A(self, stage, s, i, buf):
        dst = self.AF + buf * 16 + i * 4
        if not self.PKM:
            self.lds("ds_read_b128 %s, v%d offset:%d" % (self.vr(dst, 4), self.ARD + s, stage * P_STAGE + i * 2048), ("A", buf, i))
        else:
            off = stage * P_STAGE + s * 32 * 512
            self.lds("ds_read_b64_tr_b16 %s, v%d offset:%d" % (self.vr(dst, 2), self.ARD + i, off))
            self.lds("ds_read_b64_tr_b16 %s, v%d offset:%d" % (self.vr(dst + 2, 2), self.ARD + i, off + 4 * 512), ("A", buf, i))

    def read_B(self, stage, b):
        s, j = divmod(b, self.NB)
        dst = self.BF + (b % 4) * 4
        self.lds("ds_read_b128 %s, v%d offset:%d" % (self.vr(dst, 4), self.BRD + s * 2 + stage, j * 2048), ("B", b % 4))

    def write(self, stage, setidx, q):
        src = self.vr(self.SET[setidx] + 4 * q, 4)
        if q < self.NLD_P:
            self.lds("ds_write_b128 v%d, %s offset:%d" % (self.WRP, src, stage * P_STAGE + q * 4096))
        else:
            self.lds("ds_write_b128 v%d, %s offset:%d" % (self.WRQ + stage, src, (q - self.NLD_P) * 4096))

    def tail_reads(self, stage, which):
        """first reads of a k-tile out of `stage`: which 0 = behind the barrier, 1 / 2 = the two later Q fragments"""
        if which == 0:
            self.read_B(stage, 0)
            for i in range(4):
                self.read_A(stage, 0, i, 0)
            self.read_B(stage, 1)
        elif which == 1:
            self.read_B(stage, 2)
        else:
            self.read_B(stage, 3)

    # ---------------------------------------------------------------- global loads and the cursor
    def load(self, setidx, q):
        dst = self.vr(self.SET[setidx] + 4 * q, 4)
        if q < self.NLD_P:
            return "buffer_load_dwordx4 %s, v%d, s[64:67], 0 offen" % (dst, self.VOFFP + q)
        return "buffer_load_dwordx4 %s, v%d, s[68:71], 0 offen" % (dst, self.VOFFQ + q - self.NLD_P)

    def set_cursor(self, src):
        """cursor <- the eight dwords at s[src:src+7]: P base lo, hi, extent lo, hi, then the same of Q"""
        out = []
        for (d, ext, o) in ((64, 72, 0), (68, 74, 4)):
            out += ["s_mov_b32 s%d, s%d" % (d, src + o), "s_mov_b32 s%d, s%d" % (d + 1, src + o + 1),
                    "s_mov_b32 s%d, s%d" % (ext, src + o + 2), "s_mov_b32 s%d, s%d" % (ext + 1, src + o + 3),
                    "s_cmp_lg_u32 s%d, 0" % (ext + 1), "s_cselect_b32 s%d, -1, s%d" % (d + 2, ext),
                    "s_mov_b32 s%d, 0x00020000" % (d + 3)]
        return out

    def advance(self):
        """cursor one k-tile on: base += ktile, extent -= ktile (not below zero), num_records = min(extent, 2^32 - 1)"""
        out = []
        for (d, ext, kt) in ((64, 72, 58), (68, 74, 59)):
            out += ["s_add_u32 s%d, s%d, s%d" % (d, d, kt), "s_addc_u32 s%d, s%d, 0" % (d + 1, d + 1),
                    "s_sub_u32 s%d, s%d, s%d" % (ext, ext, kt), "s_subb_u32 s%d, s%d, 0" % (ext + 1, ext + 1),
                    "s_cselect_b32 s%d, 0, s%d" % (ext, ext), "s_cselect_b32 s%d, 0, s%d" % (ext + 1, ext + 1),
                    "s_cmp_lg_u32 s%d, 0" % (ext + 1), "s_cselect_b32 s%d, -1, s%d" % (d + 2, ext)]
        return out

    def fetch_map(self, map_sgpr):
        """gathered Q: this lane's row offsets of a tile from the staged row map in LDS (drains the LDS queue)"""
        self.e("v_add_u32 v%d, s%d, v%d" % (self.TMP, map_sgpr, self.MAPA))
        for q in range(self.NLD_Q):
            self.lds("ds_read_b32 v%d, v%d offset:%d" % (self.VOFFQ + q, self.TMP, q * 128))
        self.lds_drain()
        for q in range(self.NLD_Q):
            self.e("v_add_u32 v%d, v%d, v%d" % (self.VOFFQ + q, self.VOFFQ + q, self.KCH))

    # ---------------------------------------------------------------- one step
    def step(self, p):
        NB, NLD = self.NB, self.NLD
        total = 8 * NB
        after = {}

        def at(m, fn):
            after.setdefault(m, []).append(fn)

        # Q fragments b >= 4 of this k-tile
        for b in range(4, 2 * NB):
            at(4 * b - 13, lambda b=b: self.read_B(p, b))
        # P fragments of k-step 1
        for i in range(4):
            at(4 * (NB - 6 + i) + 1, lambda i=i: self.read_A(p, 1, i, 1))
        # loads of k-tile g+2 into set p, then the cursor moves on
        lpc = OPTS["loads_per_column"]
        for q in range(NLD):
            at(4 * (q // lpc) + 1 + (q % lpc) * (4 // lpc if lpc <= 4 else 0), lambda q=q: self.e(self.load(p, q)))
        adv = self.advance()
        m0 = 4 * ((NLD - 1) // lpc) + 4
        for n, ins in enumerate(adv):
            at(m0 + n // 2, lambda ins=ins: self.e(ins))
        assert m0 + len(adv) // 2 < total - 12
        # writes of k-tile g+1 (set 1-p) into stage 1-p
        first_w, last_w = 4 * NB + 1 + int(OPTS["write_start"] * (4 * NB - 15)), total - 14
        for q in range(NLD):
            m = first_w + (q * (last_w - first_w)) // (NLD - 1)

            def w(q=q):
                self.e("s_waitcnt vmcnt(%d)" % (NLD + NLD - 1 - q))
                self.write(1 - p, 1 - p, q)
            at(m, w)

        def barrier():
            self.lds_drain()
            self.e("s_barrier")
            self.tail_reads(1 - p, 0)
        at(total - 9, barrier)
        at(total - 5, lambda: self.tail_reads(1 - p, 1))
        at(total - 1, lambda: self.tail_reads(1 - p, 2))
        if p == 1:
            at(total - 4, lambda: self.e("s_add_u32 s76, s76, 2"))
            at(total - 3, lambda: self.e("s_cmp_lt_u32 s76, s56"))

        for m in range(total):
            s, rem = divmod(m, 4 * NB)
            j, i = divmod(rem, 4)
            b = s * NB + j
            self.need(("A", s, i), ("B", b % 4))
            self.e("v_mfma_f32_16x16x32_bf16 %s, %s, %s, %s" % (self.acc(i, j), self.vr(self.AF + s * 16 + i * 4, 4),
                                                              self.vr(self.BF + (b % 4) * 4, 4), self.acc(i, j)))
            for fn in after.get(m, []):
                fn()

    def loop_head_state(self):
        """the LDS queue as every step finds it: the first reads of its k-tile pending, in their order, nothing else"""
        self.issued, self.known_done, self.prod = 0, -1, {}
        keep, self.L = self.L, []
        for which in range(3):
            self.tail_reads(0, which)
        self.L = keep

    # ---------------------------------------------------------------- the statement
    def generate(self):
        e = self.e
        NLD = self.NLD
        # s[40:47] this tile's cursor at k-tile 0, s[48:55] the next tile's, s56 k-tiles (even), s57 bit 0: first tile of the
        # work-group, s58 / s59 bytes per k-tile of P / Q, s60 / s61 LDS address of this / the next tile's row map
        e("s_mov_b32 s76, 0")
        for ins in self.set_cursor(40):
            e(ins)
        if self.GATHER:
            self.fetch_map(60)
        e("s_bitcmp1_b32 s57, 0")
        e("s_cbranch_scc1 1f")
        for ins in self.advance() + self.advance():
            e(ins)
        e("s_branch 2f")
        e("1:")
        # first tile: k-tiles 0 and 1 from global memory, k-tile 0 into stage 0
        for setidx in range(2):
            for q in range(NLD):
                e(self.load(setidx, q))
            for ins in self.advance():
                e(ins)
        for q in range(NLD):
            e("s_waitcnt vmcnt(%d)" % (NLD + NLD - 1 - q))
            self.write(0, 0, q)
        self.lds_drain()
        e("s_barrier")
        e("2:")
        self.tail_reads(0, 0)
        self.tail_reads(0, 1)
        self.tail_reads(0, 2)
        e("3:")
        self.loop_head_state()
        # the loads of this step fetch k-tile g+2: at g + 2 == k-tiles that is the next tile's first
        e("s_add_u32 s77, s76, 2")
        e("s_cmp_eq_u32 s77, s56")
        e("s_cbranch_scc0 4f")
        for ins in self.set_cursor(48):
            e(ins)
        if self.GATHER:
            saved = (self.issued, dict(self.prod), self.known_done)
            self.fetch_map(61)
            self.issued, self.prod, self.known_done = saved      # the skipping path has drained nothing
        e("4:")
        self.step(0)
        self.loop_head_state()
        self.step(1)
        e("s_cbranch_scc1 3b")
        e("s_waitcnt vmcnt(0) lgkmcnt(0)")
        e("s_nop 7")
        e("s_nop 7")
        e("s_nop 7")
        return self.L

    def clobbers(self):
        v = ["v%d" % i for i in range(self.SET[0], self.SET[1])] + ["v%d" % i for i in range(self.AF, self.LANE_BLOCK)]
        s = ["s%d" % i for i in range(64, 80)]
        return v + s + ["scc", "vcc", "memory"]


def main():
    out = sys.argv[1] if len(sys.argv) > 1 else os.path.join(os.path.dirname(os.path.abspath(__file__)), "gemm_w4_loop.inc")
    with open(out, "w") as f:
        f.write("/* generated by gen_w4_loop.py -- do not edit */\n")
        for NB in (16, 18):
            for PKM in (False, True):
                for GATHER in (False, True):
                    v = Variant(NB, PKM, GATHER)
                    lines = v.generate()
                    f.write("#define %s_ASM \\\n" % v.name + " \\\n".join('\t"%s\\n\\t"' % x for x in lines) + "\n")
                    f.write("#define %s_CLOBBERS %s\n" % (v.name, ", ".join('"%s"' % c for c in v.clobbers())))
            v = Variant(NB, False, False)
            f.write("#define W4_NB%d_SET1 %d\n#define W4_NB%d_LANE_BLOCK %d\n#define W4_NB%d_NLD %d\n" % (NB, v.SET[1], NB, v.LANE_BLOCK, NB, v.NLD))
            for nm in ("VOFFP", "VOFFQ", "ARD", "BRD", "WRP", "WRQ", "MAPA", "KCH"):
                f.write("#define W4_NB%d_%s %d\n" % (NB, nm, getattr(v, nm) - v.LANE_BLOCK))
            # in/out operands, pinned to the registers the text names: accumulator groups g[0..NB-1] (16 registers per
            # column block), register set 1 (st[0..3], and st4 for the 288-wide tile), the two lane-constant blocks
            ops = ['"+{a[%d:%d]}"(g[%d])' % (16 * j, 16 * j + 15, j) for j in range(16)]
            ops += ['"+{v[%d:%d]}"(g[%d])' % (16 * (j - 16), 16 * (j - 16) + 15, j) for j in range(16, NB)]
            ops += ['"+{v[%d:%d]}"(st[%d])' % (v.SET[1] + 16 * n, v.SET[1] + 16 * n + 15, n) for n in range(4)]
            if 4 * v.NLD > 64:
                ops += ['"+{v[%d:%d]}"(st4)' % (v.SET[1] + 64, v.SET[1] + 67)]
            ops += ['"+{v[%d:%d]}"(lb0)' % (v.LANE_BLOCK, v.LANE_BLOCK + 15), '"+{v[%d:%d]}"(lb1)' % (v.LANE_BLOCK + 16, v.LANE_BLOCK + 31)]
            f.write("#define W4_NB%d_OUTPUTS(g, st, st4, lb0, lb1) %s\n" % (NB, ", ".join(ops)))
        f.write('#define W4_INPUTS(sa, sb, sc) "{s[40:47]}"(sa), "{s[48:55]}"(sb), "{s[56:63]}"(sc)\n')


if __name__ == "__main__":
    main()
