#!/usr/bin/env python3
"""Writes gemm_w4_loop.inc: the k-loops of the four-wave GEMM kernels of gemm_w4_kernel.h as inline-assembly text
(gemm_bf16_w4_kernel: classes Mult and Loader, described here; gemm_bf16_w4d_kernel: class Wide, described there).  Run
by the Makefile; the output is a build product.

The kernel: 256 threads, one wave per SIMD, work-group tile 256 (m) x 288 (n) x 64 (k).  The waves have two roles.

  Wave 0 loads.  It requests the operands from global memory into its own registers (buffer_load_dwordx4 into
  accumulation registers, 68 chunks of 1 KiB per k-tile: 32 of P, 36 of Q, a chunk being eight rows of 128 bytes or, for
  a k-major operand, two k-rows of 256 rows) and writes them to the LDS stages with ds_write_b128.  The stream is a
  sequence of slots, 68 per k-tile; which chunk a slot carries (its global offset and its LDS address are per-slot
  registers) is up to the caller, who rotates the chunks by work-group so that the work-groups which share an operand
  panel ask for a given line at different times.  The stream is one sliding window: behind the write of slot t comes the
  load of slot t + 60, into the registers that the write of slot t - 8 has left, so 60 KiB are in flight at any time,
  also across k-tiles and barriers.  A wave that issues a load
  while the memory pipeline of the compute unit is full waits until the load is accepted; this wave has nothing else to do.
  Waves 1-3 multiply.  Wave w owns columns [96 (w - 1), 96 w) of the tile and all 256 rows: 16 x 6 blocks of 16 x 16,
  v_mfma_f32_16x16x32_bf16, accumulators in a[0:255] and v[0:127].  They read fragments from the LDS and never touch
  global memory, so nothing but the barrier ever holds their matrix instructions up.

One barrier per k-tile: when the loader has written k-tile g+1 and the multiplying waves have read the last fragment of
k-tile g.  One asm statement per role covers the k-tiles of one output tile.

State from statement to statement (tile to tile): LDS stage 0 holds k-tile 0 of the tile, visible to all waves; the
loader's registers hold chunks 0..59 of k-tile 1, landed (the statement ends with s_waitcnt vmcnt(0)); chunks 60..67 of
k-tile 1 are the first loads of the next statement.  k-tile counts are even; the loader fetches the next tile's first
k-tiles while the last ones of this tile are multiplied (a next tile that does not exist has an empty buffer: zeros).

Multiplying wave, step g (stage p = g & 1), MFMA m = 0..191 in the order k-step s, row block i, column block j:
  * the fragment of P for row block a = 16 s + i goes to ring slot a % 4, read right behind the last MFMA of block a - 4;
  * the six fragments of Q of k-step 1 are read during k-step 0 into the second buffer, those of k-step 0 of the next
    k-tile behind the barrier;
  * behind MFMA 179: s_waitcnt lgkmcnt(0), s_barrier, then the first reads of stage 1 - p; 12 MFMAs are left to cover them.
s_waitcnt lgkmcnt values come from a simulation of the in-order LDS queue.
"""
import os
import sys

P_STAGE = 32768          # bytes of one P stage (256 rows x 64 k)
Q_STAGE = 36864          # bytes of one Q stage (288 rows x 64 k)
CHUNKS_P, CHUNKS_Q = 32, 36
CHUNKS = CHUNKS_P + CHUNKS_Q
WINDOW = 60              # chunks in flight
LAG = CHUNKS - WINDOW

# loader registers
L_VOFFP, L_VOFFQ, L_VOFFQ_NEXT, L_WR = 16, 48, 84, 120        # v[0:15]: slots 64..67; then offsets; LDS write address of every slot
# multiplying-wave registers
M_BF, M_AF, M_ARD, M_BRD = 128, 176, 192, 200                 # v[0:127]: accumulator groups 16..23

# schedule parameters (W4_OPTS="key=value,..." overrides them for experiments; ablations give wrong results, timing only)
OPTS = {"abl": "", "pre": 4, "first": 2, "every": 3, "qfirst": 14, "qevery": 13}
for kv in os.environ.get("W4_OPTS", "").split(","):
    if "=" in kv:
        k_, v_ = kv.split("=", 1)
        OPTS[k_] = type(OPTS[k_])(v_)
ABL = set(OPTS["abl"].split("+")) if OPTS["abl"] else set()


class Asm:
    def __init__(self):
        self.L = []
        self.issued, self.prod, self.known_done = 0, {}, -1

    def e(self, x):
        if ("noloads" in ABL and x.startswith("buffer_load")) or ("nowrites" in ABL and x.startswith("ds_write")) or \
           ("nobar" in ABL and x == "s_barrier") or ("nomfma" in ABL and x.startswith("v_mfma")) or \
           ("noreads" in ABL and x.startswith("ds_read_b")) or ("nolgkm" in ABL and x.startswith("s_waitcnt lgkmcnt(") and not x.endswith("(0)")) or ("novm" in ABL and x.startswith("s_waitcnt vmcnt") and "lgkm" not in x):
            return
        if "oob" in ABL and (x.startswith("s_cselect_b32 s66,") or x.startswith("s_cselect_b32 s70,")):
            x = "s_mov_b32 s%s, 0" % x.split()[1][1:3]
        self.L.append(x)

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

    def barrier(self):
        self.e("s_barrier")

    def lds_drain(self):
        self.e("s_waitcnt lgkmcnt(0)")
        self.known_done = self.issued - 1


def vr(lo, n):
    return "v%d" % lo if n == 1 else "v[%d:%d]" % (lo, lo + n - 1)


# ================================================================================================ multiplying waves
class Mult(Asm):
    """s40: k-tiles (even), s41 bit 0: first tile of the work-group"""

    def __init__(self, PKM):
        Asm.__init__(self)
        self.PKM = PKM
        self.name = "W4_MULT_%s" % ("PKM" if PKM else "PKC")

    def acc(self, i, j):
        g = (i // 4) * 6 + j
        lo = (i % 4) * 4
        if g < 16:
            return "a[%d:%d]" % (16 * g + lo, 16 * g + lo + 3)
        return "v[%d:%d]" % (16 * (g - 16) + lo, 16 * (g - 16) + lo + 3)

    def read_A(self, stage, a):
        s, i = divmod(a, 16)
        dst = M_AF + (a % 4) * 4
        if not self.PKM:
            self.lds("ds_read_b128 %s, v%d offset:%d" % (vr(dst, 4), M_ARD + s, stage * P_STAGE + i * 2048), ("A", a % 4))
        else:
            off = stage * P_STAGE + s * 32 * 512 + (i // 8) * 256
            self.lds("ds_read_b64_tr_b16 %s, v%d offset:%d" % (vr(dst, 2), M_ARD + (i % 8), off))
            self.lds("ds_read_b64_tr_b16 %s, v%d offset:%d" % (vr(dst + 2, 2), M_ARD + (i % 8), off + 4 * 512), ("A", a % 4))

    def read_B(self, stage, s, j):
        dst = M_BF + s * 24 + j * 4
        self.lds("ds_read_b128 %s, v%d offset:%d" % (vr(dst, 4), M_BRD + s * 2 + stage, j * 2048), ("B", s, j))

    def tail_reads(self, stage, which):
        if which == 0:
            self.read_B(stage, 0, 0)
            self.read_A(stage, 0)
            for j in range(1, 6):
                self.read_B(stage, 0, j)
            self.read_A(stage, 1)
        else:
            self.read_A(stage, 1 + which)

    def loop_head_state(self):
        self.issued, self.known_done, self.prod = 0, -1, {}
        keep, self.L = self.L, []
        for which in range(3):
            self.tail_reads(0, which)
        self.L = keep

    def step(self, p):
        after = {}

        def at(m, fn):
            after.setdefault(m, []).append(fn)

        for a in range(4, 32):
            at(6 * (a - 4) + 5, lambda a=a: self.read_A(p, a))
        for j in range(6):
            at(30 + 6 * j + 2, lambda j=j: self.read_B(p, 1, j))

        def barrier():
            self.lds_drain()
            self.barrier()
            self.tail_reads(1 - p, 0)
        at(179, barrier)
        at(185, lambda: self.tail_reads(1 - p, 1))
        at(191, lambda: self.tail_reads(1 - p, 2))
        if p == 1:
            at(187, lambda: self.e("s_add_u32 s76, s76, 2"))
            at(188, lambda: self.e("s_cmp_lt_u32 s76, s40"))
        for m in range(192):
            s, rem = divmod(m, 96)
            i, j = divmod(rem, 6)
            a = s * 16 + i
            self.need(("A", a % 4), ("B", s, j))
            self.e("v_mfma_f32_16x16x32_bf16 %s, %s, %s, %s" % (self.acc(i, j), vr(M_AF + (a % 4) * 4, 4), vr(M_BF + s * 24 + j * 4, 4), self.acc(i, j)))
            for fn in after.get(m, []):
                fn()

    def generate(self):
        e = self.e
        e("s_mov_b32 s76, 0")
        e("s_bitcmp1_b32 s41, 0")
        e("s_cbranch_scc0 2f")
        e("s_barrier")                      # first tile: the loader has written k-tile 0
        e("2:")
        for which in range(3):
            self.tail_reads(0, which)
        e("3:")
        self.loop_head_state()
        self.step(0)
        self.loop_head_state()
        self.step(1)
        e("s_cbranch_scc1 3b")
        e("s_waitcnt lgkmcnt(0)")
        for _ in range(3):
            e("s_nop 7")
        return self.L

    def clobbers(self):
        return ["v%d" % i for i in range(M_BF, M_ARD)] + ["s76", "scc", "memory"]


# ================================================================================================ loader wave
class Loader(Asm):
    """s[40:47] this tile's cursor at k-tile 0 (P base lo, hi, extent lo, hi, then Q), s[48:55] the next tile's,
    s56 k-tiles (even), s57 bit 0: first tile of the work-group, s58 / s59 bytes per k-tile of P / Q.
    Working registers: s[64:67] / s[68:71] buffer descriptors of P / Q at the k-tile being loaded, s[72:73] / s[74:75]
    bytes left from there, s76 the k-tile being written, s77 scratch."""

    def __init__(self, GATHER):
        Asm.__init__(self)
        self.GATHER = GATHER
        self.name = "W4_LOAD_%s" % ("GATHER" if GATHER else "PACKED")

    def chunk_regs(self, c):
        return "a[%d:%d]" % (4 * c, 4 * c + 3) if c < 64 else "v[%d:%d]" % (4 * (c - 64), 4 * (c - 64) + 3)

    def load(self, c):
        if c < CHUNKS_P:
            self.e("buffer_load_dwordx4 %s, v%d, s[64:67], 0 offen" % (self.chunk_regs(c), L_VOFFP + c))
        else:
            self.e("buffer_load_dwordx4 %s, v%d, s[68:71], 0 offen" % (self.chunk_regs(c), L_VOFFQ + c - CHUNKS_P))

    def write(self, stage, c):
        self.lds("ds_write_b128 v%d, %s offset:%d" % (L_WR + c, self.chunk_regs(c), stage * (P_STAGE if c < CHUNKS_P else Q_STAGE)))

    def set_cursor(self, src):
        for (d, ext, o) in ((64, 72, 0), (68, 74, 4)):
            for ins in ("s_mov_b32 s%d, s%d" % (d, src + o), "s_mov_b32 s%d, s%d" % (d + 1, src + o + 1),
                        "s_mov_b32 s%d, s%d" % (ext, src + o + 2), "s_mov_b32 s%d, s%d" % (ext + 1, src + o + 3),
                        "s_cmp_lg_u32 s%d, 0" % (ext + 1), "s_cselect_b32 s%d, -1, s%d" % (d + 2, ext),
                        "s_mov_b32 s%d, 0x00020000" % (d + 3)):
                self.e(ins)

    def advance(self):
        """cursor one k-tile on: base += ktile, extent -= ktile (not below zero), num_records = min(extent, 2^32 - 1)"""
        for (d, ext, kt) in ((64, 72, 58), (68, 74, 59)):
            for ins in ("s_add_u32 s%d, s%d, s%d" % (d, d, kt), "s_addc_u32 s%d, s%d, 0" % (d + 1, d + 1),
                        "s_sub_u32 s%d, s%d, s%d" % (ext, ext, kt), "s_subb_u32 s%d, s%d, 0" % (ext + 1, ext + 1),
                        "s_cselect_b32 s%d, 0, s%d" % (ext, ext), "s_cselect_b32 s%d, 0, s%d" % (ext + 1, ext + 1),
                        "s_cmp_lg_u32 s%d, 0" % (ext + 1), "s_cselect_b32 s%d, -1, s%d" % (d + 2, ext)):
                self.e(ins)

    def step(self, stage, check_switch):
        """writes the k-tile s76 into `stage`; its chunks 60..67 and chunks 0..59 of the next k-tile are requested"""
        e = self.e
        for c in range(CHUNKS):
            e("s_waitcnt vmcnt(%d)" % (WINDOW - 1))
            self.write(stage, c)
            if c == LAG:
                # the loads move on to k-tile s76 + 1: of this tile, or the first of the next
                if check_switch:
                    e("s_add_u32 s77, s76, 1")
                    e("s_cmp_eq_u32 s77, s56")
                    e("s_cbranch_scc0 5f")
                    self.set_cursor(48)
                    if self.GATHER:
                        for q in range(CHUNKS_Q):
                            e("v_mov_b32 v%d, v%d" % (L_VOFFQ + q, L_VOFFQ_NEXT + q))
                    e("s_branch 6f")
                    e("5:")
                    self.advance()
                    e("6:")
                else:
                    self.advance()
            self.load(c + WINDOW if c < LAG else c - LAG)
        e("s_waitcnt lgkmcnt(0)")
        self.barrier()

    def generate(self):
        e = self.e
        self.set_cursor(40)
        e("s_bitcmp1_b32 s57, 0")
        e("s_cbranch_scc1 1f")
        self.advance()                       # chunks 0..59 of k-tile 1 are here; the next loads are its last eight
        e("s_branch 2f")
        e("1:")
        # first tile: request chunks 0..59 of k-tile 0, then the generic step writes it into stage 0
        for c in range(WINDOW):
            self.load(c)
        e("s_mov_b32 s76, 0")
        self.step(0, False)
        e("2:")
        e("s_mov_b32 s76, 1")
        e("3:")
        self.step(1, True)
        e("s_add_u32 s76, s76, 1")
        self.step(0, False)
        e("s_add_u32 s76, s76, 1")
        e("s_cmp_le_u32 s76, s56")
        e("s_cbranch_scc1 3b")
        e("s_waitcnt vmcnt(0)")
        return self.L

    def clobbers(self):
        return ["s%d" % i for i in range(64, 78)] + ["scc", "memory"]


# ================================================================================================ four symmetric waves, 256 x 384
QW_STAGE = 49152         # bytes of one Q stage of the wide tile (384 rows x 64 k)
D_VP, D_VQ, D_VQ_NEXT = 208, 216, 228                         # this lane's offsets of the wave's 8 chunks of P, 12 of Q, the next tile's Q


class Wide(Mult):
    """gemm_bf16_w4d_kernel: tile 256 (m) x 384 (n) x 64 (k), four waves that all do both jobs.  Wave w multiplies columns
    [96 w, 96 w + 96) of the tile like a multiplying wave above (same fragment reads, same MFMA order) and loads a quarter
    of every k-tile -- chunks 8 w .. 8 w + 7 of P and 12 w .. 12 w + 11 of Q, 20 KiB -- straight into the LDS
    (buffer_load_dwordx4 ... lds), so the two stages fill all 160 KiB and there is no epilogue scratch.

    The rows of Q that a wave loads are the rows it multiplies: nobody else reads them.  So the Q part of a stage needs no
    barrier: in step g (stage p = g & 1) the wave reads its fragments of Q for the second k-step first and, with them in
    registers, loads the Q rows of k-tile g + 2 into stage p (from MFMA `qfirst` on, every `qevery` MFMAs), with most of
    two steps to land.  P is
    read by all waves: behind MFMA 179 the wave waits for its loads of k-tile g + 1 (all but the twelve newest, which are
    the Q rows of k-tile g + 2: loads complete in order) and for its fragment reads of stage p, then the barrier; the P
    rows of k-tile g + 2 follow, `pre` of them behind MFMAs 180, 183, ... and the rest behind MFMAs first, first + every, ...
    of the next step.  Loads are in flight all the time, also across the barrier.

    The two cursors (buffer descriptors of P and of Q at the k-tile being loaded) move on where their loads begin; when
    the tile has no k-tile g + 2 they switch to the next tile's first one.

    s[40:47] this tile's cursor at k-tile 0, s[48:55] the next tile's (empty buffers when there is none), s56 k-tiles
    (even), s57 bit 0: first tile of the work-group, s58 / s59 bytes per k-tile of P / Q, s61 / s62 LDS address of the
    wave's first chunk of P / Q in stage 0.  Working registers as in the loader above.

    State from statement to statement: stage 0 holds k-tile 0 of the tile, visible to all waves; the Q rows and the first
    `pre` chunks of P of k-tile 1 are in flight into stage 1; the Q offsets of the tile are in v[D_VQ ...]."""

    LOADS_P, LOADS_Q = 8, 12

    def __init__(self, PKM, GATHER):
        Mult.__init__(self, PKM)
        self.GATHER = GATHER
        self.name = "W4D_%s_%s" % ("PKM" if PKM else "PKC", "GATHER" if GATHER else "PACKED")

    # which: 0 = P (descriptor s[64:67], bytes left s[72:73]), 1 = Q (s[68:71], s[74:75])
    def set_cursor(self, src, which):
        d, ext, o = ((64, 72, 0), (68, 74, 4))[which]
        for ins in ("s_mov_b32 s%d, s%d" % (d, src + o), "s_mov_b32 s%d, s%d" % (d + 1, src + o + 1),
                    "s_mov_b32 s%d, s%d" % (ext, src + o + 2), "s_mov_b32 s%d, s%d" % (ext + 1, src + o + 3),
                    "s_cmp_lg_u32 s%d, 0" % (ext + 1), "s_cselect_b32 s%d, -1, s%d" % (d + 2, ext),
                    "s_mov_b32 s%d, 0x00020000" % (d + 3)):
            self.e(ins)

    def advance(self, which):
        d, ext, kt = ((64, 72, 58), (68, 74, 59))[which]
        for ins in ("s_add_u32 s%d, s%d, s%d" % (d, d, kt), "s_addc_u32 s%d, s%d, 0" % (d + 1, d + 1),
                    "s_sub_u32 s%d, s%d, s%d" % (ext, ext, kt), "s_subb_u32 s%d, s%d, 0" % (ext + 1, ext + 1),
                    "s_cselect_b32 s%d, 0, s%d" % (ext, ext), "s_cselect_b32 s%d, 0, s%d" % (ext + 1, ext + 1),
                    "s_cmp_lg_u32 s%d, 0" % (ext + 1), "s_cselect_b32 s%d, -1, s%d" % (d + 2, ext)):
            self.e(ins)

    def dma_p(self, stage, u):
        self.e("s_add_u32 m0, s61, %d" % (stage * P_STAGE + u * 1024))
        self.e("s_nop 0")
        self.e("buffer_load_dwordx4 v%d, s[64:67], 0 offen lds" % (D_VP + u))

    def dma_q(self, stage, q):
        self.e("s_add_u32 m0, s62, %d" % (stage * QW_STAGE + q * 1024))
        self.e("s_nop 0")
        self.e("buffer_load_dwordx4 v%d, s[68:71], 0 offen lds" % (D_VQ + q))

    def move_on(self, which, check_switch):
        """cursor `which` to k-tile s76 + 2 (of this tile, or the first of the next)"""
        e = self.e
        if check_switch:
            e("s_add_u32 s77, s76, 2")
            e("s_cmp_eq_u32 s77, s56")
            e("s_cbranch_scc0 5f")
            self.set_cursor(48, which)
            if self.GATHER and which == 1:
                for q in range(12):
                    e("v_mov_b32 v%d, v%d" % (D_VQ + q, D_VQ_NEXT + q))
            e("s_branch 6f")
            e("5:")
            self.advance(which)
            e("6:")
        else:
            self.advance(which)

    def step(self, p):
        after = {}

        def at(m, fn):
            after.setdefault(m, []).append(fn)

        pre, first, every, qfirst, qevery = OPTS["pre"], OPTS["first"], OPTS["every"], OPTS["qfirst"], OPTS["qevery"]
        assert 1 <= pre <= 4 and first + every * (self.LOADS_P - pre - 1) < qfirst
        assert qfirst >= 8 and qfirst + qevery * (self.LOADS_Q - 1) < 179
        # the rest of the P rows of k-tile g + 1, into the other stage
        for n, u in enumerate(range(pre, self.LOADS_P)):
            at(first + every * n, lambda u=u: self.dma_p(1 - p, u))
        # the fragments of Q of k-step 1 first: with them in registers the wave's Q rows of this stage are free
        for j in range(6):
            at(j, lambda j=j: self.read_B(p, 1, j))
        # this wave's Q rows of k-tile g + 2, into the stage being multiplied
        at(qfirst, lambda: self.need(*[("B", 1, j) for j in range(6)]))
        at(qfirst, lambda: self.move_on(1, p == 0))
        for q in range(self.LOADS_Q):
            at(qfirst + qevery * q, lambda q=q: self.dma_q(p, q))
        for a in range(4, 32):
            at(6 * (a - 4) + 5, lambda a=a: self.read_A(p, a))

        def barrier():
            self.e("s_waitcnt vmcnt(%d)" % self.LOADS_Q)
            self.lds_drain()
            self.barrier()
            self.tail_reads(1 - p, 0)
        at(179, barrier)
        at(180, lambda: self.move_on(0, p == 0))
        for u in range(pre):
            at(180 + 3 * u, lambda u=u: self.dma_p(p, u))
        at(185, lambda: self.tail_reads(1 - p, 1))
        at(191, lambda: self.tail_reads(1 - p, 2))
        for m in range(192):
            s, rem = divmod(m, 96)
            i, j = divmod(rem, 6)
            a = s * 16 + i
            self.need(("A", a % 4), ("B", s, j))
            self.e("v_mfma_f32_16x16x32_bf16 %s, %s, %s, %s" % (self.acc(i, j), vr(M_AF + (a % 4) * 4, 4), vr(M_BF + s * 24 + j * 4, 4), self.acc(i, j)))
            for fn in after.get(m, []):
                fn()

    def generate(self):
        e = self.e
        self.set_cursor(40, 0)
        self.set_cursor(40, 1)
        e("s_mov_b32 s76, 0")
        e("s_bitcmp1_b32 s57, 0")
        e("s_cbranch_scc0 2f")
        for u in range(self.LOADS_P):        # first tile: k-tile 0, then the first loads of k-tile 1
            self.dma_p(0, u)
        for q in range(self.LOADS_Q):
            self.dma_q(0, q)
        e("s_waitcnt vmcnt(0)")
        e("s_barrier")
        self.advance(0)
        self.advance(1)
        for u in range(OPTS["pre"]):
            self.dma_p(1, u)
        for q in range(self.LOADS_Q):
            self.dma_q(1, q)
        e("s_branch 4f")
        e("2:")
        self.advance(0)
        self.advance(1)
        e("4:")
        for which in range(3):
            self.tail_reads(0, which)
        e("3:")
        self.loop_head_state()
        self.step(0)
        self.loop_head_state()
        self.step(1)
        e("s_add_u32 s76, s76, 2")
        e("s_cmp_lt_u32 s76, s56")
        e("s_cbranch_scc1 3b")
        e("s_waitcnt lgkmcnt(0)")
        for _ in range(3):
            e("s_nop 7")
        return self.L

    def clobbers(self):
        return ["v%d" % i for i in range(M_BF, M_ARD)] + ["s%d" % i for i in range(64, 78)] + ["m0", "scc", "memory"]


def main():
    out = sys.argv[1] if len(sys.argv) > 1 else os.path.join(os.path.dirname(os.path.abspath(__file__)), "gemm_w4_loop.inc")
    with open(out, "w") as f:
        f.write("/* generated by gen_w4_loop.py -- do not edit */\n")
        for v in (Mult(False), Mult(True), Loader(False), Loader(True), Wide(False, False), Wide(False, True), Wide(True, False), Wide(True, True)):
            lines = v.generate()
            f.write("#define %s_ASM \\\n" % v.name + " \\\n".join('\t"%s\\n\\t"' % x for x in lines) + "\n")
            f.write("#define %s_CLOBBERS %s\n" % (v.name, ", ".join('"%s"' % c for c in v.clobbers())))
        # multiplying waves: accumulator groups g[0..23] (group 6 (i / 4) + j holds row blocks 4 (i / 4) .. + 3 of column block
        # j), the lane block lb (fragment read addresses), k-tiles and flags
        ops = ['"+{a[%d:%d]}"(g[%d])' % (16 * n, 16 * n + 15, n) for n in range(16)]
        ops += ['"+{v[%d:%d]}"(g[%d])' % (16 * (n - 16), 16 * (n - 16) + 15, n) for n in range(16, 24)]
        f.write("#define W4_MULT_OUTPUTS(g) %s\n" % ", ".join(ops))
        f.write('#define W4_MULT_INPUTS(lb, nkt, flags) "{v[%d:%d]}"(lb), "{s40}"(nkt), "{s41}"(flags)\n' % (M_ARD, M_ARD + 15))
        f.write("#define W4_M_ARD 0\n#define W4_M_BRD %d\n" % (M_BRD - M_ARD))
        # loader: slot registers st[0..7] (a[0:255]) and st8 (v[0:15]), offsets of P (vp) and Q (vq, vq4), of the next tile's
        # Q (gathered; vn, vn4), LDS write address of every slot (wr[0..1], wr4), cursors sa, sb, the block sc
        ops = ['"+{a[%d:%d]}"(st[%d])' % (32 * n, 32 * n + 31, n) for n in range(8)] + ['"+{v[0:15]}"(st8)']
        f.write("#define W4_LOAD_OUTPUTS(st, st8) %s\n" % ", ".join(ops))
        f.write('#define W4_LOAD_OUTPUTS_Q(vq, vq4) "+{v[%d:%d]}"(vq), "+{v[%d:%d]}"(vq4)\n' % (L_VOFFQ, L_VOFFQ + 31, L_VOFFQ + 32, L_VOFFQ + 35))
        f.write('#define W4_LOAD_INPUTS(vp, wr, wr4, sa, sb, sc) "{v[%d:%d]}"(vp), "{v[%d:%d]}"(wr[0]), "{v[%d:%d]}"(wr[1]), "{v[%d:%d]}"(wr4), "{s[40:47]}"(sa), "{s[48:55]}"(sb), "{s[56:63]}"(sc)\n' %
                (L_VOFFP, L_VOFFP + 31, L_WR, L_WR + 31, L_WR + 32, L_WR + 63, L_WR + 64, L_WR + 67))
        f.write('#define W4_LOAD_INPUTS_NEXT(vn, vn4) "{v[%d:%d]}"(vn), "{v[%d:%d]}"(vn4)\n' % (L_VOFFQ_NEXT, L_VOFFQ_NEXT + 31, L_VOFFQ_NEXT + 32, L_VOFFQ_NEXT + 35))
        # wide symmetric kernel: accumulator groups as above, fragment read addresses lb, the lane's load offsets vo (8 of P,
        # 12 of Q, 12 of the next tile's Q), cursors sa, sb and the block sc (k-tiles, flags, bytes per k-tile of P and Q,
        # unused, LDS address of the wave's first chunk of P and of Q in stage 0, unused)
        f.write('#define W4D_OUTPUTS(g, vo) W4_MULT_OUTPUTS(g), "+{v[%d:%d]}"(vo)\n' % (D_VP, D_VP + 31))
        f.write('#define W4D_INPUTS(lb, sa, sb, sc) "{v[%d:%d]}"(lb), "{s[40:47]}"(sa), "{s[48:55]}"(sb), "{s[56:63]}"(sc)\n' % (M_ARD, M_ARD + 15))
        f.write("#define W4D_VP 0\n#define W4D_VQ %d\n#define W4D_VQ_NEXT %d\n#define W4D_PRE %d\n" % (D_VQ - D_VP, D_VQ_NEXT - D_VP, OPTS["pre"]))

if __name__ == "__main__":
    main()
