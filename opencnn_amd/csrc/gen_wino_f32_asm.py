#!/usr/bin/env python3
"""Generator of the hand-scheduled gfx950 assembly of the fused Winograd F(2x2,3x3) kernel.

Emits one kernel per KW (waves of a workgroup that share a column tile), wino_f32_asm_kw2 and
wino_f32_asm_kw4, each also as a _ragged variant for shapes outside the reference's tiling.
Same mathematics and data layout as wino_f32_stream in conv_kernel_f32.hpp (which replaces the
reference's Winograd_kernel, src/convolutionForward_32x64x8.cu:169-262); what the assembly adds
is control over the things hipcc does not let the C++ source decide:

  * all 256 arch VGPRs are assigned by hand (no spills, no copies through accumulator
    registers), so the epilogue and the tile switch cannot disturb the inner loop;
  * the first MFMA step of a tile starts from the constant 0 instead of zeroing 256
    accumulator registers;
  * the output transform stores through ONE per-row buffer descriptor and four per-lane
    offsets (no 64-bit pointer arithmetic on the vector ALU, which the matrix pipe shares);
  * exactly 64 store instructions per tile, so the s_waitcnt that follows can be counted
    instead of draining the stores;
  * a tile whose channel range is cut between two workgroups is merged by pre-loading the
    published partial result INTO the accumulators (A^T M A is linear: the four outputs of a
    2x2 tile are the images of the Winograd positions (0,0), -(0,3), -(3,0), (3,3)), which
    takes the merge out of the epilogue.

Model.  A unit = one 8-channel chunk of one workgroup tile (KW filter groups x 4/KW column
tiles); unit index = tile * chunks + chunk.  Workgroup L of the persistent grid owns a
contiguous range of units, at least one tile long, so a tile is shared by at most two
workgroups: the part that starts inside a tile is its workgroup's FIRST segment (finishes
early, publishes its partial outputs past the caches and raises a flag), the part that ends
inside a tile is the other workgroup's LAST segment (merges).  Three cursors walk the range: M
(the unit being multiplied), Q = M + 1 (filter loads), P = M + 2 (patch loads).

Registers.  a[16p:16p+15] accumulator of Winograd position p (MFMA D layout: register r, lane
(h, n) = filter row 8*(r/4) + 4h + r%4, batch element n).  U0 / U1: A operands of the two
filter quads of a chunk, one dwordx4 per pair of positions.  D0 (and D1 when a wave owns two steps):
patches in flight.  VA / VB: B operands of the current / next MFMA step, read from LDS
V[cw][buf][step][p][lane].  T / TO: transform temporaries.  VOFF: per-lane byte offsets of the
16 patch elements (out of range = zero padding).  Off / Eff: the four per-lane store offsets
and their per-tile version (out of range = do not store).

Hazards handled by hand (nothing inserts wait states into assembly): 32 wait states between
the last MFMA and v_accvgpr_read and between v_accvgpr_write and the next MFMA; s_nop 4
after v_readfirstlane before the SGPR is used; no vector instruction writes an SGPR while
scalar loads are outstanding (v_readfirstlane next to s_load returned corrupted values).

Kernel arguments (one 168-byte block, see AsmKernArgs in api.hip): four pointers (input CHWN,
transformed filter in MFMA order, output KHWN, split-merge flags), 24 ints, the timeline
buffer (or null): 64 int64 per workgroup, [0] = number of stamps, [2..] = the 100 MHz realtime
counter at kernel start, after the prologue and before / after every output transform, taken
by the workgroup's first wave; then the status word of the launch's flag set (host memory that
the GPU can write) and the number of polls after which a wait for a flag gives up.

A wait for a flag is bounded so that a bug or a workgroup that never becomes resident cannot
hang the GPU.  A wave that gives up writes 1 to the status word and goes on with whatever the
output tensor holds: the launch's result is wrong, every wave still ends, and the host finds
the word at its next call (api.hip: the call fails and the flags are cleared).  The last four
ints describe the places of the tiles of a line in the image (place()).

Usage: gen_wino_f32_asm.py > wino_f32_asm.s
"""
import sys

OOB = 0x80000000
FLAGS = 0x00020000
# A^T M A is linear: output (a,b) of a 2x2 tile is the image of Winograd position (0,0), -(0,3),
# -(3,0), (3,3).  position -> (output index, negate)
MERGE_POSITIONS = {0: (0, False), 3: (1, True), 12: (2, True), 15: (3, False)}


class Alloc:
    """Bump allocator of register indices."""

    def __init__(self, first, limit):
        self.next, self.limit = first, limit

    def get(self, name, n=1, align=1):
        self.next = (self.next + align - 1) // align * align
        base = self.next
        self.next += n
        assert self.next <= self.limit, f"out of registers at {name}"
        return base


def s(i, n=1):
    return f"s{i}" if n == 1 else f"s[{i}:{i + n - 1}]"


def v(i, n=1):
    return f"v{i}" if n == 1 else f"v[{i}:{i + n - 1}]"


def a(i, n=1):
    return f"a{i}" if n == 1 else f"a[{i}:{i + n - 1}]"


class Kernel:
    K_REAL = "Kreal"  # the scalar register with the real filter count (ragged K)
    CW_IS_FREE = False  # lane_setup and decode read Cw (the wave's column tile inside the workgroup tile)

    def __init__(self, KW, ragged=False, packed=False):
        """ragged: shapes outside N % 32 == 0, K % 32 == 0, C % 8 == 0.  Groups and chunks are
        rounded up by the host; lanes whose batch element does not exist read zeros and store
        nothing (out-of-range offsets), the last channel slab ends with the tensor, filter rows
        past K fall outside the row's num_records.  The inner loop is the same."""
        self.KW = KW
        self.ragged = ragged
        # batch elements, and filters, that do not exist are masked (the fp16 / bf16 kernels always do)
        self.ragged_n = self.ragged_k = ragged
        # packed (batches that are no multiple of 32, a _ragged kernel): a column tile is 32
        # consecutive columns of the line of all (spatial tile, batch element) pairs; see lane_tile
        self.packed = packed
        self.CW = 4 // KW
        self.SPW = 4 // KW
        self.lines = []
        self.outofline = []  # rarely executed blocks, emitted behind s_endpgm
        self.nlabel = 0
        self.name = f"wino_f32_asm_kw{KW}" + ("_packed" if packed else "_ragged" if ragged else "")
        self.alloc()

    # ------------------------------------------------------------------ helpers
    def e(self, text):
        self.lines.append("\t" + text)

    def label(self, name):
        self.lines.append(f"{name}:")

    def newlabel(self, hint):
        self.nlabel += 1
        return f".L{self.name}_{hint}_{self.nlabel}"

    def comment(self, text):
        self.lines.append(f"\t; {text}")

    # ------------------------------------------------------------------ registers
    def alloc(self):
        self.alloc_sgprs()
        self.alloc_vgprs()

    def alloc_sgprs(self):
        # s[0:1] kernel argument pointer, s2 workgroup id, s[4:5] the status word's address,
        # s6 the poll limit of a flag wait, s[8:15] the four pointers, s[16:39] the 24 ints,
        # s[40:41] the timeline pointer, s42.. everything else
        S = Alloc(42, 102)
        names = ["N", "H", "W", "Chunks", "TilesW", "Ngroups", "Colgroups", "Colblocks", "Q", "HWN4",
                 "UnitsQ", "UnitsRem", "UswBytes", "GridPerXcd", "Mch", "Sch", "Mcb", "Scb", "Mng",
                 "Sng", "Mtw", "Stw", "Creal", "Kreal", "Timeline", "TimelineHi"]
        self.S = {n: 16 + i for i, n in enumerate(names)}
        self.S.update(X=8, U=10, Y=12, Sync=14, Status=4, SpinLimit=6)
        for n in ["L", "Kw", "Cw", "Wave", "Begin", "Nunits", "G", "Tp", "Cp", "Tq", "Cq", "Tm", "Cm",
                  "SegEnd", "Kind", "KgM", "KgQ", "ColStep", "RowStep", "Slab", "UoffM", "UoffQ",
                  "Dkb", "Dlive", "Dng", "Dty", "Dtx", "RowOk", "Spin", "KwSpw"]:
            self.S[n] = S.get(n)
        self.S["RsrcX"] = S.get("RsrcX", 4, 4)
        self.S["RsrcU"] = S.get("RsrcU", 4, 4)
        self.S["RsrcY"] = S.get("RsrcY", 4, 4)
        self.S["Yt"] = S.get("Yt", 2, 2)
        self.S["Fl"] = S.get("Fl", 2, 2)
        self.S["T"] = S.get("T", 8, 2)  # temporaries T0..T7 (T6:T7 = division pair)
        # place(): the magic number of the line's tile count in two user registers that are free, the
        # ranges on the line in GridPerXcd (dead after head) and the tile count in a register of
        # its own, or in Cw where nothing reads that after head (CW_IS_FREE)
        self.S.update(PlaceM=3, PlaceS=7, PlaceG=self.S["GridPerXcd"])
        self.S["PlaceTn"] = self.S["Cw"] if self.CW_IS_FREE else S.get("PlaceTn")
        self.sgpr_count = S.next

    def alloc_vgprs(self):
        V = Alloc(1, 256)
        self.V = {}
        for n, cnt, al in [("Lane", 1, 1), ("LaneX", 1, 1), ("LaneU", 1, 1), ("LaneUb", 1, 1),
                           ("Lds", 1, 1), ("LdsWr", 1, 1), ("Zero", 1, 1), ("One", 1, 1), ("Oob", 1, 1),
                           ("Tmp", 4, 1),
                           ("Off", 4, 1), ("Eff", 4, 1), ("VOFF", 16, 1),
                           ("U0", 32, 2), ("U1", 32, 2), ("D0", 16, 1), ("D1", 16, 1),
                           ("VA", 16, 2), ("VB", 16, 2), ("T", 16, 2), ("TO", 16, 2), ("MPX", 16, 1)]:
            if n == "D1" and self.SPW == 1:
                continue
            self.V[n] = V.get(n, cnt, al)
        self.vgpr_count = V.next
        # the 64 registers that receive a published partial tile (dead at a chunk boundary)
        self.MP = ([self.V["T"] + i for i in range(16)] + [self.V["TO"] + i for i in range(16)] +
                   [self.V["VB"] + i for i in range(16)] + [self.V["MPX"] + i for i in range(16)])

    def sr(self, name, n=1):
        return s(self.S[name], n)

    def t(self, i):
        return s(self.S["T"] + i)

    def vr(self, name, i=0, n=1):
        return v(self.V[name] + i, n)

    # ------------------------------------------------------------------ scalar pieces
    def div(self, dst, x, m, sh):
        """dst = x / d for x < 2^31, with (m, sh) = (ceil(2^sh / d), 31 + ceil(log2 d))."""
        t6, t7 = self.S["T"] + 6, self.S["T"] + 7
        self.e(f"s_mul_hi_u32 {s(t7)}, {x}, {m}")
        self.e(f"s_mul_i32 {s(t6)}, {x}, {m}")
        self.e(f"s_lshr_b64 {s(t6, 2)}, {s(t6, 2)}, {sh}")
        self.e(f"s_mov_b32 {dst}, {s(t6)}")

    # ------------------------------------------------------------------ where a tile of the line lies
    # The workgroups of an XCD walk through a window of neighbouring tiles of the line.  About
    # G / Tn of them (G ranges on a line of Tn tiles) are in work from the start - the tiles in
    # which a range begins - and the others are taken up one tile time later.  The patch lines a
    # tile shares with its neighbours in the image are only found in L2 while those neighbours
    # are in work too: an XCD's 4 MB do not keep a tile's patches (next to the transformed
    # filter) until a later tile asks for them.  So the tiles that are in work from the start get
    # the first places of their window and the later ones the rest: two compact blocks of the
    # image instead of an interleaved pattern.  place(t), with E(t) = t * G / Tn (the ranges that
    # begin in front of tile t, for equal ranges) and the window of XCD x = tiles
    # [ceil(x * Tn / 8), ceil((x + 1) * Tn / 8)):
    #   begins a range (E(t + 1) > E(t)):  lo + E(t) - E(lo)
    #   else:                              t + (E(next lo) - E(lo)) - (E(t) - E(lo))
    # a permutation of every window whatever the real range boundaries are (they only decide how
    # well it works).  Bit 6 of the magic shift switches it on (64-bit shifts ignore the bit).
    def place(self, T):
        """t5 = the place of tile T of the line (T itself when the host has not asked for places)."""
        t, e = self.t, self.e
        pm, ps, g, tn = self.sr("PlaceM"), self.sr("PlaceS"), self.sr("PlaceG"), self.sr("PlaceTn")
        e(f"s_lshl_b32 {t(0)}, {T}, 3")
        self.div(t(1), t(0), pm, ps)                      # x: the window
        e(f"s_mul_i32 {t(2)}, {t(1)}, {tn}")
        e(f"s_add_u32 {t(3)}, {t(2)}, {tn}")
        e(f"s_add_u32 {t(2)}, {t(2)}, 7")
        e(f"s_lshr_b32 {t(2)}, {t(2)}, 3")                # lo
        e(f"s_add_u32 {t(3)}, {t(3)}, 7")
        e(f"s_lshr_b32 {t(3)}, {t(3)}, 3")                # lo of the next window
        e(f"s_mul_i32 {t(0)}, {t(2)}, {g}")
        self.div(t(4), t(0), pm, ps)                      # E(lo)
        e(f"s_mul_i32 {t(0)}, {t(3)}, {g}")
        self.div(t(3), t(0), pm, ps)                      # E(next lo)
        e(f"s_sub_u32 {t(3)}, {t(3)}, {t(4)}")            # ranges that begin in the window
        e(f"s_mul_i32 {t(0)}, {T}, {g}")
        self.div(t(1), t(0), pm, ps)                      # E(t)
        e(f"s_add_u32 {t(0)}, {t(0)}, {g}")
        self.div(t(5), t(0), pm, ps)                      # E(t + 1)
        e(f"s_sub_u32 {t(4)}, {t(1)}, {t(4)}")            # E(t) - E(lo)
        e(f"s_add_u32 {t(2)}, {t(2)}, {t(4)}")            # the place of a tile in which a range begins
        e(f"s_add_u32 {t(3)}, {T}, {t(3)}")
        e(f"s_sub_u32 {t(3)}, {t(3)}, {t(4)}")            # the place of a later tile
        e(f"s_cmp_gt_u32 {t(5)}, {t(1)}")
        e(f"s_cselect_b32 {t(5)}, {t(2)}, {t(3)}")
        e(f"s_bitcmp1_b32 {ps}, 6")
        e(f"s_cselect_b32 {t(5)}, {t(5)}, {T}")

    def split_tile(self, T):
        """Workgroup tile T of the line -> Dkb (filter block) and T0 (column block) of its place:
        filter-block major."""
        t = self.t
        self.place(T)
        self.div(self.sr("Dkb"), t(5), self.sr("Mcb"), self.sr("Scb"))
        self.e(f"s_mul_i32 {t(0)}, {self.sr('Dkb')}, {self.sr('Colblocks')}")
        self.e(f"s_sub_u32 {t(0)}, {t(5)}, {t(0)}")  # column block

    def filter_block(self, dst, T):
        """dst = filter block of workgroup tile T (may use T0 .. T5)."""
        self.place(T)
        self.div(dst, self.t(5), self.sr("Mcb"), self.sr("Scb"))

    def decode(self, T):
        """Workgroup tile T -> Dkb (filter block), Dlive, Dng, Dty, Dtx of this wave's column tile."""
        t = self.t
        self.split_tile(T)
        if self.CW == 2:
            self.e(f"s_lshl_b32 {t(0)}, {t(0)}, 1")
            self.e(f"s_add_u32 {t(0)}, {t(0)}, {self.sr('Cw')}")
        self.e(f"s_sub_u32 {t(1)}, {self.sr('Colgroups')}, 1")
        self.e(f"s_cmp_lt_u32 {t(0)}, {self.sr('Colgroups')}")
        self.e(f"s_cselect_b32 {self.sr('Dlive')}, 1, 0")
        self.e(f"s_cselect_b32 {t(0)}, {t(0)}, {t(1)}")  # a missing column tile works on the last real one
        if self.packed:  # the column tile is a group of spatial tiles; the lanes find their own
            self.e(f"s_mov_b32 {self.sr('Dty')}, {t(0)}")
            self.e(f"s_mov_b32 {self.sr('Dng')}, 0")
            self.e(f"s_mov_b32 {self.sr('Dtx')}, 0")
            return
        # Column tile -> (spatial tile, image group).  The argument slot Ngroups holds the divisor:
        # the image groups when they are the fast index of the line of column tiles, or, with bit 6
        # of the magic shift set (64-bit shifts ignore it), the spatial tiles when those are.
        self.div(t(2), t(0), self.sr("Mng"), self.sr("Sng"))
        self.e(f"s_mul_i32 {t(3)}, {t(2)}, {self.sr('Ngroups')}")
        self.e(f"s_sub_u32 {t(3)}, {t(0)}, {t(3)}")
        self.e(f"s_bitcmp1_b32 {self.sr('Sng')}, 6")
        self.e(f"s_cselect_b32 {self.sr('Dng')}, {t(2)}, {t(3)}")
        self.e(f"s_cselect_b32 {t(2)}, {t(3)}, {t(2)}")  # spatial tile
        self.div(self.sr("Dty"), t(2), self.sr("Mtw"), self.sr("Stw"))
        self.e(f"s_mul_i32 {t(3)}, {self.sr('Dty')}, {self.sr('TilesW')}")
        self.e(f"s_sub_u32 {self.sr('Dtx')}, {t(2)}, {t(3)}")
        # With bit 6 of the magic shift Stw set, the spatial tiles are numbered in strips of two
        # tile rows, zigzag: neighbours on the line are neighbours in the image in both directions
        # (tile i+1 below or beside tile i, tile i+2 beside it).  (row r0, column c0) of the
        # row-major reading -> strip r0 / 2, position (r0 % 2) * TilesW + c0 inside it; a last
        # strip of one row keeps its row-major order.
        # (No branch: in the fp32 kernels this code is dealt out over the gaps between MFMAs.)
        self.e(f"s_add_u32 {t(3)}, {self.sr('H')}, 1")
        self.e(f"s_lshr_b32 {t(3)}, {t(3)}, 1")                    # tile rows
        self.e(f"s_or_b32 {t(4)}, {self.sr('Dty')}, 1")
        self.e(f"s_cmp_lt_u32 {t(4)}, {t(3)}")                      # the strip has two rows
        self.e(f"s_cselect_b32 {t(5)}, 1, 0")
        self.e(f"s_bitcmp1_b32 {self.sr('Stw')}, 6")
        self.e(f"s_cselect_b32 {t(5)}, {t(5)}, 0")
        self.e(f"s_and_b32 {t(3)}, {self.sr('Dty')}, 1")
        self.e(f"s_mul_i32 {t(3)}, {t(3)}, {self.sr('TilesW')}")
        self.e(f"s_add_u32 {t(3)}, {t(3)}, {self.sr('Dtx')}")       # position inside the strip
        self.e(f"s_and_b32 {t(4)}, {self.sr('Dty')}, -2")
        self.e(f"s_and_b32 {t(1)}, {t(3)}, 1")
        self.e(f"s_or_b32 {t(4)}, {t(4)}, {t(1)}")
        self.e(f"s_lshr_b32 {t(3)}, {t(3)}, 1")
        self.e(f"s_cmp_lg_u32 {t(5)}, 0")
        self.e(f"s_cselect_b32 {self.sr('Dty')}, {t(4)}, {self.sr('Dty')}")
        self.e(f"s_cselect_b32 {self.sr('Dtx')}, {t(3)}, {self.sr('Dtx')}")

    def patch_offsets(self):
        """Per-lane byte offsets of the 16 patch elements of the tile in D* (P cursor), relative to
        a two-channel slab; elements in the zero padding get an offset no num_records reaches."""
        t = self.t
        if self.packed:
            return self.patch_offsets_packed()
        self.e(f"s_lshl_b32 {t(0)}, {self.sr('Dty')}, 1")
        self.e(f"s_sub_i32 {t(0)}, {t(0)}, 1")  # first patch row
        self.e(f"s_lshl_b32 {t(1)}, {self.sr('Dtx')}, 1")
        self.e(f"s_sub_i32 {t(1)}, {t(1)}, 1")  # first patch column
        self.e(f"s_mul_i32 {t(2)}, {t(0)}, {self.sr('RowStep')}")
        self.e(f"s_mul_i32 {t(3)}, {t(1)}, {self.sr('ColStep')}")
        self.e(f"s_add_i32 {t(2)}, {t(2)}, {t(3)}")
        self.e(f"s_lshl_b32 {t(3)}, {self.sr('Dng')}, 7")
        self.e(f"s_add_i32 {t(2)}, {t(2)}, {t(3)}")  # byte offset of element (0,0), may be negative
        if self.ragged_n:
            self.alive_lanes()
        for i in range(4):
            self.e(f"s_add_i32 {t(4)}, {t(0)}, {i}")
            self.e(f"s_cmp_lt_u32 {t(4)}, {self.sr('H')}")  # unsigned: also rejects -1
            self.e(f"s_cselect_b32 {self.sr('RowOk')}, 1, 0")
            self.e(f"s_mov_b32 {t(3)}, {t(2)}")
            for j in range(4):
                self.e(f"s_add_i32 {t(4)}, {t(1)}, {j}")
                self.e(f"s_cmp_lt_u32 {t(4)}, {self.sr('W')}")
                self.e(f"s_cselect_b32 {t(4)}, {self.sr('RowOk')}, 0")
                self.e(f"s_cmp_lg_u32 {t(4)}, 0")
                self.e(f"s_cselect_b32 {t(5)}, {t(3)}, 0x{OOB:x}")
                self.e(f"v_add_u32 {self.vr('VOFF', i * 4 + j)}, {t(5)}, {self.vr('LaneX')}")
                if self.ragged_n:
                    self.e(f"v_cndmask_b32 {self.vr('VOFF', i * 4 + j)}, {self.vr('Oob')}, {self.vr('VOFF', i * 4 + j)}, vcc")
                if j < 3:
                    self.e(f"s_add_i32 {t(3)}, {t(3)}, {self.sr('ColStep')}")
            if i < 3:
                self.e(f"s_add_i32 {t(2)}, {t(2)}, {self.sr('RowStep')}")

    # ------------------------------------------------------------------ packed column tiles (N % 32 != 0)
    # The columns of all spatial tiles (numbered row-major) and their N batch elements form one
    # line, column (tile, n) at tile * N + n; column tile g holds columns 32 g .. 32 g + 31 of it,
    # so only the last column tile of a layer has empty columns.  The magic number of the slot
    # Mng / Sng divides by N.  Everything per lane happens here, at a tile switch: the units only
    # see 16 patch offsets and 4 store offsets per lane, as before.  Scratch: the transform
    # temporaries T, dead between two units.
    def lane_tile(self):
        """T[0] = batch element * 4, T[1] = 2*ty, T[2] = 2*tx of this lane's column in column tile
        Dty; T[3] = 0, or the out-of-range bit for a lane past the last column."""
        t = self.t
        T = lambda i: self.vr("T", i)
        self.e(f"v_and_b32 {T(0)}, 31, {self.vr('Lane')}")
        self.e(f"s_lshl_b32 {t(4)}, {self.sr('Dty')}, 5")
        self.e(f"v_add_u32 {T(1)}, {t(4)}, {T(0)}")                         # column on the line
        # tile = column / N with the magic number, in 64 bits as the scalar div does
        self.e(f"v_mul_lo_u32 {T(4)}, {T(1)}, {self.sr('Mng')}")
        self.e(f"v_mul_hi_u32 {T(5)}, {T(1)}, {self.sr('Mng')}")
        self.e(f"v_lshrrev_b64 {self.vr('T', 4, 2)}, {self.sr('Sng')}, {self.vr('T', 4, 2)}")
        self.e(f"v_mul_lo_u32 {T(5)}, {T(4)}, {self.sr('N')}")
        self.e(f"v_sub_u32 {T(0)}, {T(1)}, {T(5)}")                         # batch element
        self.e(f"v_mov_b32 {T(1)}, {T(4)}")                                 # spatial tile
        self.e(f"s_add_u32 {t(4)}, {self.sr('H')}, 1")
        self.e(f"s_lshr_b32 {t(4)}, {t(4)}, 1")
        self.e(f"s_mul_i32 {t(4)}, {t(4)}, {self.sr('TilesW')}")
        self.e(f"v_cmp_gt_u32 vcc, {t(4)}, {T(1)}")                         # the tile exists
        self.e(f"v_cndmask_b32 {T(3)}, {self.vr('Oob')}, {self.vr('Zero')}, vcc")
        # ty = tile / TilesW
        self.e(f"v_mul_lo_u32 {T(4)}, {T(1)}, {self.sr('Mtw')}")
        self.e(f"v_mul_hi_u32 {T(5)}, {T(1)}, {self.sr('Mtw')}")
        self.e(f"v_lshrrev_b64 {self.vr('T', 4, 2)}, {self.sr('Stw')}, {self.vr('T', 4, 2)}")
        self.e(f"v_mul_lo_u32 {T(5)}, {T(4)}, {self.sr('TilesW')}")
        self.e(f"v_sub_u32 {T(2)}, {T(1)}, {T(5)}")
        self.e(f"v_lshlrev_b32 {T(1)}, 1, {T(4)}")
        self.e(f"v_lshlrev_b32 {T(2)}, 1, {T(2)}")
        self.e(f"v_lshlrev_b32 {T(0)}, 2, {T(0)}")                          # as a byte offset

    def in_range(self, dst, x, limit, extra):
        """dst = extra, or the out-of-range bit unless 0 <= x < limit (x a VGPR, limit an SGPR)."""
        self.e(f"v_cmp_gt_u32 vcc, {limit}, {x}")  # unsigned: also rejects -1
        self.e(f"v_cndmask_b32 {dst}, {self.vr('Oob')}, {extra}, vcc")

    def patch_offsets_packed(self):
        T = lambda i: self.vr("T", i)
        self.lane_tile()
        # T[4..7]: the four patch rows' bad bits (with the lane's), T[8..11]: the columns'
        for i in range(4):
            self.e(f"v_add_u32 {T(12)}, {i - 1}, {T(1)}")
            self.in_range(T(4 + i), T(12), self.sr("H"), T(3))
        for j in range(4):
            self.e(f"v_add_u32 {T(12)}, {j - 1}, {T(2)}")
            self.in_range(T(8 + j), T(12), self.sr("W"), self.vr("Zero"))
        # element (0, 0): ((2ty - 1) * W + 2tx - 1) * N * 4 + n * 4 + the lane's channel
        self.e(f"v_and_b32 {T(12)}, 31, {self.vr('Lane')}")
        self.e(f"v_lshlrev_b32 {T(12)}, 2, {T(12)}")
        self.e(f"v_sub_u32 {T(12)}, {self.vr('LaneX')}, {T(12)}")           # the channel part of LaneX
        self.e(f"v_add_u32 {T(12)}, {T(12)}, {T(0)}")
        self.e(f"v_add_u32 {T(13)}, -1, {T(1)}")
        self.e(f"v_mul_lo_u32 {T(13)}, {T(13)}, {self.sr('RowStep')}")
        self.e(f"v_add_u32 {T(12)}, {T(12)}, {T(13)}")
        self.e(f"v_add_u32 {T(13)}, -1, {T(2)}")
        self.e(f"v_mul_lo_u32 {T(13)}, {T(13)}, {self.sr('ColStep')}")
        self.e(f"v_add_u32 {T(12)}, {T(12)}, {T(13)}")
        for i in range(4):
            self.e(f"v_mov_b32 {T(13)}, {T(12)}")
            for j in range(4):
                self.e(f"v_or3_b32 {self.vr('VOFF', i * 4 + j)}, {T(13)}, {T(4 + i)}, {T(8 + j)}")
                if j < 3:
                    self.e(f"v_add_u32 {T(13)}, {self.sr('ColStep')}, {T(13)}")
            if i < 3:
                self.e(f"v_add_u32 {T(12)}, {self.sr('RowStep')}, {T(12)}")

    def store_offsets_packed(self):
        """Eff[0..3] of the M tile: the lane's four outputs relative to its filter row."""
        t = self.t
        T = lambda i: self.vr("T", i)
        self.lane_tile()
        self.e(f"s_cmp_lg_u32 {self.sr('Dlive')}, 0")
        self.e(f"s_cselect_b32 {t(3)}, 0, 0x{OOB:x}")
        self.e(f"v_or_b32 {T(3)}, {t(3)}, {T(3)}")
        for d in range(2):
            self.e(f"v_add_u32 {T(12)}, {d}, {T(1)}")
            self.in_range(T(4 + d), T(12), self.sr("H"), T(3))
            self.e(f"v_add_u32 {T(12)}, {d}, {T(2)}")
            self.in_range(T(8 + d), T(12), self.sr("W"), self.vr("Zero"))
        # output (0, 0): (2ty * W + 2tx) * N * 4 + n * 4 + the lane's filter-row part of Off[0]
        self.e(f"v_and_b32 {T(12)}, 31, {self.vr('Lane')}")
        self.e(f"v_lshlrev_b32 {T(12)}, 2, {T(12)}")
        self.e(f"v_sub_u32 {T(12)}, {self.vr('Off', 0)}, {T(12)}")
        self.e(f"v_add_u32 {T(12)}, {T(12)}, {T(0)}")
        self.e(f"v_mul_lo_u32 {T(13)}, {T(1)}, {self.sr('RowStep')}")
        self.e(f"v_add_u32 {T(12)}, {T(12)}, {T(13)}")
        self.e(f"v_mul_lo_u32 {T(13)}, {T(2)}, {self.sr('ColStep')}")
        self.e(f"v_add_u32 {T(12)}, {T(12)}, {T(13)}")
        self.e(f"v_add_u32 {T(13)}, {self.sr('RowStep')}, {T(12)}")
        self.e(f"v_or3_b32 {self.vr('Eff', 0)}, {T(12)}, {T(4)}, {T(8)}")
        self.e(f"v_or3_b32 {self.vr('Eff', 2)}, {T(13)}, {T(5)}, {T(8)}")
        self.e(f"v_add_u32 {T(12)}, {self.sr('ColStep')}, {T(12)}")
        self.e(f"v_add_u32 {T(13)}, {self.sr('ColStep')}, {T(13)}")
        self.e(f"v_or3_b32 {self.vr('Eff', 1)}, {T(12)}, {T(4)}, {T(9)}")
        self.e(f"v_or3_b32 {self.vr('Eff', 3)}, {T(13)}, {T(5)}, {T(9)}")

    def alive_lanes(self):
        """vcc = lanes whose batch element Dng*32 + lane%32 exists (ragged N)."""
        t = self.t
        self.e(f"s_lshl_b32 {t(4)}, {self.sr('Dng')}, 5")
        self.e(f"v_and_b32 {self.vr('Tmp')}, 31, {self.vr('Lane')}")
        self.e(f"v_add_u32 {self.vr('Tmp')}, {t(4)}, {self.vr('Tmp')}")
        self.e(f"v_cmp_gt_u32 vcc, {self.sr('N')}, {self.vr('Tmp')}")

    def slab_descriptor(self, j):
        """RsrcX = the two-channel slab of MFMA step Cp*4 + kw*SPW + j."""
        t = self.t
        self.e(f"s_lshl_b32 {t(0)}, {self.sr('Cp')}, 2")
        self.e(f"s_add_u32 {t(0)}, {t(0)}, {self.sr('KwSpw')}")
        if j:
            self.e(f"s_add_u32 {t(0)}, {t(0)}, {j}")
        rx = self.S["RsrcX"]
        if self.ragged:  # channels of this slab that exist: 2, 1 (odd C) or 0 (padding of the last chunk)
            self.e(f"s_lshl_b32 {t(2)}, {t(0)}, 1")
            self.e(f"s_sub_i32 {t(2)}, {self.sr('Creal')}, {t(2)}")
            self.e(f"s_max_i32 {t(2)}, {t(2)}, 0")
            self.e(f"s_min_i32 {t(2)}, {t(2)}, 2")
            self.e(f"s_mul_i32 {s(rx + 2)}, {t(2)}, {self.sr('HWN4')}")
        self.e(f"s_mul_hi_u32 {t(1)}, {t(0)}, {self.sr('Slab')}")
        self.e(f"s_mul_i32 {t(0)}, {t(0)}, {self.sr('Slab')}")
        self.e(f"s_add_u32 {s(rx)}, {s(self.S['X'])}, {t(0)}")
        self.e(f"s_addc_u32 {s(rx + 1)}, {s(self.S['X'] + 1)}, {t(1)}")

    def u_offset(self, dst, kg, c, second):
        """dst = byte offset of filter quad 2*c (+1) of filter group kg in the MFMA-order Ww."""
        t = self.t
        self.e(f"s_mul_i32 {t(0)}, {kg}, {self.sr('Q')}")
        self.e(f"s_lshl_b32 {t(1)}, {c}, 1")
        self.e(f"s_add_u32 {t(0)}, {t(0)}, {t(1)}")
        if second:
            self.e(f"s_add_u32 {t(0)}, {t(0)}, 1")
        self.e(f"s_lshl_b32 {dst}, {t(0)}, 13")

    def m_tile_setup(self):
        """After decode(Tm): KgM, the four store offsets of this tile, the address of its first row."""
        t = self.t
        self.e(f"s_lshl_b32 {t(0)}, {self.sr('Dkb')}, {self.KW.bit_length() - 1}")
        self.e(f"s_add_u32 {self.sr('KgM')}, {t(0)}, {self.sr('Kw')}")
        yt = self.S["Yt"]
        if self.packed:
            self.store_offsets_packed()
            self.e(f"s_lshl_b32 {t(0)}, {self.sr('KgM')}, 5")
            self.e(f"s_mul_hi_u32 {t(1)}, {t(0)}, {self.sr('HWN4')}")
            self.e(f"s_mul_i32 {t(0)}, {t(0)}, {self.sr('HWN4')}")
            self.e(f"s_add_u32 {s(yt)}, {s(self.S['Y'])}, {t(0)}")
            self.e(f"s_addc_u32 {s(yt + 1)}, {s(self.S['Y'] + 1)}, {t(1)}")
            return
        # validity of the four outputs (odd H / W: the last tile row / column keeps one)
        self.e(f"s_lshl_b32 {t(0)}, {self.sr('Dty')}, 1")
        self.e(f"s_add_u32 {t(0)}, {t(0)}, 1")
        self.e(f"s_cmp_lt_u32 {t(0)}, {self.sr('H')}")
        self.e(f"s_cselect_b32 {t(0)}, {self.sr('Dlive')}, 0")  # row 1 stored
        self.e(f"s_lshl_b32 {t(1)}, {self.sr('Dtx')}, 1")
        self.e(f"s_add_u32 {t(1)}, {t(1)}, 1")
        self.e(f"s_cmp_lt_u32 {t(1)}, {self.sr('W')}")
        self.e(f"s_cselect_b32 {t(1)}, {self.sr('Dlive')}, 0")  # column 1 stored
        self.e(f"s_and_b32 {t(2)}, {t(0)}, {t(1)}")
        if self.ragged_n:
            self.alive_lanes()
        for q, ok in enumerate([self.sr("Dlive"), t(1), t(0), t(2)]):
            self.e(f"s_cmp_lg_u32 {ok}, 0")
            self.e(f"s_cselect_b32 {t(3)}, 0, 0x{OOB:x}")
            self.e(f"v_or_b32 {self.vr('Eff', q)}, {t(3)}, {self.vr('Off', q)}")
            if self.ragged_n:
                self.e(f"v_cndmask_b32 {self.vr('Eff', q)}, {self.vr('Oob')}, {self.vr('Eff', q)}, vcc")
        # first row of the tile: y + kg*32*HWN4 + ((2ty*W + 2tx)*N + ng*32)*4
        self.e(f"s_lshl_b32 {t(0)}, {self.sr('KgM')}, 5")
        self.e(f"s_mul_hi_u32 {t(1)}, {t(0)}, {self.sr('HWN4')}")
        self.e(f"s_mul_i32 {t(0)}, {t(0)}, {self.sr('HWN4')}")
        self.e(f"s_add_u32 {s(yt)}, {s(self.S['Y'])}, {t(0)}")
        self.e(f"s_addc_u32 {s(yt + 1)}, {s(self.S['Y'] + 1)}, {t(1)}")
        self.e(f"s_mul_i32 {t(0)}, {self.sr('Dty')}, {self.sr('RowStep')}")
        self.e(f"s_mul_i32 {t(1)}, {self.sr('Dtx')}, {self.sr('ColStep')}")
        self.e(f"s_add_u32 {t(0)}, {t(0)}, {t(1)}")
        self.e(f"s_lshl_b32 {t(0)}, {t(0)}, 1")
        self.e(f"s_lshl_b32 {t(1)}, {self.sr('Dng')}, 7")
        self.e(f"s_add_u32 {t(0)}, {t(0)}, {t(1)}")
        self.e(f"s_add_u32 {s(yt)}, {s(yt)}, {t(0)}")
        self.e(f"s_addc_u32 {s(yt + 1)}, {s(yt + 1)}, 0")

    # ------------------------------------------------------------------ vector pieces
    def load_u(self, dst, p, soff):
        """A operands of positions p and p + 1 (two MFMA steps each): one 16-byte load, issued in
        the slot of the even position."""
        if p % 2:
            return
        lane = self.vr("LaneU") if p < 8 else self.vr("LaneUb")
        self.e(f"buffer_load_dwordx4 {self.vr(dst, 2 * p, 4)}, {lane}, {self.sr('RsrcU', 4)}, {soff} offen offset:{(p % 8) * 512}")

    def load_patch(self, dst, p):
        self.e(f"buffer_load_dword {self.vr(dst, p)}, {self.vr('VOFF', p)}, {self.sr('RsrcX', 4)}, 0 offen")

    def read_v(self, dst, step, p):
        """Two B operands (positions p, p+1) of MFMA step `step` from the read buffer."""
        self.e(f"ds_read2st64_b32 {self.vr(dst, p, 2)}, {self.vr('Lds')} offset0:{step * 16 + p} offset1:{step * 16 + p + 1}")

    def transform(self, src):
        """V = B^T d B of one patch (columns first, then rows, the order of
        src/convolutionForward_32x64x8.cu:59-80), left in TO[0..15] for write_v."""
        d = lambda i: self.vr(src, i)
        t = lambda i: self.vr("T", i)
        o = lambda i: self.vr("TO", i)
        for c in range(4):
            self.e(f"v_sub_f32 {t(c)}, {d(c)}, {d(8 + c)}")
            self.e(f"v_add_f32 {t(4 + c)}, {d(4 + c)}, {d(8 + c)}")
            self.e(f"v_sub_f32 {t(8 + c)}, {d(8 + c)}, {d(4 + c)}")
            self.e(f"v_sub_f32 {t(12 + c)}, {d(4 + c)}, {d(12 + c)}")
        for r in range(4):
            self.e(f"v_sub_f32 {o(4 * r)}, {t(4 * r)}, {t(4 * r + 2)}")
            self.e(f"v_add_f32 {o(4 * r + 1)}, {t(4 * r + 1)}, {t(4 * r + 2)}")
            self.e(f"v_sub_f32 {o(4 * r + 2)}, {t(4 * r + 2)}, {t(4 * r + 1)}")
            self.e(f"v_sub_f32 {o(4 * r + 3)}, {t(4 * r + 1)}, {t(4 * r + 3)}")

    def write_v(self, j, p):
        """Two transformed values (positions p, p+1) of owned step j to the write buffer."""
        o = lambda i: self.vr("TO", i)
        self.e(f"ds_write2st64_b32 {self.vr('LdsWr')}, {o(p)}, {o(p + 1)} offset0:{j * 16 + p} offset1:{j * 16 + p + 1}")

    def mfma_slot(self, step, first, p, vmem, write_step):
        """MFMA p of a step and what rides behind it: vmem(p) (global loads or nothing), for
        p < 8 the LDS read of two B operands of the next step and, with write_step, the LDS write
        of two transformed values waiting in TO (owned step `write_step`)."""
        usrc = "U0" if step < 2 else "U1"
        vsrc = "VA" if step % 2 == 0 else "VB"
        vnext = "VB" if step % 2 == 0 else "VA"
        fresh = first and step == 0 and not (first == "merge" and p in MERGE_POSITIONS)
        c = "0" if fresh else a(16 * p, 16)
        self.e(f"v_mfma_f32_32x32x2_f32 {a(16 * p, 16)}, {self.vr(usrc, 2 * p + (step & 1))}, {self.vr(vsrc, p)}, {c}")
        if vmem:
            vmem(p)
        if step < 3 and p < 8:
            self.read_v(vnext, step + 1, 2 * p)
        if write_step is not None and p < 8:
            self.write_v(write_step, 2 * p)

    def mfma_step(self, step, first, vmem, write_step=None):
        """The 16 MFMAs of one step."""
        for p in range(16):
            self.mfma_slot(step, first, p, vmem, write_step)

    def mfma_step_with_cursors(self, first, vmem, write_step):
        """Step 0, during which the cursors P and Q advance: scalar instructions issue while the
        matrix pipe is busy, in front of the chunk it would wait for them.  The common case (P
        stays in its tile) is a handful of instructions behind the first MFMA, without a taken
        branch.  The tile switch of P (three divisions, 16 patch offsets: some 150 instructions)
        is a second copy of the rest of the step, out of line behind the kernel's end, with the
        switch spread over the gaps between its MFMAs."""
        t = self.t
        rare, done = self.newlabel("p_switch"), self.newlabel("step0_done")
        self.mfma_slot(0, first, 0, vmem, write_step)
        self.e(f"s_add_u32 {t(0)}, {self.sr('G')}, 2")
        self.e(f"s_cmp_lt_u32 {t(0)}, {self.sr('Nunits')}")
        self.e(f"s_addc_u32 {self.sr('Cp')}, {self.sr('Cp')}, 0")  # P -> unit G+2 when there is one
        self.e(f"s_cmp_eq_u32 {self.sr('Cp')}, {self.sr('Chunks')}")
        self.e(f"s_cbranch_scc1 {rare}")
        self.advance_q()
        for p in range(1, 16):
            self.mfma_slot(0, first, p, vmem, write_step)
        self.label(done)
        # the rare path
        main, self.lines = self.lines, []
        self.e(f"s_mov_b32 {self.sr('Cp')}, 0")
        self.e(f"s_add_u32 {self.sr('Tp')}, {self.sr('Tp')}, 1")
        self.decode(self.sr("Tp"))
        self.patch_offsets()
        switch, self.lines = self.lines, []
        self.label(rare)
        self.advance_q()  # first: it shares the scalar temporaries with the switch
        per_gap = -(-len(switch) // 15)
        for p in range(1, 16):
            self.lines.extend(switch[(p - 1) * per_gap:p * per_gap])
            self.mfma_slot(0, first, p, vmem, write_step)
        self.e(f"s_branch {done}")
        self.outofline.extend(self.lines)
        self.lines = main

    def end_of_chunk(self):
        """All LDS traffic of this wave done, workgroup barrier, swap the buffers, fetch the first
        B operands of the next chunk."""
        self.e("s_waitcnt lgkmcnt(0)")
        self.e("s_barrier")
        self.e(f"v_xor_b32 {self.vr('Lds')}, 0x4000, {self.vr('Lds')}")
        self.e(f"v_xor_b32 {self.vr('LdsWr')}, 0x4000, {self.vr('LdsWr')}")
        for p in range(0, 16, 2):
            self.read_v("VA", 0, p)

    # ------------------------------------------------------------------ cursors
    def advance_p(self, ahead=2):
        """P cursor -> unit G+ahead when there is one.  The common case (same tile) falls through
        without a taken branch; the tile switch lives out of line, behind the kernel's end."""
        rare, back = self.newlabel("p_switch"), self.newlabel("p_back")
        t = self.t
        self.e(f"s_add_u32 {t(0)}, {self.sr('G')}, {ahead}")
        self.e(f"s_cmp_lt_u32 {t(0)}, {self.sr('Nunits')}")
        self.e(f"s_addc_u32 {self.sr('Cp')}, {self.sr('Cp')}, 0")  # + SCC
        self.e(f"s_cmp_eq_u32 {self.sr('Cp')}, {self.sr('Chunks')}")
        self.e(f"s_cbranch_scc1 {rare}")
        self.label(back)
        main, self.lines = self.lines, []
        self.label(rare)
        self.e(f"s_mov_b32 {self.sr('Cp')}, 0")
        self.e(f"s_add_u32 {self.sr('Tp')}, {self.sr('Tp')}, 1")
        self.decode(self.sr("Tp"))
        self.patch_offsets()
        self.e(f"s_branch {back}")
        self.outofline.extend(self.lines)
        self.lines = main

    def advance_q(self):
        rare, back = self.newlabel("q_switch"), self.newlabel("q_back")
        t = self.t
        self.e(f"s_add_u32 {t(0)}, {self.sr('G')}, 1")
        self.e(f"s_cmp_lt_u32 {t(0)}, {self.sr('Nunits')}")
        self.e(f"s_addc_u32 {self.sr('Cq')}, {self.sr('Cq')}, 0")
        self.e(f"s_cmp_eq_u32 {self.sr('Cq')}, {self.sr('Chunks')}")
        self.e(f"s_cbranch_scc1 {rare}")
        self.label(back)
        main, self.lines = self.lines, []
        self.label(rare)
        self.e(f"s_mov_b32 {self.sr('Cq')}, 0")
        self.e(f"s_add_u32 {self.sr('Tq')}, {self.sr('Tq')}, 1")
        self.filter_block(t(0), self.sr("Tq"))
        self.e(f"s_lshl_b32 {t(0)}, {t(0)}, {self.KW.bit_length() - 1}")
        self.e(f"s_add_u32 {self.sr('KgQ')}, {t(0)}, {self.sr('Kw')}")
        self.e(f"s_branch {back}")
        self.outofline.extend(self.lines)
        self.lines = main

    # ------------------------------------------------------------------ one chunk
    def chunk(self, first):
        """MFMA work of unit G (8 channels) with the loads of the units after it in its shadow.

        Global loads in issue order: step 0 second filter quad of this unit (U1), step 1 patches
        of unit G+2 (D0), step 2 first filter quad of unit G+1 (U0), step 3 (KW = 2) second
        patch of unit G+2 (D1).  vmcnt counts in issue order, stores included; `first` = this
        chunk follows the 64 stores of an epilogue (or a drained queue), so everything it waits
        for is older than those stores and the counts grow by 64 (capped at the field's 63)."""
        two = self.SPW == 2
        wait = lambda n: self.e(f"s_waitcnt vmcnt({min(63, n + (64 if first else 0))})")
        self.comment(f"---- chunk ({'first of a segment (' + str(first) + ')' if first else 'steady state'})")
        # step 0
        wait(24 if two else 8)  # D0 of unit G+1 has landed
        self.transform("D0")
        self.u_offset(self.sr("UoffM"), self.sr("KgM"), self.sr("Cm"), True)
        wait(16 if two else 0)  # U0 of this unit has landed
        self.e("s_waitcnt lgkmcnt(0)")  # first B operands
        self.mfma_step_with_cursors(first, lambda p: self.load_u("U1", p, self.sr("UoffM")), write_step=0)
        # step 1
        self.slab_descriptor(0)
        self.e("s_waitcnt lgkmcnt(0)")
        self.mfma_step(1, first, lambda p: self.load_patch("D0", p))
        # step 2
        if two:
            self.e("s_waitcnt vmcnt(%d)" % (63 if first else 24))  # D1 of unit G+1 has landed
            self.transform("D1")
        self.u_offset(self.sr("UoffQ"), self.sr("KgQ"), self.sr("Cq"), False)
        self.e("s_waitcnt vmcnt(16)")  # U1 (step 0) has landed; only D0 (step 1) is younger
        self.e("s_waitcnt lgkmcnt(0)")
        self.mfma_step(2, first, lambda p: self.load_u("U0", p, self.sr("UoffQ")), write_step=1 if two else None)
        # step 3
        if two:
            self.slab_descriptor(1)
        self.e("s_waitcnt lgkmcnt(0)")
        self.mfma_step(3, first, (lambda p: self.load_patch("D1", p)) if two else None)
        self.end_of_chunk()
        self.e(f"s_add_u32 {self.sr('G')}, {self.sr('G')}, 1")
        self.e(f"s_add_u32 {self.sr('Cm')}, {self.sr('Cm')}, 1")

    # ------------------------------------------------------------------ epilogue
    def row_start(self):
        """RsrcY = first filter row of the tile."""
        ry = self.S["RsrcY"]
        self.e(f"s_mov_b32 {s(ry)}, {s(self.S['Yt'])}")
        self.e(f"s_mov_b32 {s(ry + 1)}, {s(self.S['Yt'] + 1)}")
        if self.ragged_k:
            self.e(f"s_lshl_b32 {self.t(2)}, {self.sr('KgM')}, 5")   # first filter of the wave tile
            self.e(f"s_lshl_b32 {self.t(3)}, {self.sr('HWN4')}, 2")  # lane offsets below this: hsel = 0
            self.row_limit(0)

    def row_limit(self, r):
        """ragged K: num_records of the row descriptor admits the lanes whose filter exists (hsel = 0:
        filter row, offsets below 4*HWN4; hsel = 1: four rows further, offsets above)."""
        t = self.t
        ry = self.S["RsrcY"]
        self.e(f"s_add_u32 {t(0)}, {t(2)}, {8 * (r >> 2) + (r & 3)}")
        self.e(f"s_cmp_lt_u32 {t(0)}, {self.sr(self.K_REAL)}")
        self.e(f"s_cselect_b32 {t(1)}, {t(3)}, 0")
        self.e(f"s_add_u32 {t(0)}, {t(0)}, 4")
        self.e(f"s_cmp_lt_u32 {t(0)}, {self.sr(self.K_REAL)}")
        self.e(f"s_cselect_b32 {s(ry + 2)}, 0x{OOB:x}, {t(1)}")

    def row_advance(self, r):
        """RsrcY: filter row 8*(r/4) + r%4 -> the row of r+1 (the 4*hsel part is in the lane offset)."""
        if r == 15:
            return
        ry = self.S["RsrcY"]
        mult = 5 if r % 4 == 3 else 1
        for _ in range(mult):
            self.e(f"s_add_u32 {s(ry)}, {s(ry)}, {self.sr('HWN4')}")
            self.e(f"s_addc_u32 {s(ry + 1)}, {s(ry + 1)}, 0")
        if self.ragged_k:
            self.row_limit(r + 1)

    def output_transform_row(self, r, o):
        """Accumulator row r of all 16 positions -> its four outputs in o(0..3)
        (Y = A^T M A, order of src/store_and_transform_output_optSTS64.cuh:29-51)."""
        m = lambda i: self.vr("T", i)
        w = lambda i: self.vr("TO", i)          # a_j: 0-3, b_j: 4-7
        for j in range(4):
            self.e(f"v_add_f32 {w(j)}, {m(j)}, {m(4 + j)}")
            self.e(f"v_sub_f32 {w(4 + j)}, {m(4 + j)}, {m(8 + j)}")
        for j in range(4):
            self.e(f"v_add_f32 {w(j)}, {w(j)}, {m(8 + j)}")
            self.e(f"v_sub_f32 {w(4 + j)}, {w(4 + j)}, {m(12 + j)}")
        self.e(f"v_add_f32 {o(0)}, {w(0)}, {w(1)}")
        self.e(f"v_sub_f32 {o(1)}, {w(1)}, {w(2)}")
        self.e(f"v_add_f32 {o(2)}, {w(4)}, {w(5)}")
        self.e(f"v_sub_f32 {o(3)}, {w(5)}, {w(6)}")
        self.e(f"v_add_f32 {o(0)}, {o(0)}, {w(2)}")
        self.e(f"v_sub_f32 {o(1)}, {o(1)}, {w(3)}")
        self.e(f"v_add_f32 {o(2)}, {o(2)}, {w(6)}")
        self.e(f"v_sub_f32 {o(3)}, {o(3)}, {w(7)}")

    def epilogue(self, through, merge=False):
        """The output transform per accumulator element and the 64 stores of the tile; `through` =
        write past the caches (a partial tile that a workgroup on another XCD will read).
        `merge`: the partial tile that the next workgroup published is added (late_merge)."""
        # final outputs are written once and never read again by this kernel: non-temporal, so that
        # they do not push the input patches that neighbouring tiles share out of L2
        pol = " sc0 sc1" if through else " nt"
        ry = self.S["RsrcY"]
        m = lambda i: self.vr("T", i)
        if merge:
            return self.late_merge(pol)
        self.row_start()
        # the last MFMAs must have written the accumulators before they are read
        self.e("s_nop 15")
        self.e("s_nop 15")
        pending = []
        for r in range(16):
            o = lambda q: self.vr("TO", 8 + 4 * (r & 1) + q)  # outputs alternate between two sets
            for p in range(16):
                self.e(f"v_accvgpr_read_b32 {m(p)}, {a(16 * p + r)}")
            if r > 0:  # the previous row's outputs, now certainly computed: store, then move on a row
                for st in pending:
                    self.e(st)
                self.row_advance(r - 1)
            self.output_transform_row(r, o)
            pending = [f"buffer_store_dword {o(q)}, {self.vr('Eff', q)}, {s(ry, 4)}, 0 offen{pol}" for q in range(4)]
            if r == 15:
                for st in pending:
                    self.e(st)

    def late_merge(self, pol):
        """The output transform of a range that ends inside a tile of a layer with fewer tiles than
        compute units.  Every workgroup of such a tile finishes its units at about the same time,
        so the partial tile of the workgroup behind this one cannot be in the accumulators before
        the first unit as in merge_init.  All 64 outputs are computed first, into registers;
        then: wait for the flag, read the partial tile past the caches, add, store.  This is the
        last thing the workgroup does, so the pipeline's registers are free - once its last
        prefetches, which nothing waits for any more, have landed."""
        ry = self.S["RsrcY"]
        m = lambda i: self.vr("T", i)
        out, land = self.late_output_registers(), self.late_merge_registers()
        assert len(set(out + land)) == 128
        self.comment("---- late merge: outputs first, then the partial tile of the workgroup behind")
        self.e("s_waitcnt vmcnt(0) lgkmcnt(0)")
        self.e("s_nop 15")
        self.e("s_nop 15")
        for r in range(16):
            for p in range(16):
                self.e(f"v_accvgpr_read_b32 {m(p)}, {a(16 * p + r)}")
            self.output_transform_row(r, lambda q: v(out[r * 4 + q]))
        self.wait_flag()
        self.row_start()
        for r in range(16):
            for q in range(4):
                self.e(f"buffer_load_dword {v(land[r * 4 + q])}, {self.vr('Eff', q)}, {s(ry, 4)}, 0 offen sc0 sc1")
            self.row_advance(r)
        self.e("s_waitcnt vmcnt(0)")
        self.store_flag(self.vr("Zero"))  # hand the flag back for the next launch
        self.row_start()
        for r in range(16):
            for q in range(4):
                self.e(f"v_add_f32 {v(out[r * 4 + q])}, {v(out[r * 4 + q])}, {v(land[r * 4 + q])}")
            for q in range(4):
                self.e(f"buffer_store_dword {v(out[r * 4 + q])}, {self.vr('Eff', q)}, {s(ry, 4)}, 0 offen{pol}")
            self.row_advance(r)

    def flag_address(self, previous):
        """Fl = &flags[((L - previous) * 4 + wave) * 2 + 1]."""
        t = self.t
        fl = self.S["Fl"]
        self.e(f"s_sub_u32 {t(0)}, {self.sr('L')}, {1 if previous else 0}")
        self.e(f"s_lshl_b32 {t(0)}, {t(0)}, 2")
        self.e(f"s_add_u32 {t(0)}, {t(0)}, {self.sr('Wave')}")
        self.e(f"s_lshl_b32 {t(0)}, {t(0)}, 3")
        self.e(f"s_add_u32 {t(0)}, {t(0)}, 4")
        self.e(f"s_add_u32 {s(fl)}, {s(self.S['Sync'])}, {t(0)}")
        self.e(f"s_addc_u32 {s(fl + 1)}, {s(self.S['Sync'] + 1)}, 0")

    def store_flag(self, value_reg):
        self.e("s_mov_b64 exec, 1")
        self.e(f"global_store_dword {self.vr('Zero')}, {value_reg}, {s(self.S['Fl'], 2)} sc0 sc1")
        self.e("s_mov_b64 exec, -1")

    def wait_flag(self):
        """Until the workgroup behind this one has published its part of the tile.  Bounded by
        SpinLimit polls: a wave that gives up reports it in the status word (out of line) and
        goes on, so that every wave ends whatever happens to the publisher."""
        t = self.t
        self.flag_address(False)
        self.e(f"s_mov_b32 {self.sr('Spin')}, 0")
        poll, got, giveup = self.newlabel("poll"), self.newlabel("got"), self.newlabel("giveup")
        self.label(poll)
        self.e(f"global_load_dword {self.vr('Tmp')}, {self.vr('Zero')}, {s(self.S['Fl'], 2)} sc0 sc1")
        self.e("s_waitcnt vmcnt(0)")
        self.e(f"v_readfirstlane_b32 {t(0)}, {self.vr('Tmp')}")
        self.e("s_nop 4")
        self.e(f"s_cmp_lg_u32 {t(0)}, 0")
        self.e(f"s_cbranch_scc1 {got}")
        self.e(f"s_add_u32 {self.sr('Spin')}, {self.sr('Spin')}, 1")
        self.e(f"s_cmp_lt_u32 {self.sr('Spin')}, {self.sr('SpinLimit')}")
        self.e(f"s_cbranch_scc0 {giveup}")
        self.e("s_sleep 8")
        self.e(f"s_branch {poll}")
        self.label(got)
        main, self.lines = self.lines, []
        self.label(giveup)
        self.e("s_mov_b64 exec, 1")
        self.e(f"global_store_dword {self.vr('Zero')}, {self.vr('One')}, {s(self.S['Status'], 2)} sc0 sc1")
        self.e("s_mov_b64 exec, -1")
        self.e(f"s_branch {got}")
        self.outofline.extend(self.lines)
        self.lines = main

    def late_merge_registers(self):
        """64 registers for the partial tile of a late merge: the filter operands."""
        return [self.V["U0"] + i for i in range(32)] + [self.V["U1"] + i for i in range(32)]

    def late_output_registers(self):
        """64 registers for the outputs of a late merge: patches and B operands."""
        names = ["D0", "D1" if self.SPW == 2 else "MPX", "VA", "VB"]
        return [self.V[n] + i for n in names for i in range(16)]

    def merge_init(self):
        """Last segment of a workgroup that ends inside a tile: the first part of that tile was
        published by the next workgroup long ago.  Wait for its flag (bounded), read the partial
        outputs past the caches and start the accumulators from them."""
        self.comment("---- merge: accumulators start from the published partial tile")
        self.wait_flag()
        ry = self.S["RsrcY"]
        self.row_start()
        for r in range(16):
            for q in range(4):
                self.e(f"buffer_load_dword {v(self.MP[r * 4 + q])}, {self.vr('Eff', q)}, {s(ry, 4)}, 0 offen sc0 sc1")
            self.row_advance(r)
        self.e("s_waitcnt vmcnt(0)")
        # the four positions that carry the partial outputs; the other twelve start from the
        # constant 0 in the first MFMA step of the segment
        for p, (q, neg) in MERGE_POSITIONS.items():
            for r in range(16):
                reg = v(self.MP[r * 4 + q])
                if neg:
                    self.e(f"v_xor_b32 {reg}, 0x80000000, {reg}")
                self.e(f"v_accvgpr_write_b32 {a(16 * p + r)}, {reg}")
        self.store_flag(self.vr("Zero"))  # hand the flag back for the next launch
        self.e("s_nop 15")
        self.e("s_nop 15")

    def stamp(self):
        """Timeline: the workgroup's first wave appends the realtime counter to its 64-entry record
        (when a buffer was given and the record has room).  The stamp count lives in the register
        that held Begin during set-up."""
        t = self.t
        skip = self.newlabel("no_stamp")
        tl = self.S["Timeline"]
        self.e(f"s_cmp_eq_u64 {s(tl, 2)}, 0")
        self.e(f"s_cbranch_scc1 {skip}")
        self.e(f"s_cmp_lg_u32 {self.sr('Wave')}, 0")
        self.e(f"s_cbranch_scc1 {skip}")
        self.e(f"s_cmp_ge_u32 {self.sr('Begin')}, 62")
        self.e(f"s_cbranch_scc1 {skip}")
        self.e(f"s_memrealtime {s(self.S['T'] + 4, 2)}")
        self.e(f"s_lshl_b32 {t(0)}, {self.sr('L')}, 9")          # 64 x 8 bytes per workgroup
        self.e(f"s_add_u32 {t(2)}, {s(tl)}, {t(0)}")
        self.e(f"s_addc_u32 {t(3)}, {s(tl + 1)}, 0")
        self.e(f"s_lshl_b32 {t(0)}, {self.sr('Begin')}, 3")
        self.e(f"s_add_u32 {self.sr('Begin')}, {self.sr('Begin')}, 1")
        self.e("s_waitcnt lgkmcnt(0)")
        self.e("s_mov_b64 exec, 1")
        self.e(f"v_mov_b32 {self.vr('Tmp', 0)}, {t(0)}")           # byte offset of the new stamp - 16
        self.e(f"v_mov_b32 {self.vr('Tmp', 1)}, {t(4)}")
        self.e(f"global_store_dword {self.vr('Tmp', 0)}, {self.vr('Tmp', 1)}, {s(self.S['T'] + 2, 2)} offset:16")
        self.e(f"v_mov_b32 {self.vr('Tmp', 1)}, {t(5)}")
        self.e(f"global_store_dword {self.vr('Tmp', 0)}, {self.vr('Tmp', 1)}, {s(self.S['T'] + 2, 2)} offset:20")
        self.e(f"v_mov_b32 {self.vr('Tmp', 1)}, {self.sr('Begin')}")
        self.e(f"global_store_dword {self.vr('Zero')}, {self.vr('Tmp', 1)}, {s(self.S['T'] + 2, 2)}")
        self.e("s_mov_b64 exec, -1")
        self.label(skip)

    # ------------------------------------------------------------------ whole kernel
    def body(self):
        self.head()
        self.lane_setup()
        self.e(f"s_mov_b32 {self.sr('Begin')}, 0")  # from here on: number of timeline stamps
        self.stamp()
        self.prologue()
        self.segments()

    SLAB_CHANNELS = 2  # channels behind one patch-load descriptor

    def range_owner(self):
        """The register that numbers this workgroup's range of units."""
        return self.sr("L")

    def weighted_unit_range(self, owner, vt):
        """The ranges cut on a weighted line: a tile counts 2 * Chunks for its units plus the cost
        of its output transform in half units (vt = the sum; its magic number in (Mch, Sch);
        UnitsQ / UnitsRem count weighted half units), so that a range with one more tile end gets
        fewer units.  Weighted position v -> tile v / vt, chunk min((v % vt + 1) / 2, Chunks)."""
        t, e = self.t, self.e
        for which, dst in ((0, self.sr("Begin")), (1, t(5))):
            if which:
                e(f"s_add_u32 {t(0)}, {owner}, 1")
            else:
                e(f"s_mov_b32 {t(0)}, {owner}")
            e(f"s_mul_i32 {t(1)}, {t(0)}, {self.sr('UnitsQ')}")
            e(f"s_min_u32 {t(2)}, {t(0)}, {self.sr('UnitsRem')}")
            e(f"s_add_u32 {t(1)}, {t(1)}, {t(2)}")          # weighted start of range `owner + which`
            self.div(t(2), t(1), self.sr("Mch"), self.sr("Sch"))  # tile
            e(f"s_mul_i32 {t(3)}, {t(2)}, {vt}")
            e(f"s_sub_u32 {t(3)}, {t(1)}, {t(3)}")
            e(f"s_add_u32 {t(3)}, {t(3)}, 1")
            e(f"s_lshr_b32 {t(3)}, {t(3)}, 1")
            e(f"s_min_u32 {t(3)}, {t(3)}, {self.sr('Chunks')}")  # chunk
            if not which:
                e(f"s_mov_b32 {self.sr('Tm')}, {t(2)}")
                e(f"s_mov_b32 {self.sr('Cm')}, {t(3)}")
            e(f"s_mul_i32 {t(2)}, {t(2)}, {self.sr('Chunks')}")
            e(f"s_add_u32 {dst}, {t(2)}, {t(3)}")
        e(f"s_sub_u32 {self.sr('Nunits')}, {t(5)}, {self.sr('Begin')}")
        # a weighted start behind a tile's last chunk is the next tile's first unit
        e(f"s_cmp_eq_u32 {self.sr('Cm')}, {self.sr('Chunks')}")
        e(f"s_cselect_b32 {self.sr('Cm')}, 0, {self.sr('Cm')}")
        e(f"s_addc_u32 {self.sr('Tm')}, {self.sr('Tm')}, 0")

    def unit_range(self, owner):
        """Begin, Nunits (units [Begin, Begin + Nunits): the first UnitsRem ranges take one more)
        and the first unit's tile Tm and chunk Cm.  Bits 8.. of the magic shift Sch (which 64-bit
        shifts ignore), when not zero: the weight of an output transform in half units, and the
        ranges are cut on the weighted line (weighted_unit_range)."""
        t, e = self.t, self.e
        plain, done = self.newlabel("plain_ranges"), self.newlabel("ranges_done")
        e(f"s_lshr_b32 {self.sr('Kind')}, {self.sr('Sch')}, 8")  # Kind, SegEnd: free until the segment loop
        e(f"s_cmp_eq_u32 {self.sr('Kind')}, 0")
        e(f"s_cbranch_scc1 {plain}")
        e(f"s_lshl_b32 {self.sr('SegEnd')}, {self.sr('Chunks')}, 1")
        e(f"s_add_u32 {self.sr('SegEnd')}, {self.sr('SegEnd')}, {self.sr('Kind')}")
        self.weighted_unit_range(owner, self.sr("SegEnd"))
        e(f"s_branch {done}")
        self.label(plain)
        self.plain_unit_range(owner)
        self.label(done)

    def plain_unit_range(self, owner):
        t, e = self.t, self.e
        e(f"s_mul_i32 {self.sr('Begin')}, {owner}, {self.sr('UnitsQ')}")
        e(f"s_min_u32 {t(0)}, {owner}, {self.sr('UnitsRem')}")
        e(f"s_add_u32 {self.sr('Begin')}, {self.sr('Begin')}, {t(0)}")
        e(f"s_cmp_lt_u32 {owner}, {self.sr('UnitsRem')}")
        e(f"s_cselect_b32 {t(0)}, 1, 0")
        e(f"s_add_u32 {self.sr('Nunits')}, {self.sr('UnitsQ')}, {t(0)}")
        self.div(self.sr("Tm"), self.sr("Begin"), self.sr("Mch"), self.sr("Sch"))
        e(f"s_mul_i32 {t(0)}, {self.sr('Tm')}, {self.sr('Chunks')}")
        e(f"s_sub_u32 {self.sr('Cm')}, {self.sr('Begin')}, {t(0)}")

    def head(self):
        """Kernel arguments, wave / workgroup identity, the unit range, cursors, descriptors."""
        S, t = self.S, self.t
        e = self.e
        KWLOG = self.KW.bit_length() - 1
        e(f"s_load_dwordx8 {s(8, 8)}, s[0:1], 0x0")
        e(f"s_load_dwordx16 {s(16, 16)}, s[0:1], 0x20")
        e(f"s_load_dwordx8 {s(32, 8)}, s[0:1], 0x60")
        e(f"s_load_dwordx2 {s(40, 2)}, s[0:1], 0x80")
        e(f"s_load_dwordx2 {s(S['Status'], 2)}, s[0:1], 0x88")
        e(f"s_load_dword {self.sr('SpinLimit')}, s[0:1], 0x90")
        e(f"v_and_b32 {self.vr('Tmp', 1)}, 0x3ff, v0")
        e(f"v_lshrrev_b32 {self.vr('Tmp')}, 6, {self.vr('Tmp', 1)}")
        e(f"v_and_b32 {self.vr('Lane')}, 63, {self.vr('Tmp', 1)}")
        e(f"v_mov_b32 {self.vr('Zero')}, 0")
        e(f"v_mov_b32 {self.vr('One')}, 1")
        e(f"v_mov_b32 {self.vr('Oob')}, 0x{OOB:x}")
        e("s_waitcnt lgkmcnt(0)")
        # only now: a vector instruction that writes an SGPR while scalar loads are still
        # outstanding came back with a corrupted value on this part
        e(f"v_readfirstlane_b32 {self.sr('Wave')}, {self.vr('Tmp')}")
        e("s_nop 4")
        e(f"s_and_b32 {self.sr('Kw')}, {self.sr('Wave')}, {self.KW - 1}")
        e(f"s_lshr_b32 {self.sr('Cw')}, {self.sr('Wave')}, {KWLOG}")
        e(f"s_mul_i32 {self.sr('KwSpw')}, {self.sr('Kw')}, {self.SPW}")
        # logical block: workgroups are dealt round-robin to the 8 XCDs; each XCD gets a contiguous range
        # (GridPerXcd == 0: a grid that does not divide by 8, a small layer; blocks in launch order)
        e(f"s_and_b32 {t(0)}, s2, 7")
        e(f"s_mul_i32 {t(0)}, {t(0)}, {self.sr('GridPerXcd')}")
        e(f"s_lshr_b32 {t(1)}, s2, 3")
        e(f"s_add_u32 {t(0)}, {t(0)}, {t(1)}")
        e(f"s_cmp_eq_u32 {self.sr('GridPerXcd')}, 0")
        e(f"s_cselect_b32 {self.sr('L')}, s2, {t(0)}")
        self.unit_range(self.range_owner())
        # the arguments of place(), into registers that are free from here on
        e(f"s_load_dword {self.sr('PlaceM')}, s[0:1], 0x94")
        e(f"s_load_dword {self.sr('PlaceS')}, s[0:1], 0x98")
        e(f"s_load_dword {self.sr('PlaceG')}, s[0:1], 0x9c")
        e(f"s_load_dword {self.sr('PlaceTn')}, s[0:1], 0xa0")
        e("s_waitcnt lgkmcnt(0)")
        for n in ("Tp", "Tq"):
            e(f"s_mov_b32 {self.sr(n)}, {self.sr('Tm')}")
        for n in ("Cp", "Cq"):
            e(f"s_mov_b32 {self.sr(n)}, {self.sr('Cm')}")
        e(f"s_lshl_b32 {self.sr('ColStep')}, {self.sr('N')}, 2")
        e(f"s_mul_i32 {self.sr('RowStep')}, {self.sr('ColStep')}, {self.sr('W')}")
        e(f"s_lshl_b32 {self.sr('Slab')}, {self.sr('HWN4')}, {self.SLAB_CHANNELS.bit_length() - 1}")
        # descriptors: words 2 (num_records) and 3 (flags) never change
        e(f"s_mov_b32 {s(S['RsrcX'] + 2)}, {self.sr('Slab')}")
        e(f"s_mov_b32 {s(S['RsrcX'] + 3)}, 0x{FLAGS:x}")
        e(f"s_mov_b32 {s(S['RsrcU'])}, {s(S['U'])}")
        e(f"s_mov_b32 {s(S['RsrcU'] + 1)}, {s(S['U'] + 1)}")
        e(f"s_mov_b32 {s(S['RsrcU'] + 2)}, {self.sr('UswBytes')}")
        e(f"s_mov_b32 {s(S['RsrcU'] + 3)}, 0x{FLAGS:x}")
        e(f"s_mov_b32 {s(S['RsrcY'] + 2)}, 0x{OOB:x}")
        e(f"s_mov_b32 {s(S['RsrcY'] + 3)}, 0x{FLAGS:x}")

    def lane_setup(self):
        """Per-lane registers: patch / store offsets, filter-load offsets, LDS addresses."""
        t, e = self.t, self.e
        tmp = lambda i: self.vr("Tmp", i)
        e(f"v_lshrrev_b32 {tmp(0)}, 5, {self.vr('Lane')}")             # hsel
        e(f"v_and_b32 {tmp(1)}, 31, {self.vr('Lane')}")                # nl
        e(f"v_lshlrev_b32 {tmp(1)}, 2, {tmp(1)}")                      # nl*4
        e(f"v_mul_lo_u32 {tmp(2)}, {tmp(0)}, {self.sr('HWN4')}")       # hsel*HWN*4
        e(f"v_add_u32 {self.vr('LaneX')}, {tmp(2)}, {tmp(1)}")
        e(f"v_lshlrev_b32 {tmp(2)}, 2, {tmp(2)}")                      # 4*hsel*HWN*4
        e(f"v_add_u32 {self.vr('Off', 0)}, {tmp(2)}, {tmp(1)}")
        e(f"v_add_u32 {self.vr('Off', 1)}, {self.sr('ColStep')}, {self.vr('Off', 0)}")
        e(f"v_add_u32 {self.vr('Off', 2)}, {self.sr('RowStep')}, {self.vr('Off', 0)}")
        e(f"v_add_u32 {self.vr('Off', 3)}, {self.sr('ColStep')}, {self.vr('Off', 2)}")
        e(f"v_lshlrev_b32 {self.vr('LaneU')}, 4, {self.vr('Lane')}")
        e(f"v_add_u32 {self.vr('LaneUb')}, 0x1000, {self.vr('LaneU')}")
        # LDS: V[cw][buf][step][p][lane] floats.  Lds = read buffer, LdsWr = write buffer + this
        # wave's first owned step; the prologue writes buffer 0, which the swap in end_of_chunk
        # then makes the read buffer.
        e(f"v_lshlrev_b32 {tmp(0)}, 2, {self.vr('Lane')}")
        e(f"s_lshl_b32 {t(0)}, {self.sr('Cw')}, 15")
        e(f"v_add_u32 {tmp(0)}, {t(0)}, {tmp(0)}")
        e(f"v_add_u32 {self.vr('Lds')}, 0x4000, {tmp(0)}")
        e(f"s_lshl_b32 {t(0)}, {self.sr('KwSpw')}, 12")
        e(f"v_add_u32 {self.vr('LdsWr')}, {t(0)}, {tmp(0)}")

    def prologue(self):
        """Unit 0 -> buffer 0 with the patches of unit 1 already in flight.  Unit 0's patches land
        in registers that are free until the first chunk (MPX, VB), so that both units' loads
        leave together and the kernel pays one trip to memory, not two."""
        e = self.e
        self.decode(self.sr("Tm"))
        self.m_tile_setup()
        e(f"s_mov_b32 {self.sr('KgQ')}, {self.sr('KgM')}")
        self.patch_offsets()
        self.u_offset(self.sr("UoffQ"), self.sr("KgM"), self.sr("Cm"), False)
        first_patch = ["MPX", "VB"]
        for j in range(self.SPW):
            self.slab_descriptor(j)
            for p in range(16):
                self.load_patch(first_patch[j], p)
        for p in range(16):
            self.load_u("U0", p, self.sr("UoffQ"))
        e(f"s_mov_b32 {self.sr('G')}, -1")
        self.advance_p()  # G + 2 = 1: on to unit 1 when there is one
        for j in range(self.SPW):
            self.slab_descriptor(j)
            for p in range(16):
                self.load_patch("D0" if j == 0 else "D1", p)
        e(f"s_mov_b32 {self.sr('G')}, 0")
        e(f"s_waitcnt vmcnt({16 * self.SPW})")  # everything but unit 1's patches
        for j in range(self.SPW):
            self.transform(first_patch[j])
            for p in range(0, 16, 2):
                self.write_v(j, p)
        self.end_of_chunk()
        e("s_waitcnt vmcnt(0)")  # the first chunk counts on a queue without surprises

    def segments(self):
        """The segment loop: chunks of one tile, then its output transform (plain, published, or
        started from a published partial tile)."""
        t, e = self.t, self.e
        seg_loop, regular, check, done = (self.newlabel(x) for x in ("seg", "regular", "check", "done"))
        plain_seg, epi_plain, after_epi = (self.newlabel(x) for x in ("plainseg", "epiplain", "afterepi"))
        self.stamp()
        self.label(seg_loop)
        # this segment: chunks Cm .. SegEnd-1 of tile Tm.  Kind: 1 publish (starts inside the tile),
        # 2 merge (ends inside the tile), 0 whole tile.
        e(f"s_sub_u32 {t(0)}, {self.sr('Nunits')}, {self.sr('G')}")
        e(f"s_sub_u32 {t(1)}, {self.sr('Chunks')}, {self.sr('Cm')}")
        e(f"s_min_u32 {t(0)}, {t(0)}, {t(1)}")
        e(f"s_add_u32 {self.sr('SegEnd')}, {self.sr('Cm')}, {t(0)}")
        e(f"s_cmp_lg_u32 {self.sr('Cm')}, 0")
        e(f"s_cselect_b32 {self.sr('Kind')}, 1, 0")
        e(f"s_cmp_lt_u32 {self.sr('SegEnd')}, {self.sr('Chunks')}")
        e(f"s_cbranch_scc0 {plain_seg}")
        # a range shorter than a tile: the merge waits until the output transform (Kind 4 and 5)
        e(f"s_or_b32 {t(0)}, {self.sr('Kind')}, 4")
        e(f"s_cmp_lt_u32 {self.sr('Nunits')}, {self.sr('Chunks')}")
        e(f"s_cselect_b32 {self.sr('Kind')}, {t(0)}, 2")
        e(f"s_cbranch_scc1 {plain_seg}")
        self.merge_init()
        self.chunk("merge")
        e(f"s_branch {check}")
        self.label(plain_seg)
        self.chunk(True)
        self.label(check)
        e(f"s_cmp_lt_u32 {self.sr('Cm')}, {self.sr('SegEnd')}")
        e(f"s_cbranch_scc0 {epi_plain}")
        self.label(regular)
        self.chunk(False)
        e(f"s_cmp_lt_u32 {self.sr('Cm')}, {self.sr('SegEnd')}")
        e(f"s_cbranch_scc1 {regular}")
        self.label(epi_plain)
        self.stamp()
        pub, late, late_pub, flag = (self.newlabel(x) for x in ("publish", "late", "latepub", "flag"))
        e(f"s_cmp_eq_u32 {self.sr('Kind')}, 1")
        e(f"s_cbranch_scc1 {pub}")
        e(f"s_cmp_ge_u32 {self.sr('Kind')}, 4")
        e(f"s_cbranch_scc1 {late}")
        self.epilogue(False)
        e(f"s_branch {after_epi}")
        self.label(pub)
        self.epilogue(True)
        self.label(flag)
        e("s_waitcnt vmcnt(0)")  # every write-through store acknowledged, then the flag
        self.flag_address(True)
        self.store_flag(self.vr("One"))  # nothing waits for it: the data it announces is acknowledged
        self.label(after_epi)
        self.stamp()
        e(f"s_cmp_lt_u32 {self.sr('G')}, {self.sr('Nunits')}")
        e(f"s_cbranch_scc0 {done}")
        e(f"s_add_u32 {self.sr('Tm')}, {self.sr('Tm')}, 1")
        e(f"s_mov_b32 {self.sr('Cm')}, 0")
        self.decode(self.sr("Tm"))
        self.m_tile_setup()
        e(f"s_branch {seg_loop}")
        self.label(done)
        e("s_endpgm")
        # the output transforms with a late merge (layers with few tiles only)
        self.label(late)
        e(f"s_cmp_eq_u32 {self.sr('Kind')}, 5")
        e(f"s_cbranch_scc1 {late_pub}")
        self.epilogue(False, merge=True)
        e(f"s_branch {after_epi}")
        self.label(late_pub)
        self.epilogue(True, merge=True)
        e(f"s_branch {flag}")
        self.lines.extend(self.outofline)

    def emit(self, out):
        self.body()
        n = self.name
        out.append(f"\t.text\n\t.protected\t{n}\n\t.globl\t{n}\n\t.p2align\t8\n\t.type\t{n},@function\n{n}:")
        out.extend(self.lines)
        out.append(f".L{n}_end:\n\t.size\t{n}, .L{n}_end-{n}")
        out.append(f"""\t.rodata
\t.p2align\t6
\t.amdhsa_kernel {n}
\t\t.amdhsa_group_segment_fixed_size 0
\t\t.amdhsa_private_segment_fixed_size 0
\t\t.amdhsa_kernarg_size 168
\t\t.amdhsa_user_sgpr_count 2
\t\t.amdhsa_user_sgpr_kernarg_segment_ptr 1
\t\t.amdhsa_system_sgpr_workgroup_id_x 1
\t\t.amdhsa_system_vgpr_workitem_id 0
\t\t.amdhsa_next_free_vgpr 512
\t\t.amdhsa_next_free_sgpr {self.sgpr_count}
\t\t.amdhsa_accum_offset 256
\t\t.amdhsa_reserve_vcc 1
\t\t.amdhsa_float_round_mode_32 0
\t\t.amdhsa_float_denorm_mode_32 3
\t\t.amdhsa_float_denorm_mode_16_64 3
\t\t.amdhsa_dx10_clamp 1
\t\t.amdhsa_ieee_mode 1
\t.end_amdhsa_kernel""")

    def metadata(self):
        args = "\n".join(f"""      - .address_space:  global
        .offset:         {8 * i}
        .size:           8
        .value_kind:     global_buffer""" for i in range(4))
        args += "\n" + "\n".join(f"""      - .offset:         {32 + 4 * i}
        .size:           4
        .value_kind:     by_value""" for i in range(24))
        args += """
      - .address_space:  global
        .offset:         128
        .size:           8
        .value_kind:     global_buffer
      - .address_space:  global
        .offset:         136
        .size:           8
        .value_kind:     global_buffer
      - .offset:         144
        .size:           4
        .value_kind:     by_value
      - .offset:         148
        .size:           4
        .value_kind:     by_value
      - .offset:         152
        .size:           4
        .value_kind:     by_value
      - .offset:         156
        .size:           4
        .value_kind:     by_value
      - .offset:         160
        .size:           4
        .value_kind:     by_value
      - .offset:         164
        .size:           4
        .value_kind:     by_value"""
        return f"""  - .agpr_count:     256
    .args:
{args}
    .group_segment_fixed_size: 0
    .kernarg_segment_align: 8
    .kernarg_segment_size: 168
    .max_flat_workgroup_size: 256
    .name:           {self.name}
    .private_segment_fixed_size: 0
    .sgpr_count:     {self.sgpr_count + 6}
    .sgpr_spill_count: 0
    .symbol:         {self.name}.kd
    .uniform_work_group_size: 1
    .uses_dynamic_stack: false
    .vgpr_count:     512
    .vgpr_spill_count: 0
    .wavefront_size: 64"""


def main():
    out = ['\t.amdgcn_target "amdgcn-amd-amdhsa--gfx950"', "\t.amdhsa_code_object_version 6"]
    kernels = [Kernel(2), Kernel(4), Kernel(2, ragged=True), Kernel(4, ragged=True),
               Kernel(2, ragged=True, packed=True), Kernel(4, ragged=True, packed=True)]
    for k in kernels:
        k.emit(out)
    out.append("\t.amdgpu_metadata\n---\namdhsa.kernels:")
    out.extend(k.metadata() for k in kernels)
    out.append("amdhsa.target:   amdgcn-amd-amdhsa--gfx950\namdhsa.version:\n  - 1\n  - 2\n...\n\t.end_amdgpu_metadata")
    sys.stdout.write("\n".join(out) + "\n")


if __name__ == "__main__":
    main()
