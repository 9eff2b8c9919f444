#!/usr/bin/env python3
"""Generator of the hand-scheduled gfx950 assembly of the fused Winograd F(2x2,3x3) kernel with
fp16 / bf16 GEMM operands: wino_f16_asm_kw4 and wino_bf16_asm_kw4.

Same persistent launch, unit split, publish / merge of cut tiles, output transform and kernel
arguments as the fp32 kernels of gen_wino_f32_asm.py (whose Kernel class this one extends), and
the same mathematics as wino_h16_fused_lds in conv_kernel_h16.hpp: transforms in fp32, the
transformed input V rounded to nearest-even on its way into LDS, the transformed filter U
rounded by the filter transform (fx_mfma_layout_h16), v_mfma_f32_32x32x16_{f16,bf16} with fp32
accumulators.  The reference has no such path (it is fp32 only).

What differs from the fp32 kernels:

  * a unit is a 16-channel chunk: ONE MFMA per Winograd position.  The matrix pipe needs 512
    cycles per unit while the operands of a unit are 96 KB per workgroup (64 KB of filters, 32 KB
    of patches) through a 64 B/clk vector memory path, so the kernel is bound by operand
    delivery and the schedule is built around the loads: every filter register is reloaded for
    the next unit right behind the MFMA that consumed it, every patch register right behind
    the transform that consumed it, which keeps one unit of loads in flight all the time;
  * fp32 VALU work co-issues with the fp16 / bf16 MFMAs (unlike the fp32 MFMAs), so the input
    transform is simply spread behind the MFMAs of the second half of a unit;
  * a lane transforms two ADJACENT channels of one batch element and packs the two results of
    a position into one dword (v_cvt_pk_*), written to V[buf][p][h][q''][n] with
    q'' = (q & 1) * 2 + (q >> 1), so that one ds_read2st64_b32 returns the dwords q = 0, 1 and a
    second one q = 2, 3 of a lane's 8-channel B operand;
  * workgroup tiles are enumerated column-block major (the filter blocks of one column block
    are neighbours in time and place, so the patches they share are still in L2, and the
    2-byte transformed filter is small enough for all blocks to stay there too);
  * s_waitcnt counts are derived by the generator from the issue order of the loads.

Any N, C, K (api.hip pads the transformed filter with zeros to whole chunks of 16 channels and
pairs of 32-wide filter groups).  In every kernel, waves of the last filter block without filters
load and store nothing (filter_descriptor); the _ragged kernels also mask batch elements and
filter rows that do not exist, as the _ragged fp32 kernels do, and end the last chunk's slab with
the tensor (slab_descriptor).

Usage: gen_wino_h16_asm.py > wino_h16_asm.s
"""
import sys

from gen_wino_f32_asm import MERGE_POSITIONS, Alloc, Kernel, a, s, v

RING = 8   # B operands in registers (positions)
LEAD = 3   # positions the LDS reads run ahead of the MFMAs


class Wait:
    """Placeholder of an s_waitcnt whose count is resolved when the chunk is complete."""

    def __init__(self, counter, tag):
        self.counter, self.tag = counter, tag


class KernelH16(Kernel):
    SLAB_CHANNELS = 4
    K_REAL = "Q"  # the argument slot Q (twice the chunks per tile in the fp32 kernels) carries K here
    CW_IS_FREE = True  # one column tile per workgroup: Cw is zero and nothing here reads it

    def __init__(self, bf16, ragged=False, packed=False):
        """ragged: shapes outside N % 32 == 0, C % 16 == 0, K % 32 == 0 (masked lanes and rows, a
        slab descriptor that ends with the tensor; a few scalar instructions per unit and row).
        packed: a _ragged kernel for batches that are no multiple of 32 (Kernel.lane_tile)."""
        self.bf16 = bf16
        self.KW, self.CW, self.SPW = 4, 1, 1
        self.ragged = False  # the fp32 kernels' two-channel slab logic is replaced, see slab_descriptor
        self.ragged_c = self.ragged_n = self.ragged_k = ragged
        self.packed = packed
        self.lines, self.outofline, self.nlabel = [], [], 0
        self.name = (f"wino_{'bf16' if bf16 else 'f16'}_asm_kw4" +
                     ("_packed" if packed else "_ragged" if ragged else ""))
        self.alloc()

    # ------------------------------------------------------------------ registers
    def alloc_vgprs(self):
        V = Alloc(1, 256)
        self.V = {}
        for n, cnt, al in [("Lane", 1, 1), ("LaneX", 1, 1), ("Lds", 1, 1), ("Lds2", 1, 1), ("LdsWr", 1, 1),
                           ("Zero", 1, 1), ("One", 1, 1), ("Oob", 1, 1), ("Tmp", 4, 2), ("Lane16", 4, 1),
                           ("Off", 4, 1), ("Eff", 4, 1), ("VOFF", 16, 1),
                           ("U", 64, 4), ("VR", 4 * RING, 4),
                           ("DA0", 16, 1), ("DB0", 16, 1), ("DA1", 16, 1), ("DB1", 16, 1),
                           ("T", 16, 2), ("TA", 16, 2), ("TB", 16, 2)]:
            self.V[n] = V.get(n, cnt, al)
        self.V["TO"] = self.V["TA"]  # the output transform's temporaries
        self.V["MPX"] = self.V["VR"]  # the ring is dead between two chunks
        self.vgpr_count = V.next
        self.MP = [self.V[n] + i for n in ("T", "TA", "TB", "MPX") for i in range(16)]

    # ------------------------------------------------------------------ tile order
    # Two ways to deal the units, chosen by the host through the sign of the argument that carries
    # the channel count (+C: way 0, -C: way 1):
    #   0  one line of (column block, chunk) units PER FILTER BLOCK.  The workgroups L = r*B + b
    #      (B filter blocks, a power of two; the Colblocks slot holds B, the Scb slot log2 B) own
    #      range r of filter block b: the B workgroups of a range sit on neighbouring CUs of one
    #      XCD and walk through the same patches at the same time, so all but one of them find
    #      them in L2.  A tile index is the column block.
    #   1  one line of (filter block, column block, chunk) units, filter-block major, as in the
    #      fp32 kernels (an XCD then works through one filter block's share of the filters).
    def alloc_sgprs(self):
        super().alloc_sgprs()
        S = Alloc(self.sgpr_count, 102)
        self.S["Lr"] = S.get("Lr")
        self.S["Kbf"] = S.get("Kbf")
        self.sgpr_count = S.next

    def head(self):
        """After the common set-up: the time-aligned chunk order.  A workgroup's g-th unit works on
        chunk g mod Chunks of its tile, so that all workgroups (they start together) are at the
        same chunk index at the same time and neighbouring tiles find their shared patch
        columns and rows in L2.  The sum over the chunks of a tile does not care about the
        order; a tile cut between two workgroups is shared as: the workgroup whose range starts
        inside it takes chunks 0 .. N1-1 (its first units, in step with everybody), the one
        whose range ends inside it takes the last Nlast chunks (the only units out of step).
          N1     units of the first tile (Chunks when the range starts with a whole tile)
          Sfull  N1 mod Chunks: the chunk index at which every later tile of the range starts
          Tlast  last tile of the range, Nlast its units (both left by unit_range)
        They live in argument registers that are dead after this set-up."""
        super().head()
        t, e = self.t, self.e
        self.S.update(N1=self.S["Kreal"], Sfull=self.S["UnitsQ"], Tlast=self.S["UnitsRem"], Nlast=self.S["Mch"])
        e(f"s_sub_u32 {t(0)}, {self.sr('Chunks')}, {self.sr('Cm')}")
        e(f"s_cmp_eq_u32 {self.sr('Cm')}, 0")
        e(f"s_cselect_b32 {self.sr('N1')}, {self.sr('Chunks')}, {t(0)}")
        e(f"s_cselect_b32 {self.sr('Sfull')}, 0, {t(0)}")
        # A layer with fewer tiles than compute units (the host sets bit 6 of the magic shift Sch,
        # which 64-bit shifts ignore): the ranges are shorter than a tile and a tile may have
        # three or more contributors, so every range works on its own chunks in the natural
        # order - from Cm to the end of its first tile, then from chunk 0 of the next.
        e(f"s_bitcmp1_b32 {self.sr('Sch')}, 6")
        e(f"s_cselect_b32 {self.sr('Cm')}, {self.sr('Cm')}, 0")
        e(f"s_cselect_b32 {self.sr('Sfull')}, 0, {self.sr('Sfull')}")
        e(f"s_cselect_b32 {self.sr('Nlast')}, {self.sr('Chunks')}, {self.sr('Nlast')}")
        for n in ("Cp", "Cq"):
            e(f"s_mov_b32 {self.sr(n)}, {self.sr('Cm')}")

    def advance_cursor(self, T, C, ahead, hint, on_switch):
        """Cursor (T, C) -> unit G+ahead when there is one: next chunk index modulo Chunks; the
        tile ends where the index reaches Sfull (out of line: not inside the last tile), and the
        last tile starts at Chunks - Nlast."""
        rare, back = self.newlabel(hint + "_switch"), self.newlabel(hint + "_back")
        t = self.t
        self.e(f"s_add_u32 {t(0)}, {self.sr('G')}, {ahead}")
        self.e(f"s_cmp_lt_u32 {t(0)}, {self.sr('Nunits')}")
        self.e(f"s_addc_u32 {C}, {C}, 0")
        self.e(f"s_cmp_eq_u32 {C}, {self.sr('Chunks')}")
        self.e(f"s_cselect_b32 {C}, 0, {C}")
        self.e(f"s_cmp_eq_u32 {C}, {self.sr('Sfull')}")
        self.e(f"s_cbranch_scc1 {rare}")
        self.label(back)
        main, self.lines = self.lines, []
        self.label(rare)
        self.e(f"s_cmp_eq_u32 {T}, {self.sr('Tlast')}")
        self.e(f"s_cbranch_scc1 {back}")
        self.e(f"s_add_u32 {T}, {T}, 1")
        self.e(f"s_sub_u32 {t(0)}, {self.sr('Chunks')}, {self.sr('Nlast')}")
        self.e(f"s_cmp_eq_u32 {T}, {self.sr('Tlast')}")
        self.e(f"s_cselect_b32 {C}, {t(0)}, {C}")
        on_switch()
        self.e(f"s_branch {back}")
        self.outofline.extend(self.lines)
        self.lines = main

    def late_merge_registers(self):
        return [self.V["U"] + i for i in range(64)]

    def late_output_registers(self):
        return [self.V[n] + i for n in ("DA0", "DB0", "DA1", "DB1") for i in range(16)]

    def advance_p(self, ahead=3):
        def switch():
            self.decode(self.sr("Tp"))
            self.patch_offsets()
        self.advance_cursor(self.sr("Tp"), self.sr("Cp"), ahead, "p", switch)

    def advance_q(self):
        def switch():
            t = self.t
            self.filter_block(t(0), self.sr("Tq"))
            self.e(f"s_lshl_b32 {t(0)}, {t(0)}, 2")
            self.e(f"s_add_u32 {self.sr('KgQ')}, {t(0)}, {self.sr('Kw')}")
            self.filter_descriptor(self.sr("KgQ"))
        self.advance_cursor(self.sr("Tq"), self.sr("Cq"), 1, "q", switch)

    def unit_range(self, owner):
        """The ranges are cut on a weighted line: a tile counts 2 * Chunks for its units plus the
        cost of its output transform in half units (a unit here is four times shorter than an
        fp32 one, so a range with one more tile end would otherwise finish 2 us late).  VT = the
        weighted length of a tile arrives in the argument slot of the ragged kernels' real filter
        count, its magic number in (Mch, Sch); UnitsQ / UnitsRem count weighted half units.
        Weighted position v -> tile v / VT, chunk min((v % VT + 1) / 2, Chunks)."""
        t, e = self.t, self.e
        vt = self.sr("Kreal")
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
            else:
                e(f"s_mov_b32 {t(4)}, {t(2)}")
            e(f"s_mul_i32 {t(2)}, {t(2)}, {self.sr('Chunks')}")
            e(f"s_add_u32 {dst}, {t(2)}, {t(3)}")
        e(f"s_sub_u32 {self.sr('Nunits')}, {t(5)}, {self.sr('Begin')}")
        # the range ends in front of (tile T4, chunk T3): its last tile and the units it has there.
        # They replace UnitsRem and Mch, which are dead from here on (see head).
        e(f"s_sub_u32 {t(0)}, {t(4)}, 1")
        e(f"s_cmp_eq_u32 {t(3)}, 0")
        e(f"s_cselect_b32 {self.sr('UnitsRem')}, {t(0)}, {t(4)}")
        e(f"s_cselect_b32 {self.sr('Mch')}, {self.sr('Chunks')}, {t(3)}")
        # a weighted start that falls on a tile's last chunk boundary is the next tile's first unit
        e(f"s_cmp_eq_u32 {self.sr('Cm')}, {self.sr('Chunks')}")
        e(f"s_cselect_b32 {self.sr('Cm')}, 0, {self.sr('Cm')}")
        e(f"s_addc_u32 {self.sr('Tm')}, {self.sr('Tm')}, 0")

    # ------------------------------------------------------------------ filter groups that do not exist
    # The last filter block may hold fewer than four filter groups (K <= 96 mod 128).  The waves
    # without one still share the input transform of the column tile; they multiply zeros (their
    # filter descriptor is empty, so their loads touch no memory) and store nothing.  A group that
    # exists in part (K % 32 != 0) finds zero rows in the padded transformed filter and stores
    # its real rows only (row_limit).  The argument slot Q carries K.
    def u_offset(self, dst, kg, c, second):
        t = self.t
        self.e(f"s_mul_i32 {t(0)}, {kg}, {self.sr('Chunks')}")
        self.e(f"s_add_u32 {t(0)}, {t(0)}, {c}")
        self.e(f"s_lshl_b32 {dst}, {t(0)}, 14")

    def filter_descriptor(self, kg):
        """RsrcU covers the transformed filter, or nothing when filter group kg does not exist."""
        t = self.t
        self.e(f"s_lshl_b32 {t(3)}, {kg}, 5")
        self.e(f"s_cmp_lt_u32 {t(3)}, {self.sr('Q')}")
        self.e(f"s_cselect_b32 {s(self.S['RsrcU'] + 2)}, {self.sr('UswBytes')}, 0")

    def m_tile_setup(self):
        t = self.t
        self.e(f"s_lshl_b32 {t(0)}, {self.sr('Dkb')}, 2")
        self.e(f"s_add_u32 {t(0)}, {t(0)}, {self.sr('Kw')}")
        self.e(f"s_lshl_b32 {t(0)}, {t(0)}, 5")
        self.e(f"s_cmp_lt_u32 {t(0)}, {self.sr('Q')}")
        self.e(f"s_cselect_b32 {self.sr('Dlive')}, {self.sr('Dlive')}, 0")
        super().m_tile_setup()

    def slab_descriptor(self, j):
        """RsrcX = the four-channel slab of this wave in chunk Cp, cut where the tensor ends: the
        channels past a count that is no multiple of 16 read as zeros (the SGPR offset that selects
        a lane's second channel takes part in the range check of the load)."""
        t = self.t
        rx = self.S["RsrcX"]
        self.e(f"s_lshl_b32 {t(0)}, {self.sr('Cp')}, 2")
        self.e(f"s_add_u32 {t(0)}, {t(0)}, {self.sr('KwSpw')}")
        if self.ragged_c:
            self.e(f"s_abs_i32 {t(2)}, {self.sr('Creal')}")
            self.e(f"s_lshl_b32 {t(1)}, {t(0)}, 2")
            self.e(f"s_sub_i32 {t(2)}, {t(2)}, {t(1)}")
            self.e(f"s_max_i32 {t(2)}, {t(2)}, 0")
            self.e(f"s_min_i32 {t(2)}, {t(2)}, 4")
            self.e(f"s_mul_i32 {s(rx + 2)}, {t(2)}, {self.sr('HWN4')}")
        self.e(f"s_mul_hi_u32 {t(1)}, {t(0)}, {self.sr('Slab')}")
        self.e(f"s_mul_i32 {t(0)}, {t(0)}, {self.sr('Slab')}")
        self.e(f"s_add_u32 {s(rx)}, {s(self.S['X'])}, {t(0)}")
        self.e(f"s_addc_u32 {s(rx + 1)}, {s(self.S['X'] + 1)}, {t(1)}")

    def range_owner(self):
        t = self.t
        self.e(f"s_cmp_gt_i32 {self.sr('Creal')}, 0")
        self.e(f"s_cselect_b32 {t(0)}, {self.sr('Scb')}, 0")
        self.e(f"s_lshr_b32 {self.sr('Lr')}, {self.sr('L')}, {t(0)}")
        self.e(f"s_sub_u32 {t(0)}, {self.sr('Colblocks')}, 1")
        self.e(f"s_and_b32 {self.sr('Kbf')}, {self.sr('L')}, {t(0)}")
        return self.sr("Lr")

    def split_tile(self, T):
        """T -> T0 (column block), Dkb (filter block)."""
        t = self.t
        self.place(T)
        self.div(t(1), t(5), self.sr("Mcb"), self.sr("Scb"))  # meaningless in mode 0, not used there
        self.e(f"s_mul_i32 {t(0)}, {t(1)}, {self.sr('Colblocks')}")
        self.e(f"s_sub_u32 {t(0)}, {t(5)}, {t(0)}")
        self.e(f"s_cmp_gt_i32 {self.sr('Creal')}, 0")
        self.e(f"s_cselect_b32 {self.sr('Dkb')}, {self.sr('Kbf')}, {t(1)}")
        self.e(f"s_cselect_b32 {t(0)}, {t(5)}, {t(0)}")

    def filter_block(self, dst, T):
        t = self.t
        self.place(T)
        self.div(t(1), t(5), self.sr("Mcb"), self.sr("Scb"))
        self.e(f"s_cmp_gt_i32 {self.sr('Creal')}, 0")
        self.e(f"s_cselect_b32 {dst}, {self.sr('Kbf')}, {t(1)}")

    def flag_address(self, previous):
        """Fl = &flags[(M * 4 + wave) * 2 + 1], M = the workgroup that merges: this one, or (previous)
        the owner of the range in front of this one's: L - 1, or L - B in mode 0."""
        t = self.t
        fl = self.S["Fl"]
        if previous:
            self.e(f"s_cmp_gt_i32 {self.sr('Creal')}, 0")
            self.e(f"s_cselect_b32 {t(0)}, {self.sr('Colblocks')}, 1")
            self.e(f"s_sub_u32 {t(0)}, {self.sr('L')}, {t(0)}")
        else:
            self.e(f"s_mov_b32 {t(0)}, {self.sr('L')}")
        self.e(f"s_lshl_b32 {t(0)}, {t(0)}, 2")
        self.e(f"s_add_u32 {t(0)}, {t(0)}, {self.sr('Wave')}")
        self.e(f"s_lshl_b32 {t(0)}, {t(0)}, 3")
        self.e(f"s_add_u32 {t(0)}, {t(0)}, 4")
        self.e(f"s_add_u32 {s(fl)}, {s(self.S['Sync'])}, {t(0)}")
        self.e(f"s_addc_u32 {s(fl + 1)}, {s(self.S['Sync'] + 1)}, 0")

    # ------------------------------------------------------------------ per lane
    def lane_setup(self):
        t, e = self.t, self.e
        tmp = lambda i: self.vr("Tmp", i)
        e(f"v_lshrrev_b32 {tmp(0)}, 5, {self.vr('Lane')}")             # j: lane half
        e(f"v_and_b32 {tmp(1)}, 31, {self.vr('Lane')}")                # n
        e(f"v_lshlrev_b32 {tmp(1)}, 2, {tmp(1)}")                      # n*4
        e(f"v_mul_lo_u32 {tmp(2)}, {tmp(0)}, {self.sr('HWN4')}")       # j*HWN*4
        # patches: the lane owns channels 2j and 2j+1 of its wave's four-channel slab
        e(f"v_lshlrev_b32 {tmp(3)}, 1, {tmp(2)}")
        e(f"v_add_u32 {self.vr('LaneX')}, {tmp(3)}, {tmp(1)}")
        # stores: accumulator register r of lane (j, n) is filter row 8*(r/4) + 4j + r%4
        e(f"v_lshlrev_b32 {tmp(2)}, 2, {tmp(2)}")
        e(f"v_add_u32 {self.vr('Off', 0)}, {tmp(2)}, {tmp(1)}")
        e(f"v_add_u32 {self.vr('Off', 1)}, {self.sr('ColStep')}, {self.vr('Off', 0)}")
        e(f"v_add_u32 {self.vr('Off', 2)}, {self.sr('RowStep')}, {self.vr('Off', 0)}")
        e(f"v_add_u32 {self.vr('Off', 3)}, {self.sr('ColStep')}, {self.vr('Off', 2)}")
        # filters: one dwordx4 per position, 1 KB per position and wave
        e(f"v_lshlrev_b32 {self.vr('Lane16', 0)}, 4, {self.vr('Lane')}")
        for k in range(1, 4):
            e(f"v_add_u32 {self.vr('Lane16', k)}, 0x{4096 * k:x}, {self.vr('Lane16', 0)}")
        # LDS: V[buf][p][h][q''][n] dwords (16 KB per buffer).  Reads: lane (h, n) = lane*4 inside a
        # position's h-block... h*512 + n*4, dwords q'' = 0, 2 from Lds, q'' = 1, 3 from Lds2.
        e(f"v_lshlrev_b32 {tmp(2)}, 9, {tmp(0)}")                      # h*512
        e(f"v_add_u32 {tmp(2)}, {tmp(2)}, {tmp(1)}")
        e(f"v_add_u32 {self.vr('Lds')}, 0x4000, {tmp(2)}")
        e(f"v_add_u32 {self.vr('Lds2')}, 0x4080, {tmp(2)}")
        # writes: wave kw, lane half j own channel pair q = 2*(kw & 1) + j of half h = kw >> 1
        e(f"s_and_b32 {t(0)}, {self.sr('Kw')}, 1")
        e(f"s_lshl_b32 {t(0)}, {t(0)}, 7")                             # (kw & 1) * 128
        e(f"s_lshr_b32 {t(1)}, {self.sr('Kw')}, 1")
        e(f"s_lshl_b32 {t(1)}, {t(1)}, 9")                             # h * 512
        e(f"s_add_u32 {t(0)}, {t(0)}, {t(1)}")
        e(f"v_lshlrev_b32 {tmp(2)}, 8, {tmp(0)}")                      # 2j * 128
        e(f"v_add_u32 {tmp(2)}, {tmp(2)}, {tmp(1)}")
        e(f"v_add_u32 {self.vr('LdsWr')}, {t(0)}, {tmp(2)}")

    # ------------------------------------------------------------------ vector pieces
    def load_u(self, p, soff):
        return (f"buffer_load_dwordx4 {self.vr('U', 4 * p, 4)}, {self.vr('Lane16', p // 4)}, "
                f"{self.sr('RsrcU', 4)}, {soff} offen offset:{(p % 4) * 1024}")

    def load_patch(self, dst, i, second):
        soff = self.sr("HWN4") if second else "0"
        return f"buffer_load_dword {self.vr(dst, i)}, {self.vr('VOFF', i)}, {self.sr('RsrcX', 4)}, {soff} offen"

    def read_v(self, p):
        """The B operand of position p into its ring slot: q = 0, 1 and q = 2, 3."""
        r = self.V["VR"] + 4 * (p % RING)
        return [f"ds_read2st64_b32 {v(r, 2)}, {self.vr('Lds')} offset0:{4 * p} offset1:{4 * p + 1}",
                f"ds_read2st64_b32 {v(r + 2, 2)}, {self.vr('Lds2')} offset0:{4 * p} offset1:{4 * p + 1}"]

    def columns(self, src):
        d = lambda i: self.vr(src, i)
        t = lambda i: self.vr("T", i)
        out = []
        for c in range(4):
            out += [f"v_sub_f32 {t(c)}, {d(c)}, {d(8 + c)}",
                    f"v_add_f32 {t(4 + c)}, {d(4 + c)}, {d(8 + c)}",
                    f"v_sub_f32 {t(8 + c)}, {d(8 + c)}, {d(4 + c)}",
                    f"v_sub_f32 {t(12 + c)}, {d(4 + c)}, {d(12 + c)}"]
        return out

    def rows(self, dst):
        t = lambda i: self.vr("T", i)
        o = lambda i: self.vr(dst, i)
        out = []
        for r in range(4):
            out += [f"v_sub_f32 {o(4 * r)}, {t(4 * r)}, {t(4 * r + 2)}",
                    f"v_add_f32 {o(4 * r + 1)}, {t(4 * r + 1)}, {t(4 * r + 2)}",
                    f"v_sub_f32 {o(4 * r + 2)}, {t(4 * r + 2)}, {t(4 * r + 1)}",
                    f"v_sub_f32 {o(4 * r + 3)}, {t(4 * r + 1)}, {t(4 * r + 3)}"]
        return out

    def pack(self, p):
        op = "v_cvt_pk_bf16_f32" if self.bf16 else "v_cvt_pk_f16_f32"
        return f"{op} {self.vr('TA', p)}, {self.vr('TA', p)}, {self.vr('TB', p)}"

    def write_v(self, p):
        return (f"ds_write2st64_b32 {self.vr('LdsWr')}, {self.vr('TA', p)}, {self.vr('TA', p + 1)} "
                f"offset0:{4 * p} offset1:{4 * p + 4}")

    def end_of_chunk(self):
        self.e("s_waitcnt lgkmcnt(0)")
        self.e("s_barrier")
        for n in ("Lds", "Lds2", "LdsWr"):
            self.e(f"v_xor_b32 {self.vr(n)}, 0x4000, {self.vr(n)}")

    # ------------------------------------------------------------------ one chunk
    def chunk(self, first, par):
        """MFMA work of unit G (16 channels, G & 1 == par): 16 slots, one per position.  Slot p:
        MFMA p, then the reload of its filter registers with unit G+1 and the LDS read of the B
        operand LEAD positions ahead; the first ten slots also carry the input transform of unit
        G+1 in steps of eight VALU instructions (they co-issue with the fp16 MFMAs), each column
        step followed by the reload of the four patch registers it consumed with unit G+3.
        The patches live in two register sets, unit X in set X & 1, so a patch load has two
        units to arrive (they come from beyond L2) while a filter load has one.

        `first` (a unit that follows an output transform's 64 stores, a merge or the prologue):
        every load it waits for is at least 64 memory instructions old, so all counts saturate."""
        ops = []  # str | ("vmem", text, tag) | ("lds", text, tag or None) | Wait
        da, db = f"DA{par ^ 1}", f"DB{par ^ 1}"
        self.comment(f"---- chunk, G & 1 == {par} ({'first of a segment (' + str(first) + ')' if first else 'steady state'})")
        self.advance_p(3)
        self.advance_q()
        self.slab_descriptor(0)
        self.u_offset(self.sr("UoffQ"), self.sr("KgQ"), self.sr("Cq"), False)

        def reads(p):
            r = self.read_v(p)
            ops.append(("lds", r[0], None))
            ops.append(("lds", r[1], ("V", p)))

        def patch_loads(dst, second, idx):
            for i in idx:
                ops.append(("vmem", self.load_patch(dst, i, second), (dst, i)))

        # the input transform of unit G+1 as a list of steps; a step = (wait, VALU ops, patch reloads)
        def column_steps(src, second):
            cols = self.columns(src)
            out = []
            for c in range(4):
                idx = [c, 4 + c, 8 + c, 12 + c]  # the patch registers column c consumes, then reloads
                out.append((Wait("vm", (src, 12 + c)), cols[4 * c:4 * c + 4], (src, second, idx)))
            return out

        rows_a, rows_b = self.rows("TA"), self.rows("TB")
        steps = (column_steps(da, False) +
                 [(None, rows_a[0:8], None), (None, rows_a[8:16], None)] +
                 column_steps(db, True) +
                 [(None, rows_b[0:8], None), (None, rows_b[8:16], None)] +
                 [(None, [self.pack(q) for q in range(0, 8)], None),
                  (None, [self.pack(q) for q in range(8, 16)], "writes0"),
                  (None, [], "writes1")])

        def run(step):
            wait, valu, tail = step
            if wait:
                ops.append(wait)
            ops.extend(valu)
            if tail == "writes0":
                for q in range(0, 8, 2):
                    ops.append(("lds", self.write_v(q), None))
            elif tail == "writes1":
                for q in range(8, 16, 2):
                    ops.append(("lds", self.write_v(q), None))
            elif tail:
                patch_loads(*tail)

        for p in range(LEAD):
            reads(p)
        # two column steps in front of the first MFMA: they do not depend on the LDS reads
        run(steps[0])
        run(steps[1])
        # slot p >= 0 takes the steps sched[p]
        sched = {0: [2, 3], 1: [4], 2: [5], 3: [6, 7], 4: [8, 9], 5: [10], 6: [11], 7: [12], 8: [13], 9: [14]}
        mfma = "v_mfma_f32_32x32x16_bf16" if self.bf16 else "v_mfma_f32_32x32x16_f16"
        for p in range(16):
            ops.append(Wait("vm", ("U", p)))
            ops.append(Wait("lgkm", ("V", p)))
            fresh = first and not (first == "merge" and p in MERGE_POSITIONS)
            c = "0" if fresh else a(16 * p, 16)
            ops.append(f"{mfma} {a(16 * p, 16)}, {self.vr('U', 4 * p, 4)}, "
                       f"{v(self.V['VR'] + 4 * (p % RING), 4)}, {c}")
            ops.append(("vmem", self.load_u(p, self.sr("UoffQ")), ("U", p)))
            if p + LEAD < 16:
                reads(p + LEAD)
            for k in sched.get(p, []):
                run(steps[k])
        self.resolve(ops, first)
        self.end_of_chunk()
        self.e(f"s_add_u32 {self.sr('G')}, {self.sr('G')}, 1")
        self.e(f"s_add_u32 {self.sr('Cm')}, {self.sr('Cm')}, 1")
        self.e(f"s_cmp_eq_u32 {self.sr('Cm')}, {self.sr('Chunks')}")
        self.e(f"s_cselect_b32 {self.sr('Cm')}, 0, {self.sr('Cm')}")

    # Diagnostic builds (wrong results; make diagnostic): what is left of a unit.
    #   "all"         the kernel
    #   "loads_only"  the filter and patch loads with their waits: no MFMA, no transform, no LDS traffic
    #   "no_units"    neither: scalar code, barrier, prologue, output transforms and hand-overs remain
    KEEP = "all"

    def kept(self, ops):
        if self.KEEP == "all":
            return ops
        work = ("v_mfma", "v_sub_f32", "v_add_f32", "v_cvt_pk")
        out = []
        for op in ops:
            if isinstance(op, str):
                drop = op.split()[0].startswith(work)
            elif isinstance(op, tuple):
                drop = op[0] == "lds" or self.KEEP == "no_units"
            else:
                drop = op.counter == "lgkm" or self.KEEP == "no_units"
            if not drop:
                out.append(op)
        return out

    def resolve(self, ops, first):
        """Emit the chunk with its s_waitcnt counts.  vmcnt: memory instructions issued after the
        awaited load, which sits behind its consumer in an earlier pass of the same sequence
        (cyclic count, saturated at the counter's 63: the wave then also waits for some younger
        loads).  lgkmcnt: LDS instructions issued after the awaited read, inside this chunk."""
        ops = self.kept(ops)
        vm_pos = {op[2]: i for i, op in enumerate(ops) if isinstance(op, tuple) and op[0] == "vmem"}
        n_vm = sum(1 for op in ops if isinstance(op, tuple) and op[0] == "vmem")
        lds_pos = {op[2]: i for i, op in enumerate(ops) if isinstance(op, tuple) and op[0] == "lds" and op[2]}
        for i, op in enumerate(ops):
            if isinstance(op, str):
                self.e(op)
            elif isinstance(op, tuple):
                self.e(op[1])
            elif op.counter == "vm":
                j = vm_pos[op.tag]
                assert j > i, f"{op.tag} is awaited behind its reload"
                after = sum(1 for o in ops[j + 1:] if isinstance(o, tuple) and o[0] == "vmem")
                before = sum(1 for o in ops[:i] if isinstance(o, tuple) and o[0] == "vmem")
                assert after + before < n_vm or self.KEEP != "all"
                # a filter load was issued by the previous chunk, a patch load by the one before
                # that (same sequence of memory instructions in every chunk)
                count = after + before + (0 if op.tag[0] == "U" else n_vm)
                count = 63 if first else min(63, count)
                self.e(f"s_waitcnt vmcnt({count})")
            else:
                j = lds_pos[op.tag]
                assert j < i, f"{op.tag} is read behind its consumer"
                count = sum(1 for o in ops[j + 1:i] if isinstance(o, tuple) and o[0] == "lds")
                self.e(f"s_waitcnt lgkmcnt({min(15, count)})")

    # ------------------------------------------------------------------ prologue
    def prologue(self):
        """Unit 0 -> LDS buffer 0, with the filters of unit 0 and the patches of units 1 and 2 in
        flight; unit 0's patches land in the transform temporaries."""
        e = self.e
        self.decode(self.sr("Tm"))
        self.m_tile_setup()
        e(f"s_mov_b32 {self.sr('KgQ')}, {self.sr('KgM')}")
        self.filter_descriptor(self.sr("KgQ"))
        self.patch_offsets()
        self.u_offset(self.sr("UoffQ"), self.sr("KgM"), self.sr("Cm"), False)
        self.slab_descriptor(0)
        for i in range(16):
            e(self.load_patch("TA", i, False))
            e(self.load_patch("TB", i, True))
        for p in range(16):
            e(self.load_u(p, self.sr("UoffQ")))
        for unit in (1, 2):  # unit X -> set X & 1
            e(f"s_mov_b32 {self.sr('G')}, {unit - 3}")
            self.advance_p(3)
            self.slab_descriptor(0)
            for i in range(16):
                e(self.load_patch(f"DA{unit & 1}", i, False))
            for i in range(16):
                e(self.load_patch(f"DB{unit & 1}", i, True))
        e(f"s_mov_b32 {self.sr('G')}, 0")
        e("s_waitcnt vmcnt(63)")  # 112 loads issued, unit 0's patches are the oldest 32
        for src in ("TA", "TB"):
            for line in self.columns(src) + self.rows(src):
                e(line)
        for p in range(16):
            e(self.pack(p))
        for p in range(0, 16, 2):
            e(self.write_v(p))
        self.end_of_chunk()
        e("s_waitcnt vmcnt(0)")  # the first chunk counts on a queue without surprises

    # ------------------------------------------------------------------ segments
    def segments(self):
        """The segment loop of the fp32 kernels with every chunk in two versions, for even and odd
        G (the patch register set a chunk transforms and reloads)."""
        t, e = self.t, self.e
        seg_loop, done, plain_seg, after_epi, epi = (self.newlabel(x) for x in
                                                     ("seg", "done", "plainseg", "afterepi", "epi"))
        check = [self.newlabel("check0"), self.newlabel("check1")]
        late_seg, late, late_pub, flag = (self.newlabel(x) for x in ("lateseg", "late", "latepub", "flag"))
        self.stamp()
        self.label(seg_loop)
        e(f"s_bitcmp1_b32 {self.sr('Sch')}, 6")
        e(f"s_cbranch_scc1 {late_seg}")
        # this segment: the units of tile Tm that belong to this workgroup; SegEnd in units of G.
        # Kind: 1 publish (the range starts inside the tile), 2 merge (it ends inside), 0 whole tile.
        e(f"s_cmp_eq_u32 {self.sr('G')}, 0")
        e(f"s_cselect_b32 {t(0)}, {self.sr('N1')}, {self.sr('Chunks')}")
        e(f"s_cmp_lt_u32 {t(0)}, {self.sr('Chunks')}")
        e(f"s_cselect_b32 {self.sr('Kind')}, 1, 0")
        e(f"s_cmp_eq_u32 {self.sr('G')}, 0")   # a range's first tile is never its last partial one
        e(f"s_cselect_b32 {t(1)}, -1, {self.sr('Tlast')}")
        e(f"s_cmp_eq_u32 {self.sr('Tm')}, {t(1)}")
        e(f"s_cselect_b32 {t(0)}, {self.sr('Nlast')}, {t(0)}")
        e(f"s_sub_u32 {t(1)}, {self.sr('Nunits')}, {self.sr('G')}")
        e(f"s_min_u32 {t(0)}, {t(0)}, {t(1)}")
        e(f"s_add_u32 {self.sr('SegEnd')}, {self.sr('G')}, {t(0)}")
        e(f"s_cmp_lt_u32 {t(0)}, {self.sr('Chunks')}")
        e(f"s_cselect_b32 {t(1)}, 1, 0")
        e(f"s_cmp_eq_u32 {self.sr('Kind')}, 1")
        e(f"s_cselect_b32 {t(1)}, 0, {t(1)}")   # short and not the publishing one: the merging one
        e(f"s_cmp_eq_u32 {t(1)}, 0")
        e(f"s_cbranch_scc1 {plain_seg}")
        e(f"s_mov_b32 {self.sr('Kind')}, 2")
        self.merge_init()
        for kind, entry in (("merge", None), (True, plain_seg)):
            if entry:
                self.label(entry)
            odd = self.newlabel("odd")
            e(f"s_bitcmp1_b32 {self.sr('G')}, 0")
            e(f"s_cbranch_scc1 {odd}")
            self.chunk(kind, 0)
            e(f"s_branch {check[1]}")
            self.label(odd)
            self.chunk(kind, 1)
            e(f"s_branch {check[0]}")
        # steady state: even chunk, odd chunk, ...
        self.label(check[0])
        e(f"s_cmp_lt_u32 {self.sr('G')}, {self.sr('SegEnd')}")
        e(f"s_cbranch_scc0 {epi}")
        self.chunk(False, 0)
        self.label(check[1])
        e(f"s_cmp_lt_u32 {self.sr('G')}, {self.sr('SegEnd')}")
        e(f"s_cbranch_scc0 {epi}")
        self.chunk(False, 1)
        e(f"s_branch {check[0]}")
        self.label(epi)
        self.stamp()
        pub = self.newlabel("publish")
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
        e(f"s_sub_u32 {t(0)}, {self.sr('Chunks')}, {self.sr('Nlast')}")
        e(f"s_cmp_eq_u32 {self.sr('Tm')}, {self.sr('Tlast')}")
        e(f"s_cselect_b32 {self.sr('Cm')}, {t(0)}, {self.sr('Cm')}")  # else it is at Sfull already
        self.decode(self.sr("Tm"))
        self.m_tile_setup()
        e(f"s_branch {seg_loop}")
        self.label(done)
        e("s_endpgm")
        # A segment of a range in the natural chunk order (a layer with fewer tiles than compute
        # units, Kernel.late_merge): chunks Cm .. of tile Tm, up to the tile's or the range's end.
        # Kind 1: it starts inside the tile and reaches its end: it publishes; 4: it starts with
        # the tile and ends inside: it merges and stores the tile; 5: both; 0: a whole tile.
        self.label(late_seg)
        e(f"s_sub_u32 {t(0)}, {self.sr('Chunks')}, {self.sr('Cm')}")
        e(f"s_sub_u32 {t(1)}, {self.sr('Nunits')}, {self.sr('G')}")
        e(f"s_min_u32 {t(0)}, {t(0)}, {t(1)}")
        e(f"s_add_u32 {self.sr('SegEnd')}, {self.sr('G')}, {t(0)}")
        e(f"s_cmp_lg_u32 {self.sr('Cm')}, 0")
        e(f"s_cselect_b32 {self.sr('Kind')}, 1, 0")
        e(f"s_add_u32 {t(1)}, {self.sr('Cm')}, {t(0)}")
        e(f"s_or_b32 {t(0)}, {self.sr('Kind')}, 4")
        e(f"s_cmp_lt_u32 {t(1)}, {self.sr('Chunks')}")
        e(f"s_cselect_b32 {self.sr('Kind')}, {t(0)}, {self.sr('Kind')}")
        e(f"s_branch {plain_seg}")
        self.label(late)
        e(f"s_cmp_eq_u32 {self.sr('Kind')}, 5")
        e(f"s_cbranch_scc1 {late_pub}")
        self.epilogue(False, merge=True)
        e(f"s_branch {after_epi}")
        self.label(late_pub)
        self.epilogue(True, merge=True)
        e(f"s_branch {flag}")
        self.lines.extend(self.outofline)


def main():
    if len(sys.argv) == 3 and sys.argv[1] == "--keep" and sys.argv[2] in ("all", "loads_only", "no_units"):
        KernelH16.KEEP = sys.argv[2]
    elif len(sys.argv) > 1:
        sys.exit("usage: gen_wino_h16_asm.py [--keep all|loads_only|no_units]")
    out = ['\t.amdgcn_target "amdgcn-amd-amdhsa--gfx950"', "\t.amdhsa_code_object_version 6"]
    kernels = [KernelH16(bf16, ragged, packed) for ragged, packed in ((False, False), (True, False), (True, True))
               for bf16 in (False, True)]
    for k in kernels:
        k.emit(out)
    out.append("\t.amdgpu_metadata\n---\namdhsa.kernels:")
    out.extend(k.metadata() for k in kernels)
    out.append("amdhsa.target:   amdgcn-amd-amdhsa--gfx950\namdhsa.version:\n  - 1\n  - 2\n...\n\t.end_amdgpu_metadata")
    sys.stdout.write("\n".join(out) + "\n")


if __name__ == "__main__":
    main()
