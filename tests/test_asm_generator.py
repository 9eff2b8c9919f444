"""CPU checks of the assembly generator (opencnn_amd/csrc/gen_wino_f32_asm.py): it runs, stays
inside the register file, keeps the invariants its wait counts rely on, and its output assembles
for gfx950 (no GPU needed: the assembler cross-compiles)."""
import importlib.util
import os
import re
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
GEN = os.path.join(ROOT, "opencnn_amd", "csrc", "gen_wino_f32_asm.py")
CLANG = "/opt/rocm/lib/llvm/bin/clang"


@pytest.fixture(scope="module")
def gen():
    spec = importlib.util.spec_from_file_location("gen_wino_f32_asm", GEN)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


VARIANTS = [(False, False), (True, False), (True, True)]  # (ragged, packed)


@pytest.mark.parametrize("ragged,packed", VARIANTS)
@pytest.mark.parametrize("kw", [2, 4])
def test_register_budget(gen, kw, ragged, packed):
    k = gen.Kernel(kw, ragged, packed)
    assert k.vgpr_count <= 256          # arch VGPRs; the 256 accumulators are AGPRs
    assert k.sgpr_count <= 100          # s0 .. s101 less VCC, which the kernel descriptor reserves (the assembler checks too)
    assert len(set(k.MP)) == 64         # landing registers of a published partial tile
    live_at_boundary = set()
    for name in ("U0", "U1", "D0", "D1", "VA", "VOFF", "Off", "Eff"):
        if name in k.V:
            n = {"U0": 32, "U1": 32, "D0": 16, "D1": 16, "VA": 16, "VOFF": 16, "Off": 4, "Eff": 4}[name]
            live_at_boundary |= set(range(k.V[name], k.V[name] + n))
    assert not live_at_boundary & set(k.MP), "partial tile would land on live pipeline registers"


@pytest.mark.parametrize("ragged,packed", VARIANTS)
@pytest.mark.parametrize("kw", [2, 4])
def test_kernel_text_invariants(gen, kw, ragged, packed):
    k = gen.Kernel(kw, ragged, packed)
    k.body()
    text = "\n".join(k.lines)
    assert k.name.endswith("_packed" if packed else "_ragged" if ragged else f"kw{kw}")
    # per-lane tiles (a 64-bit shift for the division by the tiles per row) only when packed
    assert ("v_lshrrev_b64" in text) == packed
    # one workgroup barrier per chunk variant + the prologue; three chunk variants
    assert text.count("s_barrier") == 4
    # 64 MFMAs per chunk variant, plus the second copy of step 0 (MFMAs 1..15) that carries the
    # tile switch of the patch cursor
    assert len(re.findall(r"v_mfma_f32_32x32x2_f32", text)) == 3 * (64 + 15)
    # first step of a tile: 16 MFMAs from the constant 0 (15 in the second copy); a merging segment
    # keeps four accumulators (three of them among MFMAs 1..15)
    assert len(re.findall(r"v_mfma_f32_32x32x2_f32 [^\n]*, 0$", text, re.M)) == (16 + 15) + (12 + 12)
    # the counted waits rely on exactly 64 stores per epilogue (four epilogues: plain, publishing,
    # and both again with the partial tile of the next workgroup added, for ranges inside a tile)
    assert len(re.findall(r"buffer_store_dword", text)) == 4 * 64
    assert len(re.findall(r"buffer_store_dword [^\n]* sc0 sc1", text)) == 2 * 64
    # partial tiles are read past the caches: merge_init and the two late merges, 64 loads each
    assert len(re.findall(r"buffer_load_dword v\d+, [^\n]* sc0 sc1", text)) == 3 * 64
    # s_waitcnt fields: vmcnt has 6 bits, lgkmcnt 4
    assert all(int(n) <= 63 for n in re.findall(r"vmcnt\((\d+)\)", text))
    assert all(int(n) <= 15 for n in re.findall(r"lgkmcnt\((\d+)\)", text))
    # every label that is branched to exists exactly once
    labels = re.findall(r"^(\.L\w+):", text, re.M)
    assert len(labels) == len(set(labels))
    for target in re.findall(r"s_c?branch\w* (\.L\w+)", text):
        assert target in labels


def check_bounded_waits(k, text):
    """Every wait for a flag (merge in front of a segment, two merges inside an output transform)
    is bounded by the poll limit of the argument block, and the wave that gives up stores to the
    status word before it goes on: no silent wrong tile, no endless loop."""
    polls = re.findall(r"^(\.L\w+_poll_\d+):", text, re.M)
    assert len(polls) == 3
    limit, status = f"s{k.S['SpinLimit']}", f"s[{k.S['Status']}:{k.S['Status'] + 1}]"
    assert f"s_load_dwordx2 {status}, s[0:1], 0x88" in text
    assert f"s_load_dword {limit}, s[0:1], 0x90" in text
    assert "0x100000" not in text  # no compiled-in limit left
    lines = text.splitlines()
    for poll in polls:
        i = lines.index(poll + ":")
        loop = lines[i:i + 14]
        back = [j for j, l in enumerate(loop) if l.strip() == f"s_branch {poll}"]
        assert back, "poll loop without its backward branch"
        loop = loop[:back[0] + 1]
        # the only ways out: the flag is there, or the limit is reached
        exits = [l.split()[-1] for l in loop if "s_cbranch" in l]
        assert len(exits) == 2
        got, giveup = exits
        assert "_got_" in got and "_giveup_" in giveup
        cmp_limit = [j for j, l in enumerate(loop) if l.strip().startswith("s_cmp_lt_u32") and l.strip().endswith(limit)]
        assert cmp_limit and "s_cbranch_scc0 " + giveup in loop[cmp_limit[0] + 1]
        j = lines.index(giveup + ":")
        block = [l.strip() for l in lines[j + 1:j + 5]]
        assert block[0] == "s_mov_b64 exec, 1"
        assert re.fullmatch(r"global_store_dword v\d+, v\d+, " + re.escape(status) + " sc0 sc1", block[1])
        assert block[1].split()[2].rstrip(",") == f"v{k.V['One']}"
        assert block[2] == "s_mov_b64 exec, -1" and block[3] == f"s_branch {got}"
    # the status word's registers are written by the argument load only
    for reg in (k.S["Status"], k.S["Status"] + 1, k.S["SpinLimit"]):
        writers = re.findall(rf"^\s*([sv]_\w+) s{reg}\b", text, re.M)
        assert writers in (["s_load_dword"], []), writers


@pytest.mark.parametrize("ragged,packed", VARIANTS)
@pytest.mark.parametrize("kw", [2, 4])
def test_flag_waits_are_bounded_and_report(gen, kw, ragged, packed):
    k = gen.Kernel(kw, ragged, packed)
    k.body()
    check_bounded_waits(k, "\n".join(k.lines))


@pytest.mark.skipif(not os.path.exists(CLANG), reason="ROCm LLVM assembler not installed")
def test_output_assembles_for_gfx950(tmp_path):
    src = tmp_path / "k.s"
    with open(src, "w") as f:
        subprocess.run(["python3", GEN], check=True, stdout=f)
    obj = tmp_path / "k.o"
    subprocess.run([CLANG, "-x", "assembler", "-target", "amdgcn-amd-amdhsa", "-mcpu=gfx950",
                    "-c", str(src), "-o", str(obj)], check=True)
    assert obj.stat().st_size > 10000
    lld = shutil.which("ld.lld") or "/opt/rocm/lib/llvm/bin/ld.lld"
    subprocess.run([lld, "-shared", str(obj), "-o", str(tmp_path / "k.hsaco")], check=True)


# ---------------------------------------------------------------- fp16 / bf16 kernels
GEN_H16 = os.path.join(ROOT, "opencnn_amd", "csrc", "gen_wino_h16_asm.py")


@pytest.fixture(scope="module")
def gen_h16(gen):
    import sys
    sys.modules.setdefault("gen_wino_f32_asm", gen)  # the fp16 / bf16 generator extends its Kernel class
    spec = importlib.util.spec_from_file_location("gen_wino_h16_asm", GEN_H16)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


@pytest.mark.parametrize("ragged,packed", VARIANTS)
@pytest.mark.parametrize("bf16", [False, True])
def test_h16_register_budget(gen_h16, bf16, ragged, packed):
    k = gen_h16.KernelH16(bf16, ragged, packed)
    assert k.vgpr_count <= 256
    assert k.sgpr_count <= 100
    assert len(set(k.MP)) == 64
    live_at_boundary = set()
    for name, n in (("U", 64), ("DA0", 16), ("DB0", 16), ("DA1", 16), ("DB1", 16), ("VOFF", 16),
                    ("Off", 4), ("Eff", 4), ("Lane16", 4)):
        live_at_boundary |= set(range(k.V[name], k.V[name] + n))
    assert not live_at_boundary & set(k.MP), "partial tile would land on live pipeline registers"
    # MFMA operand tuples start on even registers
    assert k.V["U"] % 2 == 0 and k.V["VR"] % 2 == 0


@pytest.mark.parametrize("ragged,packed", VARIANTS)
@pytest.mark.parametrize("bf16", [False, True])
def test_h16_kernel_text_invariants(gen_h16, bf16, ragged, packed):
    k = gen_h16.KernelH16(bf16, ragged, packed)
    k.body()
    text = "\n".join(k.lines)
    assert k.name.endswith("_packed" if packed else "_ragged" if ragged else "kw4")
    assert ("v_lshrrev_b64" in text) == packed
    # lane masks (batch elements that do not exist) only in the _ragged kernels
    assert ("v_cndmask_b32" in text) == ragged
    op = "v_mfma_f32_32x32x16_bf16" if bf16 else "v_mfma_f32_32x32x16_f16"
    other = "v_mfma_f32_32x32x16_f16" if bf16 else "v_mfma_f32_32x32x16_bf16"
    # six chunk bodies (plain first / merging first / steady state, each for even and odd units)
    assert text.count(op) == 6 * 16 and other not in text
    assert text.count("s_barrier") == 6 + 1
    # first chunk of a tile: 16 MFMAs from the constant 0; a merging segment keeps four accumulators
    assert len(re.findall(op + r" [^\n]*, 0$", text, re.M)) == 2 * 16 + 2 * 12
    cvt = "v_cvt_pk_bf16_f32" if bf16 else "v_cvt_pk_f16_f32"
    assert text.count(cvt) == 7 * 16
    # per chunk body: 16 filter loads, 32 patch loads; prologue: 16 + 3 * 32
    assert text.count("buffer_load_dwordx4") == 7 * 16
    # + 64 loads each for the merge in front of a segment and the two merges in an output transform
    assert len(re.findall(r"buffer_load_dword v", text)) == 6 * 32 + 3 * 32 + 3 * 64
    assert len(re.findall(r"buffer_store_dword", text)) == 4 * 64
    assert all(int(n) <= 63 for n in re.findall(r"vmcnt\((\d+)\)", text))
    assert all(int(n) <= 15 for n in re.findall(r"lgkmcnt\((\d+)\)", text))
    labels = re.findall(r"^(\.L\w+):", text, re.M)
    assert len(labels) == len(set(labels))
    for target in re.findall(r"s_c?branch\w* (\.L\w+)", text):
        assert target in labels
    # LDS: two 16 KB buffers; every access stays below 32 KB for the largest lane offsets
    assert max(int(n) for n in re.findall(r"offset1:(\d+)", text)) * 256 + 0x4000 + 0x80 + 636 < 32768


@pytest.mark.parametrize("ragged,packed", VARIANTS)
@pytest.mark.parametrize("bf16", [False, True])
def test_h16_flag_waits_are_bounded_and_report(gen_h16, bf16, ragged, packed):
    k = gen_h16.KernelH16(bf16, ragged, packed)
    k.body()
    check_bounded_waits(k, "\n".join(k.lines))


@pytest.mark.parametrize("keep", ["loads_only", "no_units"])
def test_h16_diagnostic_builds_drop_what_they_say(gen_h16, keep, monkeypatch):
    """gen_wino_h16_asm.py --keep (make diagnostic): timing-only kernels with the work of a unit taken
    out.  The chunks lose their MFMAs, transform and LDS traffic (and, for no_units, their loads);
    prologue, output transforms and hand-overs stay as they are."""
    full = gen_h16.KernelH16(False)
    full.body()
    full_text = "\n".join(full.lines)
    monkeypatch.setattr(gen_h16.KernelH16, "KEEP", keep)
    k = gen_h16.KernelH16(False)
    k.body()
    text = "\n".join(k.lines)
    assert "v_mfma" not in text
    assert text.count("s_barrier") == full_text.count("s_barrier")
    assert text.count("buffer_store_dword") == full_text.count("buffer_store_dword")
    # the prologue's filter loads and LDS writes remain; the six chunk bodies' 16 + 32 loads only in loads_only
    chunk_loads = 6 * 16 if keep == "loads_only" else 0
    assert text.count("buffer_load_dwordx4") == 16 + chunk_loads
    assert text.count("ds_read2st64_b32") == 0
    assert text.count("ds_write2st64_b32") == 8
    assert all(int(n) <= 63 for n in re.findall(r"vmcnt\((\d+)\)", text))


@pytest.mark.skipif(not os.path.exists(CLANG), reason="ROCm LLVM assembler not installed")
def test_h16_output_assembles_for_gfx950(tmp_path):
    src = tmp_path / "k.s"
    with open(src, "w") as f:
        subprocess.run(["python3", GEN_H16], check=True, stdout=f)
    obj = tmp_path / "k.o"
    subprocess.run([CLANG, "-x", "assembler", "-target", "amdgcn-amd-amdhsa", "-mcpu=gfx950",
                    "-c", str(src), "-o", str(obj)], check=True)
    assert obj.stat().st_size > 10000


# ---------------------------------------------------------------- the tile order, executed on the CPU
class ScalarMachine:
    """Interpreter of the few scalar instructions the generators use for index arithmetic: runs the
    text a generator emitted, so the tests below check the emitted code, not a restatement."""

    def __init__(self):
        self.s, self.scc = {}, 0

    def val(self, x):
        if x.startswith("s"):
            return self.s.get(int(x[1:]), 0)
        return int(x, 0) & 0xFFFFFFFF

    def run(self, lines):
        for line in lines:
            line = line.strip()
            if not line or line.startswith(";"):
                continue
            op, rest = line.split(None, 1)
            a = [x.strip() for x in rest.split(",")]
            m = 0xFFFFFFFF
            if op == "s_mov_b32":
                self.s[int(a[0][1:])] = self.val(a[1])
            elif op in ("s_add_u32", "s_add_i32", "s_sub_u32", "s_sub_i32"):
                x, y = self.val(a[1]), self.val(a[2])
                r = x + y if "add" in op else x - y
                self.scc = int(r > m or r < 0)
                self.s[int(a[0][1:])] = r & m
            elif op == "s_addc_u32":
                r = self.val(a[1]) + self.val(a[2]) + self.scc
                self.scc = int(r > m)
                self.s[int(a[0][1:])] = r & m
            elif op == "s_min_u32":
                x, y = self.val(a[1]), self.val(a[2])
                self.scc = int(x < y)
                self.s[int(a[0][1:])] = min(x, y)
            elif op == "s_mul_i32":
                self.s[int(a[0][1:])] = (self.val(a[1]) * self.val(a[2])) & m
            elif op == "s_mul_hi_u32":
                self.s[int(a[0][1:])] = (self.val(a[1]) * self.val(a[2])) >> 32
            elif op in ("s_lshl_b32", "s_lshr_b32"):
                x, n = self.val(a[1]), self.val(a[2]) & 31
                r = (x << n) & m if op == "s_lshl_b32" else x >> n
                self.s[int(a[0][1:])], self.scc = r, int(r != 0)
            elif op == "s_lshr_b64":
                lo = int(re.match(r"s\[(\d+):", a[0]).group(1))
                src = int(re.match(r"s\[(\d+):", a[1]).group(1))
                v = (self.s.get(src, 0) | (self.s.get(src + 1, 0) << 32)) >> (self.val(a[2]) & 63)
                self.s[lo], self.s[lo + 1], self.scc = v & m, v >> 32, int(v != 0)
            elif op in ("s_and_b32", "s_or_b32"):
                x, y = self.val(a[1]), (int(a[2]) & m if re.fullmatch(r"-\d+", a[2]) else self.val(a[2]))
                r = x & y if op == "s_and_b32" else x | y
                self.s[int(a[0][1:])], self.scc = r, int(r != 0)
            elif op in ("s_cmp_lt_u32", "s_cmp_gt_u32", "s_cmp_eq_u32", "s_cmp_lg_u32", "s_cmp_gt_i32"):
                x, y = self.val(a[0]), self.val(a[1])
                if op.endswith("i32"):
                    x, y = (x ^ 0x80000000) - 0x80000000, (y ^ 0x80000000) - 0x80000000
                self.scc = int({"lt": x < y, "gt": x > y, "eq": x == y, "lg": x != y}[op.split("_")[2]])
            elif op == "s_cselect_b32":
                self.s[int(a[0][1:])] = self.val(a[1]) if self.scc else self.val(a[2])
            elif op == "s_bitcmp1_b32":
                self.scc = (self.val(a[0]) >> (self.val(a[1]) & 31)) & 1
            else:
                raise AssertionError(f"the test's interpreter does not know {op}")


def magic(d):
    l = 0
    while (1 << l) < d:
        l += 1
    return ((1 << (31 + l)) + d - 1) // d, 31 + l


def decoded_tiles(k, H, W, ngroups, order_bits):
    """(image group, tile row, tile column, live) of every column tile, as the kernel's decode()
    computes them (one filter block, KW waves on one column tile)."""
    th, tw = (H + 1) // 2, (W + 1) // 2
    colgroups = th * tw * ngroups
    k.lines = []
    k.decode(f"s{k.S['Tp']}")
    code = [l for l in k.lines]
    assert not any(re.match(r"^\S+:$", l) or "s_cbranch" in l or "s_branch" in l for l in code), \
        "decode() is dealt out over the gaps between MFMAs: it must not branch"
    out = []
    for t in range(colgroups // k.CW):
        for cw in range(k.CW):
            m = ScalarMachine()
            S = k.S
            m.s.update({S["H"]: H, S["W"]: W, S["TilesW"]: tw, S["Colgroups"]: colgroups, S["Cw"]: cw,
                        S["Colblocks"]: colgroups // k.CW, S["Tp"]: t})
            m.s[S["Mcb"]], m.s[S["Scb"]] = magic(colgroups // k.CW)
            div = th * tw if order_bits & 1 else ngroups
            m.s[S["Ngroups"]] = div
            m.s[S["Mng"]], m.s[S["Sng"]] = magic(div)
            m.s[S["Sng"]] |= 64 if order_bits & 1 else 0
            m.s[S["Mtw"]], m.s[S["Stw"]] = magic(tw)
            m.s[S["Stw"]] |= 64 if order_bits & 2 else 0
            m.run(code)
            out.append((m.s[S["Dng"]], m.s[S["Dty"]], m.s[S["Dtx"]], m.s[S["Dlive"]], m.s[S["Dkb"]]))
    return out


@pytest.mark.parametrize("order_bits", [0, 1, 2, 3])
@pytest.mark.parametrize("kw,H,W,ngroups", [(4, 14, 14, 4), (2, 7, 9, 2), (4, 13, 6, 3), (2, 2, 2, 2), (4, 1, 5, 1),
                                            (2, 56, 56, 2)])
def test_every_tile_order_visits_every_tile_once(gen, kw, H, W, ngroups, order_bits):
    k = gen.Kernel(kw)
    tiles = decoded_tiles(k, H, W, ngroups, order_bits)
    th, tw = (H + 1) // 2, (W + 1) // 2
    assert all(live == 1 and kb == 0 for (_, _, _, live, kb) in tiles)
    seen = {(ng, ty, tx) for (ng, ty, tx, _, _) in tiles}
    assert len(seen) == len(tiles) == th * tw * ngroups
    assert all(ng < ngroups and ty < th and tx < tw for (ng, ty, tx) in seen)
    if order_bits & 1 and ngroups * th * tw > 1:
        # neighbours on the line are neighbours in the image (or the next strip / image group begins)
        far = sum(1 for a, b in zip(tiles, tiles[1:]) if abs(a[1] - b[1]) + abs(a[2] - b[2]) > (2 if order_bits & 2 else 1))
        assert far <= (th + 1) * ngroups


@pytest.mark.parametrize("tiles,ranges", [(196, 128), (196, 8), (392, 256), (49, 48), (784, 256), (3000, 1024),
                                          (8, 8), (1000, 8), (65, 64), (12345, 256), (130, 128)])
@pytest.mark.parametrize("family", ["f32_kw2", "f32_kw4", "f16"])
def test_places_of_a_line_are_a_permutation_of_each_window(gen, gen_h16, family, tiles, ranges):
    k = {"f32_kw2": lambda: gen.Kernel(2), "f32_kw4": lambda: gen.Kernel(4), "f16": lambda: gen_h16.KernelH16(False)}[family]()
    k.lines = []
    src = f"s{k.S['Tm']}"
    k.place(src)
    code = list(k.lines)
    assert not any("branch" in l for l in code)
    t5 = k.S["T"] + 5
    mg, sh = magic(tiles)
    placed = []
    for on in (False, True):
        placed = []
        for t in range(tiles):
            m = ScalarMachine()
            m.s.update({k.S["Tm"]: t, k.S["PlaceM"]: mg, k.S["PlaceS"]: sh | (64 if on else 0),
                        k.S["PlaceG"]: ranges, k.S["PlaceTn"]: tiles})
            m.run(code)
            placed.append(m.s[t5])
        if not on:
            assert placed == list(range(tiles))
    assert sorted(placed) == list(range(tiles))
    for x in range(8):  # inside its XCD's window, the tiles in which a range begins first
        lo, nxt = (x * tiles + 7) // 8, ((x + 1) * tiles + 7) // 8
        window = placed[lo:nxt]
        assert sorted(window) == list(range(lo, nxt))
        begins = [t for t in range(lo, nxt) if (t + 1) * ranges // tiles > t * ranges // tiles]
        assert [placed[t] for t in begins] == list(range(lo, lo + len(begins)))


@pytest.mark.parametrize("tiles,chunks,ranges,weight", [
    (392, 8, 256, 2), (784, 8, 256, 3), (392, 16, 256, 1), (300, 8, 256, 4), (1176, 8, 256, 2), (256, 64, 256, 5),
    (1000, 3, 128, 6), (257, 1, 256, 1), (12345, 32, 256, 2)])
@pytest.mark.parametrize("kw", [2, 4])
def test_weighted_ranges_cover_the_line_of_units(gen, kw, tiles, chunks, ranges, weight):
    # fp32 kernels, ranges cut on the weighted line (a tile = 2 * chunks + weight half units): the
    # emitted code, run for every range, must give ranges that follow each other without gap or
    # overlap from unit 0 to the last unit, none empty, each starting at its (tile, chunk), and
    # the ranges must be those of the closed form.
    k = gen.Kernel(kw)
    k.lines = []
    k.weighted_unit_range(f"s{k.S['L']}", f"s{k.S['SegEnd']}")
    code = list(k.lines)
    assert not any("branch" in l or re.match(r"^\S+:$", l) for l in code)
    vt = 2 * chunks + weight
    total = tiles * vt
    q, rem = divmod(total, ranges)
    mg, sh = magic(vt)
    pos = lambda v: (v // vt) * chunks + min((v % vt + 1) // 2, chunks)
    at = 0
    for L in range(ranges):
        m = ScalarMachine()
        m.s.update({k.S["L"]: L, k.S["SegEnd"]: vt, k.S["UnitsQ"]: q, k.S["UnitsRem"]: rem, k.S["Chunks"]: chunks,
                    k.S["Mch"]: mg, k.S["Sch"]: sh | (weight << 8)})
        m.run(code)
        begin, n, tm, cm = (m.s[k.S[x]] for x in ("Begin", "Nunits", "Tm", "Cm"))
        assert begin == at and n > 0 and cm < chunks and tm * chunks + cm == begin
        assert begin == pos(L * q + min(L, rem)) and begin + n == pos((L + 1) * q + min(L + 1, rem))
        at += n
    assert at == tiles * chunks
