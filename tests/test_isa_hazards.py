"""Wait-state hazards around the inline-assembly memory instructions of the HIP kernels.

The compiler inserts the wait states gfx9-family hardware needs between certain instruction pairs, but it does not
look inside inline assembly.  Three of those pairs involve the hand-written vector-memory instructions of the tuned
kernels (direct-to-LDS copies, non-temporal stores):
  * a vector instruction writes a scalar register (v_readlane / v_readfirstlane, e.g. the reload of a spilled scalar)
    and a vector-memory instruction reads that register fewer than five wait states later: it sees the old value --
    for a buffer descriptor that means a wild address;
  * a 12- or 16-byte store is followed within two wait states by a vector instruction that overwrites its data
    registers: the store writes the new value;
  * a scalar instruction writes m0 and the very next instruction is a copy to LDS (a buffer load with the lds
    modifier), which takes its LDS address from m0: one wait state must lie between them.
The first two were met while developing these kernels (a GPU memory fault, and wrong dwords in the output); the
third is the rule the compiler applies to its own copies of this kind.  The build keeps
the device assembly (triton_grouped_gemm_amd/build/*.gfx950.s); this test scans it.  The scanner itself is checked
on hand-written snippets, so the file tests something even where the library has not been built.
"""
import re
from pathlib import Path

import pytest

BUILD = Path(__file__).resolve().parents[1] / "triton_grouped_gemm_amd" / "build"


def _regs(tok: str, kind: str):
    m = re.match(kind + r"\[(\d+):(\d+)\]$", tok)
    if m:
        return set(range(int(m.group(1)), int(m.group(2)) + 1))
    m = re.match(kind + r"(\d+)$", tok)
    return {int(m.group(1))} if m else set()


def _wait_states(line: str) -> int:
    m = re.match(r"s_nop (\d+)", line)
    return int(m.group(1)) + 1 if m else 1


def scan(text: str):
    """Returns a list of (first instruction, second instruction, wait states between them) for every hazard found."""
    code = []
    for raw in text.splitlines():
        line = raw.split(";")[0].strip()
        if line and not line.startswith(".") and not line.endswith(":"):
            code.append(line)
    bad = []
    for i, line in enumerate(code):
        op = line.split()[0]
        toks = [t.strip(",") for t in line.split()[1:]]
        if not op.startswith(("buffer_", "global_", "flat_", "scratch_")):
            continue
        if op.startswith("buffer_load") and toks[-1] == "lds" and i > 0:
            prev = code[i - 1].split()
            if prev[0].startswith("s_") and len(prev) > 1 and prev[1].strip(",") == "m0":
                bad.append((code[i - 1], line, 0))
        need = set().union(*[_regs(t, "s") for t in toks]) if toks else set()
        ws = 0
        for d in range(1, 8):
            if not need or i - d < 0 or ws >= 5:
                break
            prev = code[i - d]
            ptoks = prev.split()
            if ptoks[0].startswith("v_") and len(ptoks) > 1 and _regs(ptoks[1].strip(","), "s") & need:
                bad.append((prev, line, ws))
                break
            ws += _wait_states(prev)
        if re.match(r"(buffer|global|flat|scratch)_store_dwordx[34]", op):
            data = _regs(toks[0], "v") if op.startswith("buffer") else _regs(toks[1], "v")
            ws = 0
            for d in range(1, 4):
                if i + d >= len(code) or ws >= 2:
                    break
                nxt = code[i + d]
                ntoks = nxt.split()
                if ntoks[0].startswith("v_") and len(ntoks) > 1 and _regs(ntoks[1].strip(","), "v") & data:
                    bad.append((line, nxt, ws))
                    break
                ws += _wait_states(nxt)
    return bad


def test_scanner_finds_scalar_write_before_vector_memory_read():
    hazard = "v_readlane_b32 s47, v254, 19\ns_waitcnt lgkmcnt(0)\nbuffer_store_dwordx4 v[2:5], v6, s[44:47], 0 offen nt\n"
    assert len(scan(hazard)) == 1
    spaced = "v_readlane_b32 s47, v254, 19\ns_nop 4\nbuffer_store_dwordx4 v[2:5], v6, s[44:47], 0 offen nt\ns_nop 1\n"
    assert scan(spaced) == []
    other_register = "v_readlane_b32 s12, v254, 19\nbuffer_load_dwordx4 v1, s[44:47], 0 offen lds\n"
    assert scan(other_register) == []
    scalar_writer = "s_mov_b32 s44, s3\nbuffer_load_dwordx4 v1, s[44:47], 0 offen lds\n"  # scalar writes are interlocked
    assert scan(scalar_writer) == []


def test_scanner_finds_overwritten_store_data():
    hazard = "global_store_dwordx4 v[8:9], v[0:3], off nt\nv_add_u32_e32 v0, 64, v8\n"
    assert len(scan(hazard)) == 1
    assert scan("global_store_dwordx4 v[8:9], v[0:3], off nt\ns_nop 1\nv_add_u32_e32 v0, 64, v8\n") == []
    assert scan("global_store_dwordx4 v[8:9], v[0:3], off nt\nv_add_u32_e32 v12, 64, v8\nv_mov_b32_e32 v13, v1\nv_mov_b32_e32 v0, v1\n") == []
    assert scan("global_store_dwordx2 v[8:9], v[0:1], off\nv_add_u32_e32 v0, 64, v8\n") == []  # 8-byte stores are not affected


def test_scanner_finds_copy_to_lds_right_after_a_write_of_m0():
    assert len(scan("s_mov_b32 m0, s2\nbuffer_load_dwordx4 v2, s[44:47], 0 offen lds\n")) == 1
    assert len(scan("s_add_u32 m0, s2, 16\nbuffer_load_dword v2, s[44:47], 0 offen lds\n")) == 1
    assert scan("s_mov_b32 m0, s2\ns_nop 0\nbuffer_load_dwordx4 v2, s[44:47], 0 offen lds\n") == []
    assert scan("s_mov_b32 m0, s2\nv_add_u32_e32 v2, 64, v8\nbuffer_load_dwordx4 v2, s[44:47], 0 offen lds\n") == []
    assert scan("s_mov_b32 m0, s2\nbuffer_load_dwordx4 v[2:5], v1, s[44:47], 0 offen\n") == []  # an ordinary load does not read m0


def test_built_kernels_have_no_unspaced_hazard():
    files = sorted(BUILD.glob("*.gfx950.s"))
    if not files:
        pytest.skip("no device assembly in the build directory (the library was built elsewhere or not yet)")
    for f in files:
        found = scan(f.read_text())
        assert not found, f"{f.name}: {len(found)} hazards, first: {found[0]}"


# The four-wave kernel keeps operand chunks that are in flight across loop iterations in v[192:255], named in the
# text of its own load and LDS-write statements; the compiler must never have allocated one of them for itself (it
# would move or overwrite a value it knows nothing about).
_RESERVED = set(range(192, 256))


def stray_uses_of_reserved_registers(text: str):
    """Lines of the four-wave kernels that touch v192..v255 other than the staging loads and LDS writes."""
    stray, inside = [], False
    for raw in text.splitlines():
        line = raw.split(";")[0].strip()
        if line.endswith(":") and not line.startswith("."):
            inside = "gemm_w4_kernel" in line
            continue
        if not inside or not line or line.startswith("."):
            continue
        toks = [t.strip(",") for t in line.split()]
        used = set().union(*[_regs(t, "v") for t in toks[1:]]) & _RESERVED
        if not used:
            continue
        staged_load = toks[0] == "buffer_load_dwordx4" and _regs(toks[1], "v") == used and toks[-1] != "lds"
        staged_write = toks[0] == "ds_write_b128" and _regs(toks[2], "v") == used
        if not (staged_load or staged_write):
            stray.append(line)
    return stray


def test_reserved_register_scanner_on_snippets():
    head = "_ZN3tgg14gemm_w4_kernelILi0ELi0EEEvNS_10GemmParamsE:\n"
    assert stray_uses_of_reserved_registers(head + "buffer_load_dwordx4 v[192:195], v130, s[12:15], s85 offen\n") == []
    assert stray_uses_of_reserved_registers(head + "ds_write_b128 v146, v[252:255] offset:0x7000\n") == []
    assert len(stray_uses_of_reserved_registers(head + "v_mov_b32_e32 v200, v3\n")) == 1
    assert len(stray_uses_of_reserved_registers(head + "v_add_u32_e32 v3, v3, v255\n")) == 1
    assert len(stray_uses_of_reserved_registers(head + "ds_write_b128 v192, v[4:7]\n")) == 1  # as the address
    assert stray_uses_of_reserved_registers("other_kernel:\nv_mov_b32_e32 v200, v3\n") == []


def test_four_wave_kernel_keeps_its_reserved_registers_to_itself():
    f = BUILD / "gemm_w4.gfx950.s"
    if not f.exists():
        pytest.skip("no device assembly in the build directory (the library was built elsewhere or not yet)")
    text = f.read_text()
    assert "gemm_w4_kernel" in text
    stray = stray_uses_of_reserved_registers(text)
    assert not stray, f"{len(stray)} compiler-generated uses of v[192:255], first: {stray[0]}"


# The four-wave kernel's multiplies are inline assembly, so the compiler does not know when their results land: it
# places the epilogue's v_accvgpr_read wherever the source order allows.  The source order is written so that a block
# is read no sooner than three multiplies (48 cycles of issue) after the multiply that wrote it, or behind a
# statement of idle cycles; this scanner checks the kept assembly for it, in text order (what crosses a loop's back
# edge is further apart than what it sees).
_MIN_MULTIPLIES_BETWEEN = 3
_MIN_IDLE_WAIT_STATES = 12


def accumulator_reads_too_early(text: str):
    """(multiply, read, multiplies in between, idle wait states in between) for every v_accvgpr_read in a four-wave
    kernel that follows the multiply that wrote its register too closely."""
    bad, inside = [], False
    last_write = {}  # accumulator register -> (index of the multiply that wrote it, its text, idle wait states issued so far)
    n_mul, idle = 0, 0
    for raw in text.splitlines():
        line = raw.split(";")[0].strip()
        if line.endswith(":") and not line.startswith("."):
            inside = "gemm_w4_kernel" in line
            last_write, n_mul, idle = {}, 0, 0
            continue
        if not inside or not line or line.startswith("."):
            continue
        toks = [t.strip(",") for t in line.split()]
        if toks[0].startswith("v_mfma"):
            for r in _regs(toks[1], "a"):
                last_write[r] = (n_mul, line, idle)
            n_mul += 1
        elif toks[0] == "s_nop":
            idle += _wait_states(line)
        elif toks[0] == "v_accvgpr_read_b32":
            for r in _regs(toks[2], "a"):
                if r in last_write:
                    at, mul, idle_then = last_write[r]
                    between, waited = n_mul - at - 1, idle - idle_then
                    if between < _MIN_MULTIPLIES_BETWEEN and waited < _MIN_IDLE_WAIT_STATES:
                        bad.append((mul, line, between, waited))
    return bad


def test_accumulator_read_scanner_on_snippets():
    head = "_ZN3tgg14gemm_w4_kernelILi0ELi0ELb0EEEvNS_10GemmParamsE:\n"
    mul = lambda a: f"v_mfma_f32_16x16x32_bf16 a[{a}:{a + 3}], v[2:5], v[6:9], a[{a}:{a + 3}]\n"
    assert len(accumulator_reads_too_early(head + mul(0) + "v_accvgpr_read_b32 v1, a2\n")) == 1
    assert len(accumulator_reads_too_early(head + mul(0) + mul(4) + mul(8) + "v_accvgpr_read_b32 v1, a0\n")) == 1
    assert accumulator_reads_too_early(head + mul(0) + mul(4) + mul(8) + mul(12) + "v_accvgpr_read_b32 v1, a3\n") == []
    assert accumulator_reads_too_early(head + mul(0) + "s_nop 15\ns_nop 7\nv_accvgpr_read_b32 v1, a1\n") == []
    assert accumulator_reads_too_early(head + mul(0) + "v_accvgpr_read_b32 v1, a9\n") == []  # another block
    assert accumulator_reads_too_early("other_kernel:\n" + mul(0) + "v_accvgpr_read_b32 v1, a2\n") == []


def test_four_wave_kernel_reads_no_accumulator_right_behind_its_multiply():
    f = BUILD / "gemm_w4.gfx950.s"
    if not f.exists():
        pytest.skip("no device assembly in the build directory (the library was built elsewhere or not yet)")
    found = accumulator_reads_too_early(f.read_text())
    assert not found, f"{len(found)} reads too close behind the multiply, first: {found[0]}"
