"""Static checks on the gfx950 assembly hipcc generates for the direct-to-LDS kernels (no GPU needed).

The ring kernels issue their LDS fragment reads as inline assembly and retire them with an explicit
`s_waitcnt lgkmcnt(0)`: the compiler does not know that a destination register is not yet valid between the read
and that wait.  If it ever handed such a register to something else (a copy, an address computation), the kernel
would compute with, or load from, garbage -- a timing probe variant of the kernel once faulted exactly that way.
These tests compile every instantiation the library ships to assembly and check, per kernel:

  * no instruction between an LDS read and the next `s_waitcnt lgkmcnt(0)` names a register the read writes;
  * nothing is spilled to scratch memory inside the main loop;
  * the 16x16x32 kernel claims exactly the accumulation registers its MFMAs name (64, 128 or 256), so none of
    them can be given to another value.
"""
import os
import re
import subprocess
from concurrent.futures import ThreadPoolExecutor

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "gemm_mmbo_amd", "csrc")
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
         "-Wno-unused-command-line-argument", "--cuda-device-only", "-S"]

pytestmark = pytest.mark.skipif(not os.path.exists(HIPCC), reason="hipcc not installed")

#        source file            defines
UNITS = [("inst_x16.hip", ["-DMMBO_DTYPE=%d" % d, "-DMMBO_TILE=%d" % t]) for d in (0, 1) for t in range(8)] + \
        [("inst_ring.hip", ["-DMMBO_DTYPE=%d" % d, "-DMMBO_TILE=%d" % t]) for d in (0, 1) for t in range(4)]


def _compile(unit, outdir):
    src, defs = unit
    out = os.path.join(outdir, src.replace(".hip", "") + "".join(d.replace("-D", "_").replace("=", "") for d in defs) + ".s")
    r = subprocess.run([HIPCC] + FLAGS + defs + [os.path.join(CSRC, src), "-o", out], capture_output=True, text=True)
    assert r.returncode == 0, r.stderr[-3000:]
    return out


def _kernels(path):
    """{kernel symbol: list of instruction lines (and '.LBB..:' labels)} of one assembly file."""
    lines = open(path).read().split("\n")
    starts = [i for i, l in enumerate(lines) if re.match(r"^_Z\w+:", l)]
    out = {}
    for n, i in enumerate(starts):
        end = starts[n + 1] if n + 1 < len(starts) else len(lines)
        body = []
        for l in lines[i + 1:end]:
            t = l.strip()
            if t.startswith(".amdhsa_kernel") or t.startswith(".section"):
                break
            if re.match(r"^\.LBB\w+:", t):
                body.append(t.split(":")[0] + ":")
            elif t and not t.startswith(";") and not t.startswith("."):
                body.append(t.split(";")[0].strip())
        out[lines[i].split(":")[0]] = body
    return out


def _vregs(text):
    regs = set()
    for a, b in re.findall(r"\bv\[(\d+):(\d+)\]", text):
        regs.update(range(int(a), int(b) + 1))
    regs.update(int(a) for a in re.findall(r"\bv(\d+)\b", text))
    return regs


def _sregs(text):
    regs = set()
    for a, b in re.findall(r"\bs\[(\d+):(\d+)\]", text):
        regs.update(range(int(a), int(b) + 1))
    regs.update(int(a) for a in re.findall(r"\bs(\d+)\b", text))
    return regs


def _inflight_violations(body):
    """Forward data flow over the kernel's control-flow graph: the set of registers with an LDS read in flight at
    each instruction is the union over its predecessors; a read adds its destination, `s_waitcnt lgkmcnt(0)` empties
    the set, and any other instruction that names a register of the set is a violation.

    The walk follows one kind of infeasible path no further: for `if (c) A else B` between two long straight-line
    blocks the compiler emits "B (when !c), flag = 0 -- or flag = -1 -- then: A when flag", with the flag in a scalar
    register pair (`s_mov_b64 s[a:b], 0` / `-1` ... `s_and_b64` or `s_andn2_b64 vcc, exec, s[a:b]` ... `s_cbranch_vccz` / `vccnz`).  The state
    therefore carries the flags whose constant value is known on the path at hand, and a branch on such a flag has one
    successor."""
    label = {t[:-1]: i for i, t in enumerate(body) if t.endswith(":")}

    def step_flags(t, flags, vcc):
        """(flags, vcc) after instruction t.  flags: frozenset of ((lo, hi), value); vcc: None, 0 or 1."""
        m = re.match(r"s_mov_b64 s\[(\d+):(\d+)\], (0|-1)$", t)
        if m:
            key = (int(m.group(1)), int(m.group(2)))
            return frozenset({f for f in flags if f[0] != key} | {(key, 0 if m.group(3) == "0" else 1)}), vcc
        m = re.match(r"s_(and|andn2)_b64 vcc, exec, s\[(\d+):(\d+)\]$", t)
        if m:
            key = (int(m.group(2)), int(m.group(3)))
            known = next((v for k, v in flags if k == key), None)
            return flags, known if known is None or m.group(1) == "and" else 1 - known
        if t.startswith(("s_", "v_cmp", "v_readlane", "v_readfirstlane")) and not t.startswith(("s_cbranch", "s_branch", "s_waitcnt", "s_nop", "s_barrier")):
            dst = t.split(None, 1)[1].split(",")[0] if " " in t else ""
            if "vcc" in dst or t.startswith("v_cmp"):
                vcc = None
            hit = _sregs(dst)
            if hit:
                flags = frozenset(f for f in flags if not (set(range(f[0][0], f[0][1] + 1)) & hit))
        return flags, vcc

    def succ(i, t, vcc):
        if t.startswith("s_endpgm"):
            return []
        m = re.match(r"s_(c?branch\w*) (\.LBB\w+)", t)
        if m:
            tgt = label[m.group(2)]
            if m.group(1) == "branch":
                return [tgt]
            if vcc is not None and m.group(1) in ("cbranch_vccz", "cbranch_vccnz"):
                taken = (vcc == 0) == (m.group(1) == "cbranch_vccz")
                return [tgt] if taken else [i + 1]
            return [i + 1, tgt]
        return [i + 1] if i + 1 < len(body) else []

    start = (0, frozenset(), None)
    pend_in = {start: frozenset()}
    work, bad = [start], {}
    while work:
        node = work.pop()
        i, flags, vcc = node
        t, cur = body[i], pend_in[node]
        out = cur
        nflags, nvcc = flags, vcc
        if not t.endswith(":"):
            m = re.match(r"ds_read\w* (v\[\d+:\d+\]|v\d+),", t)
            if m:
                if _vregs(t[m.end():]) & cur:
                    bad[i] = t
                out = cur | _vregs(m.group(1))
            elif t.startswith("s_waitcnt") and "lgkmcnt(0)" in t:
                out = frozenset()
            elif cur and (_vregs(t) & cur):
                bad[i] = t
            nflags, nvcc = step_flags(t, flags, vcc)
        for j in succ(i, t, vcc):
            nxt = (j, nflags, nvcc)
            new = out if nxt not in pend_in else pend_in[nxt] | out
            if nxt not in pend_in or new != pend_in[nxt]:
                pend_in[nxt] = frozenset(new)
                work.append(nxt)
    return [bad[i] for i in sorted(bad)]


@pytest.fixture(scope="module")
def asm_files(tmp_path_factory):
    outdir = str(tmp_path_factory.mktemp("asm"))
    with ThreadPoolExecutor(max_workers=min(8, os.cpu_count() or 1)) as ex:
        return list(ex.map(lambda u: _compile(u, outdir), UNITS))


def test_checker_follows_a_constant_flag_but_not_an_unknown_one():
    # "if (c) A else B" as the compiler lays it out: B, flag = 0, then A under the flag.  With the flag known the path from
    # B's read into A does not exist; with the flag unknown (set from a comparison) it does, and A's use is a violation.
    tail = ["s_and_b64 vcc, exec, s[6:7]", "s_cbranch_vccz .LBB0_9", "v_add_u32_e32 v11, s3, v9", ".LBB0_9:", "s_waitcnt lgkmcnt(0)", "s_endpgm"]
    known = ["ds_read_b128 v[10:13], v5 offset:64", "s_mov_b64 s[6:7], 0", ".LBB0_8:"] + tail
    assert _inflight_violations(known) == []
    unknown = ["ds_read_b128 v[10:13], v5 offset:64", "s_cselect_b64 s[6:7], -1, 0", ".LBB0_8:"] + tail
    assert _inflight_violations(unknown) == ["v_add_u32_e32 v11, s3, v9"]
    overwritten = ["ds_read_b128 v[10:13], v5 offset:64", "s_mov_b64 s[6:7], 0", "s_or_b64 s[6:7], s[6:7], s[20:21]", ".LBB0_8:"] + tail
    assert _inflight_violations(overwritten) == ["v_add_u32_e32 v11, s3, v9"]
    set_one = ["ds_read_b128 v[10:13], v5 offset:64", "s_mov_b64 s[6:7], -1", ".LBB0_8:"] + tail
    assert _inflight_violations(set_one) == ["v_add_u32_e32 v11, s3, v9"]
    # the complemented form: vcc = exec & ~flag, skip A when vcc != 0
    tail2 = ["s_andn2_b64 vcc, exec, s[6:7]", "s_cbranch_vccnz .LBB0_9"] + tail[2:]
    assert _inflight_violations(["ds_read_b128 v[10:13], v5 offset:64", "s_mov_b64 s[6:7], 0", ".LBB0_8:"] + tail2) == []
    assert _inflight_violations(["ds_read_b128 v[10:13], v5 offset:64", "s_mov_b64 s[6:7], -1", ".LBB0_8:"] + tail2) == ["v_add_u32_e32 v11, s3, v9"]


def test_checker_sees_a_planted_violation():
    body = ["ds_read_b128 v[10:13], v5 offset:64", "v_add_u32_e32 v11, s3, v9", "s_waitcnt lgkmcnt(0)"]
    assert _inflight_violations(body) == ["v_add_u32_e32 v11, s3, v9"]
    ok = ["ds_read_b64_tr_b16 v[10:11], v5", "v_mfma_f32_16x16x32_f16 a[0:3], v[20:23], v[24:27], a[0:3]",
          "s_waitcnt vmcnt(2)", "s_waitcnt lgkmcnt(0)", "v_mfma_f32_16x16x32_f16 a[0:3], v[10:13], v[24:27], a[0:3]"]
    assert _inflight_violations(ok) == []
    # control flow: the block after an unconditional branch is not its successor, the branch target is
    jump = ["ds_read_b32 v7, v3", "s_branch .LBB0_2", ".LBB0_1:", "v_mov_b32_e32 v7, 0", "s_endpgm", ".LBB0_2:",
            "s_waitcnt lgkmcnt(0)", "v_add_u32_e32 v8, v7, v7", "s_endpgm"]
    assert _inflight_violations(jump) == []
    loop = [".LBB0_1:", "v_add_u32_e32 v9, v7, v7", "ds_read_b32 v7, v3", "s_cbranch_scc1 .LBB0_1", "s_waitcnt lgkmcnt(0)",
            "s_endpgm"]
    assert _inflight_violations(loop) == ["v_add_u32_e32 v9, v7, v7"]       # the back edge carries the read in flight


def test_no_register_is_touched_while_its_lds_read_is_in_flight(asm_files):
    checked = 0
    for path in asm_files:
        for name, body in _kernels(path).items():
            if not any(t.startswith("ds_read") for t in body):
                continue
            bad = _inflight_violations(body)
            assert not bad, f"{name}: {bad[:3]}"
            checked += 1
    assert checked >= 4 * (10 + 8)         # four transposes of every tile of both families, both element types


def _compiler_generated(path):
    """{kernel symbol: instruction lines the compiler generated itself}, i.e. everything outside the ;;#ASMSTART ... ;;#ASMEND
    brackets the compiler puts around the text of an asm statement."""
    lines = open(path).read().split("\n")
    starts = [i for i, l in enumerate(lines) if re.match(r"^_Z\w+:", l)]
    out = {}
    for n, i in enumerate(starts):
        end = starts[n + 1] if n + 1 < len(starts) else len(lines)
        body, inside = [], False
        for l in lines[i + 1:end]:
            t = l.strip()
            if t.startswith(".amdhsa_kernel") or t.startswith(".section"):
                break
            if t.startswith(";;#ASMSTART"):
                inside = True
            elif t.startswith(";;#ASMEND"):
                inside = False
            elif not inside and t and not t.startswith(";") and not t.startswith(".") and not re.match(r"^\.?LBB\w+:", t):
                body.append(t.split(";")[0].strip())
        out[lines[i].split(":")[0]] = body
    return out


def test_nothing_but_the_direct_loads_touches_m0(asm_files):
    """The direct loads set M0 (the LDS destination) inside their own asm statement and leave it changed without telling
    the compiler, which refuses M0 in a clobber list.  That is only sound while the compiler keeps nothing in M0 itself:
    no instruction it generated for these kernels may name M0."""
    checked = 0
    for path in asm_files:
        for name, body in _compiler_generated(path).items():
            bad = [t for t in body if re.search(r"\bm0\b", t)]
            assert not bad, f"{name}: compiler-generated use of m0: {bad[:3]}"
            checked += 1
        text = open(path).read()
        assert "buffer_load_dwordx4" in text and " lds" in text        # the asm statements are there (and inside brackets)
    assert checked >= 4 * (10 + 8)


def _main_loops(body):
    """(first, last) instruction index of the innermost backward-branch ranges that hold MFMAs but neither a store to
    global memory nor the zeroing of an accumulator: the steady-state slice loops.  (The loop over the tiles of a resident
    work-group holds both.  Ranges that enclose another such range are left out: the compiler shares blocks between
    the ring fill and the last slices and jumps back to them, which looks like a loop around the steady-state one.)"""
    labels = {t[:-1]: i for i, t in enumerate(body) if t.endswith(":")}
    loops = []
    for i, t in enumerate(body):
        if t.startswith(("s_branch", "s_cbranch")):
            j = labels.get(t.split()[-1], i + 1)
            if j < i:
                inside = body[j:i + 1]
                if any(x.startswith("v_mfma") for x in inside) and \
                        not any(x.startswith(("global_store", "buffer_store", "flat_store")) or
                                re.match(r"v_accvgpr_write_b32 a\[?\w+\]?, 0$", x) for x in inside):
                    loops.append((j, i))
    return [(a, b) for (a, b) in loops if not any((c, d) != (a, b) and a <= c and d <= b for (c, d) in loops)]


def test_main_loop_finder_on_planted_code():
    body = ["s_nop 0", ".LBB0_1:", "v_mfma_f32_16x16x32_f16 a[0:3], v[0:3], v[4:7], a[0:3]", "scratch_load_dword v1, off, off",
            "s_cbranch_scc1 .LBB0_1", "v_mfma_f32_16x16x32_f16 a[0:3], v[0:3], v[4:7], a[0:3]", "global_store_dword v[0:1], v2, off",
            "s_cbranch_scc1 .LBB0_1", "s_endpgm"]
    assert _main_loops(body) == [(1, 4)]
    body2 = [".LBB0_1:", "v_accvgpr_write_b32 a[0x1f], 0", ".LBB0_2:", "v_mfma_f32_16x16x32_f16 a[0:3], v[0:3], v[4:7], a[0:3]",
             "s_cbranch_scc1 .LBB0_2", "scratch_load_dword v1, off, off", "s_cbranch_scc1 .LBB0_1", "s_endpgm"]
    assert _main_loops(body2) == [(2, 4)]
    body3 = [".LBB0_0:", "scratch_load_dword v1, off, off", ".LBB0_1:", "v_mfma_f32_16x16x32_f16 a[0:3], v[0:3], v[4:7], a[0:3]",
             "s_cbranch_scc1 .LBB0_1", "v_mfma_f32_16x16x32_f16 a[0:3], v[0:3], v[4:7], a[0:3]", "s_cbranch_scc1 .LBB0_0", "s_endpgm"]
    assert _main_loops(body3) == [(2, 4)]


def test_no_scratch_spills_in_the_main_loop(asm_files):
    """A spilled register inside the main loop would be reloaded through vector memory, and the wait for it would
    drain the ring of direct loads.  No loop over slices may touch scratch; a few values parked around the ring fill
    and the partial last slice of the fullest kernels are tolerated (most in the fp16 256 x 256 kernel with neither
    operand k-contiguous: about 20 values, stored before the ring fill and fetched back after the slice loop)."""
    for path in asm_files:
        # The eight-wave form of the 256 x 256 tile has 128 registers per lane beside its accumulators: with the
        # resident-work-group bookkeeping it spills a few values.  It is never picked automatically (the four-wave
        # form is faster) and stays only so that a sweep can show it.
        if "inst_x16" in path and path.endswith("_MMBO_TILE1.s"):
            continue
        for name, body in _kernels(path).items():
            mf = [i for i, t in enumerate(body) if t.startswith("v_mfma")]
            sc = [i for i, t in enumerate(body) if t.startswith("scratch_")]
            if not mf:
                assert not sc, f"{name} spills to scratch"
                continue
            loops = _main_loops(body)
            assert loops, f"{name}: no slice loop found"
            assert not [i for i in sc if any(a <= i <= b for a, b in loops)], f"{name} spills to scratch inside its main loop"
            assert len(sc) <= 48, f"{name}: {len(sc)} scratch accesses"


def test_x16_kernels_claim_exactly_their_accumulation_registers(asm_files):
    seen = 0
    for path in asm_files:
        if "inst_x16" not in path:
            continue
        text = open(path).read()
        for name, body in _kernels(path).items():
            used = set()
            for t in body:
                # (the assembler prints register indices above 64 in hex)
                for a, b in re.findall(r"\ba\[(\w+):(\w+)\]", t):
                    used.update(range(int(a, 0), int(b, 0) + 1))
                used.update(int(a, 0) for a in re.findall(r"\ba\[(\w+)\]", t))
                # no accumulation register may appear outside the MFMAs, the zeroing and the read-back
                # (an MFMA statement only declares the four registers it writes as clobbered, so the compiler believes the
                # others free at that point: it must never have put a value of its own into one -- the only writes are
                # the MFMAs and the zeroing at the start of a tile)
                if re.search(r"\ba\[?\d", t):
                    assert t.startswith(("v_mfma_f32_16x16x32_f16", "v_mfma_f32_16x16x4_f32", "v_accvgpr_write_b32",
                                         "v_accvgpr_read_b32")), (name, t)
                    if t.startswith("v_accvgpr_write_b32"):
                        assert re.match(r"v_accvgpr_write_b32 a\[?\w+\]?, 0$", t), (name, t)
            # and none of that is the compiler's own: every instruction that names an accumulation register sits inside an asm
            # statement (under register pressure the compiler parks values of its own in accumulation registers)
            own = [t for t in _compiler_generated(path)[name] if re.search(r"\ba\[?\d", t)]
            assert not own, (name, own[:3])
            m = re.search(r"\.amdhsa_kernel " + re.escape(name) + r"\b.*?\.amdhsa_next_free_vgpr (\d+).*?\.amdhsa_accum_offset (\d+)",
                          text, re.S)
            assert m, name
            agprs = int(m.group(1)) - int(m.group(2))       # registers past the unified file's accumulation offset
            assert used == set(range(len(used))) and len(used) in (64, 128, 256), (name, len(used))
            assert agprs == len(used), (name, agprs, len(used))
            seen += 1
    # 8 tiles x 2 element types x 4 transposes, + 6 fp16 tiles x 4 transposes with the old-C variant, + the TN variant with both
    # operands on the even slices for the 5 tiles with five ring buffers x 2 element types, + its 5 fp16 old-C forms
    assert seen == 88 + 10 + 5


def _unpadded_wide_stores(body):
    """Buffer stores of more than 8 bytes whose data registers the very next instruction writes.  The compiler pads such
    a pair with wait states only when the store has no scalar offset register; with one it takes the hazard not to
    exist, and on this chip lanes then stored the next value (seen with an accumulator read-back right behind the
    store).  The epilogues therefore keep the scalar offset at literal zero."""
    bad = []
    for i, t in enumerate(body):
        m = re.match(r"buffer_store_dwordx[34] (v\[\d+:\d+\]), \S+ s\[\d+:\d+\], (\S+)", t)
        if not m:
            continue
        j = i + 1
        while j < len(body) and body[j].endswith(":"):
            j += 1
        if j < len(body) and body[j].startswith("v_") and not body[j].startswith("v_cmp"):
            dst = body[j].split(None, 1)[1].split(",")[0]
            if _vregs(dst) & _vregs(m.group(1)):
                bad.append((t, body[j]))
    return bad


def test_wide_store_checker_sees_a_planted_pair():
    body = ["buffer_store_dwordx4 v[16:19], v68, s[40:43], s0 offen nt", "v_accvgpr_read_b32 v16, a[4]", "s_endpgm"]
    assert len(_unpadded_wide_stores(body)) == 1
    body = ["buffer_store_dwordx4 v[16:19], v68, s[40:43], 0 offen sc1", "s_nop 1", "v_accvgpr_read_b32 v16, a[4]", "s_endpgm"]
    assert not _unpadded_wide_stores(body)


def test_no_wide_buffer_store_is_followed_by_a_write_to_its_data(asm_files):
    seen = 0
    for path in asm_files:
        for name, body in _kernels(path).items():
            stores = [t for t in body if t.startswith("buffer_store_dwordx")]
            for t in stores:
                # (no scalar offset register on any of them: that is what makes the compiler pad the pair)
                assert re.search(r"s\[\d+:\d+\], 0 offen", t), (name, t)
            assert not _unpadded_wide_stores(body), (name, _unpadded_wide_stores(body)[:2])
            seen += bool(stores)
    assert seen >= 64           # every x16 kernel stores C through a buffer
