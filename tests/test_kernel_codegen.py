"""What the compiler made of the hand-ordered main loops of the direct-load kernels (no GPU needed).

A step of those loops is meant to hold nothing but MFMAs, direct loads, LDS reads, waits, the barrier and
scalar instructions: a vector instruction between f64 MFMAs waits for the matrix pipe, and a branch cuts the
step into blocks the MFMAs do not overlap.  Neither shows in a parity test, and both have happened (LDS read
addresses recomputed before every read; the test for a short last K tile in every step): configuration 3
took 107.7 instead of 98 us.  So the device assembly of the instantiations the benchmark configurations run
is checked here: the loop that holds the MFMAs of a whole ring of K tiles has no vector ALU instruction and
no branch but its own."""
import os
import re
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
KDIR = os.path.join(ROOT, "hiptensor_amd", "csrc", "kernels")


_ASM = {}

# every translation unit a test of this file looks at: the first request compiles them all, side by side
UNITS = ["contract_f64", "contract_c32", "contract_f16_hd", "contract_f32", "contract_c64",
         "contract_f16_hk_kx", "contract_f16_hk_rx", "contract_bf16_hk_kx", "contract_bf16_hk_rx",
         "contract_f16_hr192_kx", "contract_f16_hr192_rx", "contract_bf16_hr192_kx", "contract_bf16_hr192_rx"]


def device_asm(unit, tmp_path):
    if unit not in _ASM:
        from concurrent.futures import ThreadPoolExecutor

        todo = [u for u in dict.fromkeys([unit] + UNITS) if u not in _ASM]
        with ThreadPoolExecutor(max_workers=min(8, os.cpu_count() or 1)) as pool:
            for u, lines in zip(todo, pool.map(lambda u: _compile(u, tmp_path), todo)):
                _ASM[u] = lines
    return _ASM[unit]


def _compile(unit, tmp_path):
    out = tmp_path / (unit + ".s")
    subprocess.run(["hipcc", "--offload-arch=gfx950", "-O3", "-std=c++17", "-Xclang", "-target-feature", "-Xclang",
                    "-packed-fp32-ops", "-Wno-unused-command-line-argument", "-Wno-option-ignored",
                    "-I" + os.path.join(ROOT, "include"), "-I" + KDIR, "--cuda-device-only", "-S", "-o", str(out),
                    os.path.join(KDIR, unit + ".hip")], check=True, capture_output=True)
    return out.read_text().split("\n")


def kernel_body(lines, symbol):
    start = next(i for i, l in enumerate(lines) if l.startswith(symbol + ":"))
    end = next(i for i in range(start, len(lines)) if "s_endpgm" in lines[i])
    return lines[start:end]


def main_loops(body, min_mfma):
    """(first, last) line of every loop (label ... backward conditional branch to it) with at least min_mfma MFMAs
    that holds no other such loop."""
    labels = {m.group(1): i for i, l in enumerate(body) if (m := re.match(r"^(\.LBB\d+_\d+):", l))}
    loops = []
    for i, l in enumerate(body):
        m = re.search(r"s_cbranch_\w+\s+(\.LBB\d+_\d+)", l)
        if m and labels.get(m.group(1), i) < i:
            a = labels[m.group(1)]
            if sum("v_mfma" in x for x in body[a:i]) >= min_mfma:
                loops.append((a, i))
    return [(a, b) for a, b in loops if not any((c, d) != (a, b) and a <= c and d <= b for c, d in loops)]


def opcodes(body, a, b):
    ops = []
    for l in body[a:b]:
        t = l.strip().split()
        if t and not t[0].startswith((";", ".", "#")) and not t[0].endswith(":"):
            ops.append(t[0])
    return ops


CASES = [
    # configuration 3: f64, 64 x 64 tile, K tiles of 8, ring of 4, row-contiguous operands, K a multiple of the K tile
    ("contract_f64", "_ZN5hiptk18contract_wd_kernelINS_10WTraitsF64ELi8ELi4ELb0ELb0ELb0ELb0EEEvNS_5KArgsE", 4 * 8),
    # configuration 4: complex f32, the same geometry (four k-steps a tile, four MFMAs per complex product)
    ("contract_c32", "_ZN5hiptk18contract_wd_kernelINS_10WTraitsC32ELi8ELi8ELb0ELb0ELb0ELb0EEEvNS_5KArgsE", 8 * 4 * 4),
    # configuration 2: f16, 256 x 256 tile, both operands row-contiguous, one K stride
    ("contract_f16_hd", "_ZN5hiptk18contract_hd_kernelINS_9TraitsF16ELb0ELb0ELi256ELb1EEEvNS_5KArgsE", 128),
]


@pytest.mark.parametrize("unit,symbol,mfmas", CASES, ids=[c[0] for c in CASES])
def test_main_loop_is_mfma_loads_and_scalar_only(tmp_path, unit, symbol, mfmas):
    body = kernel_body(device_asm(unit, tmp_path), symbol)
    loops = main_loops(body, mfmas)
    assert loops, "no loop with %d MFMAs found: the ring is no longer unrolled as one loop" % mfmas
    for a, b in loops:
        ops = opcodes(body, a, b)
        assert sum(o.startswith("v_mfma") for o in ops) == mfmas, (a, b, sum(o.startswith("v_mfma") for o in ops))
        valu = sorted({o for o in ops if o.startswith("v_") and not o.startswith("v_mfma")})
        assert not valu, f"vector ALU instructions in the main loop of {symbol}: {valu}"
        assert not any(o.startswith(("s_cbranch", "s_branch")) for o in ops), "a branch inside the main loop"
        assert not any(o.startswith(("scratch_", "buffer_store", "global_store")) for o in ops), "stores or spills in the main loop"


@pytest.mark.parametrize("unit", ["contract_f32", "contract_f64", "contract_c32", "contract_c64"])
def test_every_32_64_bit_direct_load_instantiation(tmp_path, unit):
    """... and the same for every instantiation of the 32/64-bit direct-load kernel for K a multiple of the K tile
    (64 x 64 and 32 x 32 tiles, row- and k-contiguous operands): each has its ring unrolled as one clean loop."""
    lines = device_asm(unit, tmp_path)
    symbols = [l.split(":")[0] for l in lines if re.match(r"^_ZN5hiptk18contract_wd_kernel.*ELb0EEEvNS_5KArgsE:", l)]
    assert len(symbols) >= 2, symbols
    for symbol in symbols:
        body = kernel_body(lines, symbol)
        loops = main_loops(body, 16)
        assert loops, f"{symbol}: no main loop found"
        for a, b in loops:
            ops = opcodes(body, a, b)
            valu = sorted({o for o in ops if o.startswith("v_") and not o.startswith("v_mfma")})
            assert not valu, f"vector ALU instructions in the main loop of {symbol}: {valu}"
            assert not any(o.startswith(("s_cbranch", "s_branch", "scratch_")) for o in ops), symbol


@pytest.mark.parametrize("unit", ["contract_f16_hk_kx", "contract_f16_hk_rx", "contract_bf16_hk_kx", "contract_bf16_hk_rx"])
def test_16x16x32_direct_load_loops_hold_no_wait_states(tmp_path, unit):
    """The 16-bit kernels on v_mfma_f32_16x16x32 (K tiles of 64).  A 16-cycle MFMA leaves a single wave three issue
    slots, and s_nop N holds N + 1 of them, so the direct loads inside the loop are issued WITHOUT the wait states the
    load helper otherwise puts in front (they guard a scalar register written by a vector instruction, e.g. the
    reload of a spilled SGPR, being read by the load within 5 wait states; one such read of a stale address faulted
    the device once).  That is safe only while the loop holds no vector instruction that writes a scalar register
    and nothing but these helpers writes M0: both are checked here, for every wave position's copy of the loop of every
    instantiation, beside what the other main loops are held to."""
    lines = device_asm(unit, tmp_path)
    symbols = [l.split(":")[0] for l in lines if re.match(r"^_ZN5hiptk18contract_hk_kernel.*EvNS_5KArgsE:", l)]
    assert len(symbols) == 2, symbols
    for symbol in symbols:
        body = kernel_body(lines, symbol)
        # two K tiles of 2 x 64 MFMAs: the rings' common period (the epilogue's loops, which enclose the K tail's MFMAs, are longer)
        loops = [(a, b) for a, b in main_loops(body, 256) if len(opcodes(body, a, b)) < 1024]
        assert len(loops) == 4, f"{symbol}: {len(loops)} main loops (one per wave position expected)"
        for a, b in loops:
            ops = opcodes(body, a, b)
            assert sum(o.startswith("v_mfma_f32_16x16x32") for o in ops) == 256, symbol
            valu = sorted({o for o in ops if o.startswith("v_") and not o.startswith("v_mfma")})
            assert not valu, f"vector ALU instructions in the main loop of {symbol}: {valu}"
            assert not any(o.startswith(("s_cbranch", "s_branch", "scratch_", "buffer_store", "global_store")) for o in ops), symbol
            # (the first load of a window keeps its wait states: one s_nop per K tile in one wave position's copy, where the
            # compiler adds an s_nop 0 of its own in front of the next write of M0)
            assert sum(o == "s_nop" for o in ops) <= 4, f"{symbol}: s_nop in the main loop"
            assert sum(o == "global_load_lds_dwordx4" for o in ops) == 32, symbol
            # M0 is written by the load helpers' s_add_u32 only, once per four loads (which reach consecutive KiB of LDS
            # through their offset fields), in front of the MFMA before the first of them
            text = [l for l in body[a:b] if "m0" in l.split(";")[0]]
            assert len(text) == 8 and all(l.strip().startswith("s_add_u32 m0,") for l in text), text[:5]
            offs = sorted({int(m.group(1), 0) for l in body[a:b] for m in [re.search(r"global_load_lds_dwordx4 .*offset:(0x[0-9a-f]+|\d+)", l)] if m})
            assert offs == [0, 1024, 2048, 3072], offs
            # instructions beside the MFMAs: fewer than three per MFMA on average
            assert len(ops) - 256 < 3 * 256 // 2, f"{symbol}: {len(ops) - 256} instructions beside 256 MFMAs"
            # ... and no more than three between two MFMAs (a fourth delays the MFMA behind it): the scalar arithmetic that
            # opens a tile's window of loads is spread over four MFMAs, and M0 for the load right behind a barrier is written
            # in front of the barrier, for that.  (The first MFMA of the period may have four in front of it, and the two
            # behind a barrier, which wait anyway, five, the wait and the barrier included.)
            gaps, run = [], []
            for o in ops:
                if o.startswith("v_mfma"):
                    gaps.append(run)
                    run = []
                else:
                    run.append(o)
            plain = [len(g) for g in gaps if "s_barrier" not in g]
            assert max(plain) <= 4 and sum(n == 4 for n in plain) <= 1, (symbol, [g for g in gaps if len(g) > 3])
            assert all(len(g) <= 5 for g in gaps), (symbol, [g for g in gaps if len(g) > 5])


@pytest.mark.parametrize("unit", ["contract_f16_hr192_kx", "contract_f16_hr192_rx", "contract_bf16_hr192_kx", "contract_bf16_hr192_rx"])
def test_ring_kernel_loops(tmp_path, unit):
    """The 16-bit kernel on v_mfma_f32_16x16x32 that loads K tiles of 32 into a ring of four stages and reads its k
    offsets from tables.  Its loads are issued without wait states too; its loop does hold vector ALU instructions
    (they turn table entries into load offsets), so the check is that none of them writes a scalar register.  Every
    barrier of the loop must directly follow the wait for the loads of the tile after next AND for the wave's own LDS
    reads (the stage those reads came from is overwritten after the barrier)."""
    lines = device_asm(unit, tmp_path)
    symbols = [l.split(":")[0] for l in lines if re.match(r"^_ZN5hiptk18contract_hr_kernel.*EvNS_5KArgsE:", l)]
    assert len(symbols) == 2, symbols
    for symbol in symbols:
        body = kernel_body(lines, symbol)
        # four K tiles of 48 MFMAs: the period of the ring, the table slots and the offset sets
        loops = [(a, b) for a, b in main_loops(body, 192) if len(opcodes(body, a, b)) < 1024]
        assert len(loops) == 4, f"{symbol}: {len(loops)} main loops (one per wave position expected)"
        for a, b in loops:
            ops = opcodes(body, a, b)
            assert sum(o.startswith("v_mfma_f32_16x16x32") for o in ops) == 192, symbol
            valu = sorted({o for o in ops if o.startswith("v_") and not o.startswith("v_mfma")})
            assert valu and all(o.startswith(("v_min_u32", "v_add_lshl_u32", "v_lshl_add_u32", "v_add_u32", "v_lshlrev_b32")) for o in valu), \
                f"vector ALU instructions in the main loop of {symbol}: {valu}"
            assert not any(o.startswith(("s_cbranch", "s_branch", "scratch_", "buffer_store", "global_store")) for o in ops), symbol
            # (the compiler puts one s_nop 0 per K tile in front of the table request's first write of M0)
            assert sum(o == "s_nop" for o in ops) <= 4, f"{symbol}: s_nop in the main loop"
            # seven loads of 16 bytes a lane and two of table entries per K tile, each with its own write of M0
            assert sum(o == "global_load_lds_dwordx4" for o in ops) == 28 and sum(o == "global_load_lds_dword" for o in ops) == 8, symbol
            text = [l for l in body[a:b] if "m0" in l.split(";")[0]]
            assert len(text) == 36 and all(l.strip().startswith("s_add_u32 m0,") for l in text), text[:5]
            code = [l.split(";")[0].strip() for l in body[a:b]]
            code = [l for l in code if l and not l.endswith(":") and not l.startswith(".")]
            bars = [i for i, l in enumerate(code) if l.startswith("s_barrier")]
            assert len(bars) == 4, symbol
            for i in bars:
                assert code[i - 1].startswith("s_waitcnt") and "vmcnt(20)" in code[i - 1] and "lgkmcnt(0)" in code[i - 1], \
                    f"{symbol}: '{code[i - 1]}' in front of a barrier of the main loop"
            # instructions beside the MFMAs: fewer than two per MFMA (a 16-cycle MFMA leaves the wave three issue slots)
            assert len(ops) - 192 < 2 * 192, f"{symbol}: {len(ops) - 192} instructions beside 192 MFMAs"
            # ... and never more than three in front of one MFMA (four where the period begins: the loop's own bookkeeping)
            gaps, run = [], []
            for o in ops:
                if o.startswith("v_mfma"):
                    gaps.append(run)
                    run = []
                else:
                    run.append(o)
            assert sum(len(g) > 3 for g in gaps) <= 1 and max(len(g) for g in gaps) <= 4, (symbol, [g for g in gaps if len(g) > 3])


def test_direct_load_loops_leave_m0_alone(tmp_path):
    """The 32 x 32 x 16 direct-load kernel writes M0 one MFMA ahead of the load that reads it, in separate asm
    statements: nothing the compiler generates in between may touch M0."""
    body = kernel_body(device_asm("contract_f16_hd", tmp_path), "_ZN5hiptk18contract_hd_kernelINS_9TraitsF16ELb0ELb0ELi256ELb1EEEvNS_5KArgsE")
    for a, b in main_loops(body, 128):
        text = [l for l in body[a:b] if "m0" in l.split(";")[0]]
        assert text and all(l.strip().startswith("s_add_u32 m0,") for l in text), text[:5]
