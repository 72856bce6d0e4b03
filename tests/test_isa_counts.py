"""The step-by-step form of the staged GEMV waits for its loads by count (s_waitcnt vmcnt(N) with N worked out by
hand from the order the loads are issued in).  The compiler is free to restructure branches around the load-to-LDS
instructions -- it once threaded four equal lane-mask conditions into one divergent branch and issued the weight loads
in between once per side, two more loads than the waits counted, a silent race between 5 and 15 rows.  This test
compiles the kernel file to gfx950 assembly (no GPU needed) and counts the load-to-LDS instructions of every
instantiation: 14 per chunk issue (1 or 4 of x sharing their first instruction, 8 of weights, 2 of zeros/scales)."""
import os
import re
import shutil
import subprocess

import pytest

from nanoquantization_amd import build as nq_build


@pytest.mark.skipif(shutil.which(nq_build.HIPCC) is None and not os.path.exists(nq_build.HIPCC), reason="hipcc not found")
def test_staged_gemv_issues_each_load_once(tmp_path):
    src = os.path.join(nq_build.CSRC, "awq_gemv.hip")
    out = tmp_path / "awq_gemv.s"
    flags = [f for f in nq_build.FLAGS if f not in ("-shared", "-fPIC")]
    cmd = [nq_build.HIPCC, *flags, *nq_build.EXTRA.get("awq_gemv.hip", []), "--cuda-device-only", "-S", src, "-o", str(out)]
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    assert proc.returncode == 0, proc.stdout[-2000:]
    asm = out.read_text()
    names = re.findall(r"^(_ZN3awq15gemv_dma_kernel[^:\s]*):", asm, re.M)
    assert len(names) >= 32, names            # 2 types x 2 wave counts x the forms
    seen_stream = seen_chunked = 0
    for name in names:
        begin = asm.index("\n" + name + ":")
        body = asm[begin:asm.index(".Lfunc_end", begin)]
        loads = len(re.findall(r"\bglobal_load_lds_dword", body))
        # template arguments: <T, WK, MODE, STREAM>; the mangled name spells STREAM as Lb1 / Lb0
        stream = re.search(r"ELi\dELi\dELb(\d)", name).group(1) == "1"
        if stream:
            assert loads == 14, (name, loads)      # issued once: the wave has one chunk
            seen_stream += 1
        else:
            assert loads == 28, (name, loads)      # the first chunk's issue and the one in the loop
            seen_chunked += 1
    assert seen_stream >= 10 and seen_chunked >= 10
    # The shared-chunk kernel with three staging buffers counts too.  Per issue site a wave runs 4 weight loads, its x
    # load (one m-tile: one piece, brought by waves 0..3) and one of the two zero/scale loads; the two byte-half paths of
    # the kernel keep their own weight loads and share the zero/scale block -- and the x load where only some waves
    # run it (512 columns: 8 + 1 + 2 instructions per site; 256 columns: 8 + 2 + 2; 256 columns and two m-tiles:
    # 8 + 4 + 2), DEPTH sites.
    wide = re.findall(r"^(_ZN3awq16gemv_wide_kernel[^:\s]*):", asm, re.M)
    deep = [n for n in wide if re.search(r"ELi3ELi[12]ELb[01]ELi[24]E", n)]
    assert len(deep) == 10, wide              # 2 types x ((second pass, in-kernel tail) x (512, 256 columns) + 256 columns x two m-tiles)
    for name in deep:
        begin = asm.index("\n" + name + ":")
        body = asm[begin:asm.index(".Lfunc_end", begin)]
        loads = len(re.findall(r"\bglobal_load_lds_dword", body))
        if re.search(r"ELi3ELi2E", name):      # two m-tiles on 256 columns: two x pieces per wave on either path
            per_site = 8 + 4 + 2
        else:
            per_site = 11 if re.search(r"ELb[01]ELi4E", name) else 12
        assert loads == 3 * per_site, (name, loads)
    # The 16-byte publish store is issued as assembly (publish_f32x4), out of sight of the compiler's hazard pass: a
    # store of more than 8 bytes reads its data registers up to two wait states after it issues (gfx940 and later),
    # and the compiler, to which those registers are free at once, has put the next address computation into them one
    # instruction later -- the store then published that value now and then.  Every such store carries its own two
    # wait states.
    stores = [m.end() for m in re.finditer(r"global_store_dwordx4 [^\n]* sc1\n", asm)]
    assert len(stores) >= 50, len(stores)
    for pos in stores:
        assert re.match(r"\s*s_nop 1\b", asm[pos:pos + 40]), asm[pos - 80:pos + 80]
    # The 16-byte fetches of the exchange are assembly too (fetch_f32x4_nowait) and arrive behind the compiler's back:
    # until the s_waitcnt vmcnt(0) that the code issues by hand, nothing may touch their destination registers -- a
    # copy or a select placed there by the compiler would read what the registers held before.  (A linear scan of the
    # listing: the fetch sites are straight-line code up to their wait.)
    def vregs(text):
        regs = set()
        for m in re.finditer(r"\bv\[(\d+):(\d+)\]", text):
            regs |= set(range(int(m.group(1)), int(m.group(2)) + 1))
        regs |= {int(m.group(1)) for m in re.finditer(r"\bv(\d+)\b", text)}
        return regs
    pending, fetches = set(), 0
    for line in asm.split("\n"):
        line = line.strip()
        if not line or line[0] in ";." or line.endswith(":"):
            continue
        if line.startswith("s_waitcnt") and "vmcnt(0)" in line:
            pending = set()
            continue
        m = re.match(r"global_load_dwordx4 (v\[\d+:\d+\]), (v\[\d+:\d+\]), off sc1", line)
        if m:
            assert not (vregs(m.group(2)) & pending), line
            pending |= vregs(m.group(1))
            fetches += 1
            continue
        if pending and line.split()[0].startswith(("v_", "ds_", "global_", "buffer_")):
            assert not (vregs(line.split(None, 1)[1] if " " in line else "") & pending), line
    assert fetches >= 500, fetches


@pytest.mark.skipif(shutil.which(nq_build.HIPCC) is None and not os.path.exists(nq_build.HIPCC), reason="hipcc not found")
def test_matrix_core_attention_counts_its_tile_loads(tmp_path):
    """paged_attn_decode_tr_kernel brings a K tile and a V tile with eight load-to-LDS instructions each and reads the
    K tile after s_waitcnt vmcnt(8): the eight loads of the V tile may still be on their way, nothing else.  Every
    instantiation must issue exactly those sixteen loads, in one run with no other vector-memory instruction among them,
    and wait by that count right behind them."""
    src = os.path.join(nq_build.CSRC, "nq_decode_ops.hip")
    out = tmp_path / "nq_decode_ops.s"
    flags = [f for f in nq_build.FLAGS if f not in ("-shared", "-fPIC")]
    cmd = [nq_build.HIPCC, *flags, *nq_build.EXTRA.get("nq_decode_ops.hip", []), "--cuda-device-only", "-S", src, "-o", str(out)]
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    assert proc.returncode == 0, proc.stdout[-2000:]
    asm = out.read_text()
    names = re.findall(r"^(_ZN3awq\S*paged_attn_decode_tr_kernel[^:\s]*):", asm, re.M)
    assert len(names) == 4, names             # 2 types x (8 heads per kv head at compile time, the count at run time)
    for name in names:
        begin = asm.index("\n" + name + ":")
        body = asm[begin:asm.index(".Lfunc_end", begin)]
        ins = [l.strip() for l in body.split("\n")]
        ins = [l for l in ins if l and l[0] not in ";." and not l.endswith(":")]
        dma = [k for k, l in enumerate(ins) if "global_load_lds_dwordx4" in l]
        assert len(dma) == 16, (name, len(dma))
        assert ins[dma[-1] + 1].startswith("s_waitcnt vmcnt(8)"), (name, ins[dma[-1] + 1])
        between = [l for l in ins[dma[0]:dma[-1]] if l.split()[0].startswith(("global_", "buffer_", "flat_"))]
        assert len(between) == 15, (name, between)
