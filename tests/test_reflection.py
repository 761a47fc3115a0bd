"""Codegen checks on the compiled kernels (no GPU needed): the analogue of the reference's PTX
string matches, test/device/wmma.jl:254-291 (store_d on a Global / Shared pointer must emit the
.global. / .shared. instruction variants, not generic ones), plus resource usage of the GEMM."""
import collections
import re


def _ops(text):
    return collections.Counter(l.split()[0] for l in text.splitlines()
                               if l.strip() and not l.strip().startswith(("<", ";")))


def test_store_d_addressing(miw):
    for T in ("float", "_Float16"):
        isa = miw.reflection.code_gcn(f"k_frag_store<{T}>")
        assert len(isa) == 1
        ops = _ops(next(iter(isa.values())))
        assert any(o.startswith("ds_write") for o in ops)          # LDS pointer overload -> ds_write
        assert any(o.startswith("global_store") for o in ops)      # global pointer -> global_store
        assert not any(o.startswith(("flat_store", "scratch_")) for o in ops)


def test_load_addressing(miw):
    for T in ("float", "_Float16"):
        isa = miw.reflection.code_gcn(f"k_frag_load<{T}>")
        assert len(isa) == 1
        ops = _ops(next(iter(isa.values())))
        assert any(o.startswith("ds_read") for o in ops) and any(o.startswith("global_load") for o in ops)
        assert not any(o.startswith(("flat_load", "scratch_")) for o in ops)


def test_fragment_mma_uses_the_16x16x16_matrix_instruction(miw):
    isa = miw.reflection.code_gcn("k_frag_mma<float, float>")
    assert _ops(next(iter(isa.values())))["v_mfma_f32_16x16x16_f16"] == 1


def test_default_gemm_kernel_codegen_and_resources(miw):
    name = "k_gemm_pp<256, 256, 2, 4, false, true, float, float>"    # column-major A and B: the benchmark's kernel
    isa = miw.reflection.code_gcn(name)
    assert len(isa) == 1
    ops = _ops(next(iter(isa.values())))
    assert ops["v_mfma_f32_16x16x32_f16"] >= 64                  # two unrolled clusters of 8 x 4 tiles
    assert ops["global_load_lds_dwordx4"] >= 8                   # direct-to-LDS operand loads
    assert ops["ds_read_b64_tr_b16"] >= 16 and ops["ds_read_b128"] >= 4   # transpose reads for A, b128 for B
    assert not any(o.startswith(("scratch_", "flat_", "ds_write", "v_accvgpr")) for o in ops)
    res = {k: v for k, v in miw.reflection.kernel_resources().items() if name in k}
    (r,) = res.values()
    assert r["spills"] == 0 and r["scratch"] == 0 and r["max_threads"] == 512
    assert r["vgpr"] + r["agpr"] <= 256                          # two wavefronts per SIMD
    # both operands K-major: no transpose read at all
    kk = miw.reflection.code_gcn("k_gemm_pp<256, 256, 2, 4, true, true, float, float>")
    assert "ds_read_b64_tr_b16" not in _ops(next(iter(kk.values())))


def test_auto_picked_4096_kernels_have_no_spills(miw):
    """The kernels miw_gemm picks by itself for a 4096^3 problem, one per operand layout: the 256 x 256
    ping-pong kernel.  None of them may touch scratch memory, and all fit two wavefronts per SIMD."""
    res = miw.reflection.kernel_resources()
    picked = ["k_gemm_pp<256, 256, 2, 4, %s, float, float>" % l for l in ("true, false", "false, true", "false, false", "true, true")]
    for name in picked:
        (r,) = [v for k, v in res.items() if name in k]
        assert r["spills"] == 0 and r["scratch"] == 0 and r["vgpr"] + r["agpr"] <= 256 and r["max_threads"] == 512, name
    # and no ping-pong kernel of any tile, layout or type spills
    for k, r in res.items():
        if "k_gemm_pp" in k:
            assert r["spills"] == 0 and r["scratch"] == 0, k


def test_tiled_kernels_keep_spills_out_of_the_steady_state(miw):
    """The rolled K loop (the two pipeline steps up to the backward branch) never touches scratch
    memory; the unrolled trips that fold C in may hold a few spills in one operand layout."""
    for name, text in miw.reflection.code_gcn("k_gemm_tiled<").items():
        lines = [l for l in text.splitlines() if l.strip() and not l.strip().startswith(("<", ";"))]
        mfma = [i for i, l in enumerate(lines) if "v_mfma" in l]
        assert mfma, name
        # the first backward branch after the first MFMA (conditional, or unconditional where the compiler
        # rotated the loop) closes the rolled loop: a 16-bit word offset >= 0x8000
        back = next(i for i, l in enumerate(lines) if i > mfma[0] and
                    (m := re.match(r"\s*s_c?branch\w* (\d+)", l)) and int(m.group(1)) >= 0x8000)
        per_trip = sum(1 for i in mfma if i < back)
        body = lines[mfma[0]:back]          # no MFMA precedes the loop: this is its body
        assert per_trip >= 2 and not [l for l in body if re.match(r"\s*scratch_", l)], name
        if "256, 256, 2, 2, 2" in name:
            continue    # 256 accumulators per lane: the 4-wavefront tile spills around its loop
        assert sum(1 for l in lines[mfma[0]:mfma[-1]] if re.match(r"\s*scratch_", l)) <= 48, name


def _regs(tok):
    """Registers named by one operand: 'v12' -> {('v', 12)}, 'a[4:7]' -> {('a', 4) .. ('a', 7)}."""
    m = re.fullmatch(r"([va])(\d+)", tok)
    if m:
        return {(m.group(1), int(m.group(2)))}
    m = re.fullmatch(r"([va])\[(\d+):(\d+)\]", tok)
    if m:
        return {(m.group(1), i) for i in range(int(m.group(2)), int(m.group(3)) + 1)}
    return set()


def test_wave128_kernels_keep_the_matrix_instruction_hazards(miw):
    """The one-wavefront-per-SIMD GEMM kernel writes its MFMAs as inline assembly (accumulators in
    AGPRs), so the compiler does not keep the distances the hardware asks for around them.  Checked
    here on the built code of every instance: no MFMA reads a register that a VALU instruction
    (a copy the register allocator placed, an address addition) wrote less than two wait states
    before it; no accumulator is copied out of its AGPR less than 18 wait states behind the MFMA
    that wrote it; the rolled K loops hold neither such copies nor scratch traffic; the accumulators
    fill the AGPRs and the kernel runs one wavefront per SIMD."""
    isa = miw.reflection.code_gcn("k_gemm_w128<")
    assert len(isa) == 16                                       # four layouts x C type x D type
    res = miw.reflection.kernel_resources()
    for name, text in isa.items():
        lines = [l.split("//")[0].strip() for l in text.splitlines()]
        lines = [l for l in lines if l and not l.startswith(("<", ";"))]
        ops = [l.replace(",", " ").split() for l in lines]
        mfma = [i for i, o in enumerate(ops) if o[0].startswith("v_mfma")]
        assert len(mfma) >= 7 * 64, name                        # the unrolled steps of 8 x 8 tiles
        for i in mfma:
            assert ops[i][1].startswith("a[") and ops[i][4] == ops[i][1], (name, lines[i])
            sources = _regs(ops[i][2]) | _regs(ops[i][3]) | _regs(ops[i][4])
            wait, j = 0, i - 1
            while wait < 2 and j >= 0:
                o = ops[j]
                if o[0] == "s_nop":
                    wait += int(o[1]) + 1
                else:
                    if o[0].startswith("v_") and not o[0].startswith("v_mfma"):
                        assert not (_regs(o[1]) & sources), (name, lines[j], lines[i])
                    assert not o[0].startswith(("s_cbranch", "s_branch", "s_endpgm")), (name, lines[j], lines[i])
                    wait += 1
                j -= 1
        for i, o in enumerate(ops):
            if o[0] in ("v_accvgpr_read_b32", "v_accvgpr_mov_b32"):
                src = _regs(o[2])
                wait, j = 0, i - 1
                while wait < 18 and j >= 0:
                    p = ops[j]
                    if p[0] in ("s_branch", "s_endpgm", "s_setpc_b64"):
                        break                                   # no fall-through: what precedes in the listing does not run before
                    if p[0] == "s_nop":
                        wait += int(p[1]) + 1
                    else:
                        assert not (p[0].startswith("v_mfma") and _regs(p[1]) & src), (name, lines[j], lines[i])
                        wait += 1
                    j -= 1
        # the rolled loops: from the target of every backward branch to the branch
        back = [i for i, o in enumerate(ops) if re.match(r"s_c?branch", o[0]) and o[1].isdigit() and int(o[1]) >= 0x8000]
        k_loops = 0
        for b in back:
            body, words = [], 65536 - int(ops[b][1]) - 1
            j = b - 1
            while words > 0 and j >= 0:                         # (MFMAs, loads and reads are two words, most scalar instructions one)
                body.append(ops[j][0])
                words -= 1 if ops[j][0].startswith(("s_", "v_add", "v_mov", "v_and")) and "0x" not in lines[j] else 2
                j -= 1
            if not any(o.startswith("v_mfma") for o in body):
                continue                                        # (a loop of the epilogue)
            k_loops += 1
            assert sum(o.startswith("v_mfma") for o in body) >= 96, (name, len(body))
            assert not [o for o in body if o.startswith(("scratch_", "v_accvgpr"))], name
        assert k_loops == 2, name                               # the loop with the short pointer bookkeeping and the general one
        (r,) = [v for k, v in res.items() if name in k]
        assert r["agpr"] == 256 and r["max_threads"] == 256, name
