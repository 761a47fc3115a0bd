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
