"""The hazards that `asm` statements hide from the compiler, re-checked on the generated gfx950
assembly (no GPU needed: hipcc cross-compiles)."""
import shutil

import pytest

from maester_amd import isa_check

FAULTY = """
_ZN2ma4demoEv: ; @demo
	;;#ASMSTART
	s_load_dwordx4 s[52:55], s[2:3], 0x0
	;;#ASMEND
	v_writelane_b32 v170, s52, 9
	;;#ASMSTART
	s_waitcnt lgkmcnt(0)
	;;#ASMEND
	;;#ASMSTART
	v_mfma_f32_32x32x16_bf16 v[0:15], v[16:19], a[0:3], v[0:15]
	;;#ASMEND
	v_add_f32_e32 v1, v1, v20
	s_endpgm
"""


def test_checker_flags_every_kind_of_hazard():
    bad, stats = isa_check.check_assembly(FAULTY)
    assert stats == {"_ZN2ma4demoEv": (1, 1)}
    assert len(bad) == 2 and "load in flight" in bad[0] and "MFMA result" in bad[1]
    clean = FAULTY.replace("\tv_writelane_b32 v170, s52, 9\n", "").replace("\tv_add_f32_e32 v1, v1, v20\n", "\ts_nop 15\n\tv_add_f32_e32 v1, v1, v20\n")
    assert isa_check.check_assembly(clean)[0] == []
    # an operand copied into place right in front of the asm MFMA that reads it
    copied = clean.replace("\t;;#ASMSTART\n\tv_mfma", "\tv_accvgpr_write_b32 a1, v40\n\t;;#ASMSTART\n\tv_mfma")
    bad = isa_check.check_assembly(copied)[0]
    assert len(bad) == 1 and "written by the vector ALU" in bad[0]
    padded = copied.replace("\tv_accvgpr_write_b32 a1, v40\n", "\tv_accvgpr_write_b32 a1, v40\n\ts_nop 1\n")
    assert isa_check.check_assembly(padded)[0] == []


@pytest.mark.skipif(shutil.which("hipcc") is None, reason="hipcc not installed")
def test_generated_assembly_of_the_attention_kernels_is_hazard_free():
    res = {}
    bad, stats = isa_check.check_all(resources=res)
    assert not bad, "\n".join(bad[:20])
    # every bf16 attention kernel went through the checker, and its asm MFMAs were seen
    # (three head dims x with / without document ids; the pair forward and the dK/dV kernel also with plain or
    # descriptor tile loads, the dK/dV kernel with / without the dS hand-over)
    for kernel, count in (("attn_fwd_bf16_kernel", 6), ("attn_fwd_pair_bf16_kernel", 12), ("attn_bwd_dq_bf16_kernel", 6),
                          ("attn_bwd_dq_ds_bf16_kernel", 6), ("attn_bwd_dkv_bf16_kernel", 24)):
        hits = [v for k, v in stats.items() if kernel in k]
        assert len(hits) == count and all(n_mfma > 0 for n_mfma, _ in hits), (kernel, hits)
    # The register budget the kernels are written around: no vector register of any bf16 attention kernel spills
    # (a spill inside an MFMA chain costs whole factors and no numerics test would notice), the D = 256 kernels
    # that hold two heads' accumulators use the whole file (all 256 accumulation registers), and the scalar
    # registers spilled to vector lanes stay within what the step loops were tuned with.
    attn = {k: v for k, v in res.items() if "attn_" in k and "bf16" in k}
    assert len(attn) >= 60, len(attn)
    assert all(v["vgpr_spill"] == 0 for v in attn.values()), {k: v["vgpr_spill"] for k, v in attn.items() if v["vgpr_spill"]}
    assert all(v["sgpr_spill"] <= 80 for v in attn.values()), {k: v["sgpr_spill"] for k, v in attn.items() if v["sgpr_spill"] > 80}
    for kernel in ("attn_fwd_pair_bf16_kernelILi256E", "attn_bwd_dkv_bf16_kernelILi256E", "attn_bwd_dq_ds_pair_bf16_kernelILi256E"):
        hits = [v for k, v in attn.items() if kernel in k]
        assert hits and all(v["agpr"] == 256 and v["vgpr"] <= 512 for v in hits), (kernel, hits)
