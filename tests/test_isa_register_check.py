"""The build checks the compiler's assembly of every kernel for registers that are read and never written
(nnlib.jl_amd/csrc/check_isa_registers.py; the Makefile runs it on each object).  These cases pin the checker itself on
hand-written fragments: the miscompile it exists for (a matrix operand a[156:159] of which only a[156:158] is
reloaded), destinations it must recognise (loads, cross-lane reads, matrix results), and the registers the hardware
initialises."""
import importlib.util
import os

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
spec = importlib.util.spec_from_file_location("check_isa_registers", os.path.join(ROOT, "nnlib.jl_amd", "csrc", "check_isa_registers.py"))
chk = importlib.util.module_from_spec(spec)
spec.loader.exec_module(chk)

HEAD = "\t.text\n\t.globl\tkern\nkern:\n"
TAIL = "\ts_endpgm\n\t.section\t.rodata,\"a\",@progbits\n\t.amdhsa_kernel kern\n\t.end_amdhsa_kernel\n"


def run(tmp_path, body):
    f = tmp_path / "k.s"
    f.write_text(HEAD + body + TAIL)
    return chk.check(str(f))


def test_partial_reload_is_found(tmp_path):
    body = ("\tds_read_b128 v[10:13], v0\n"
            "\tv_accvgpr_write_b32 a171, v13           ;  Reload Reuse\n"
            "\tscratch_load_dwordx3 a[156:158], off, off ; 12-byte Folded Reload\n"
            "\tv_accvgpr_write_b32 a56, v1\n"
            "\tv_mfma_f32_32x32x16_bf16 a[56:71], v[10:13], a[156:159], a[56:71]\n"
            "\tv_accvgpr_read_b32 v20, a60\n"
            "\tglobal_store_dword v[10:11], v20, off\n")
    found = run(tmp_path, body)
    assert any("a159" in f for f in found), found
    # a57 .. a71 are never written before the matrix instruction reads them as its accumulator input either
    assert all(("a159" in f) or any(f"a{i} " in f for i in range(57, 72)) for f in found), found


def test_clean_kernel_passes(tmp_path):
    body = ("\tv_lshlrev_b32_e32 v3, 2, v0\n"                       # v0: work-item id, set by the hardware
            "\tds_read_b128 v[10:13], v3\n"
            "\tds_read_b64_tr_b16 v[14:15], v3 offset:64\n"
            "\tds_bpermute_b32 v16, v3, v10\n"
            "\tscratch_load_dwordx4 a[0:3], off, off\n"
            "\tv_accvgpr_mov_b32 a4, a0\n"
            "\tv_mov_b32_e32 v17, 0\n"
            "\tv_mov_b32_e32 v18, 0\n"
            "\tv_mov_b32_e32 v19, 0\n"
            "\tv_mov_b32_e32 v20, 0\n"
            "\tv_mfma_f32_16x16x32_bf16 v[17:20], v[10:13], a[0:3], v[17:20]\n"
            "\tv_add_f32_e32 v21, v16, v14\n"
            "\tv_add_f32_e32 v21, v21, v15\n"
            "\tv_accvgpr_read_b32 v22, a4\n"
            "\tglobal_store_dwordx4 v[10:11], v[17:20], off\n"
            "\tglobal_store_dwordx2 v[10:11], v[21:22], off\n")
    assert run(tmp_path, body) == []


def test_two_kernels_are_checked_apart(tmp_path):
    f = tmp_path / "two.s"
    f.write_text(HEAD + "\tv_mov_b32_e32 v5, 1\n\tglobal_store_dword v[0:1], v5, off\n" + TAIL
                 + "\t.globl\tother\nother:\n\tglobal_store_dword v[0:1], v5, off\n\ts_endpgm\n\t.amdhsa_kernel other\n\t.end_amdhsa_kernel\n")
    found = chk.check(str(f))
    assert len(found) == 1 and "other" in found[0] and "v5" in found[0], found
