"""Host logic of the HIP backend that runs without a GPU: the library loads, exports every symbol the headers
declare, and turns the reference's define blocks into the kernels the reference's callers then ask for by name."""
import ctypes
import os
import re

import pytest

import qwental_amd as q
from qwental_amd.gpu import SYMBOLS, compile_check

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_functions():
    names = set()
    for h in ("gpu.h", "qw_hip_ext.h", "qw_path.h", "qw_gguf.h", "qw_par.h"):
        text = open(os.path.join(ROOT, "include", h)).read()
        text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
        names |= set(re.findall(r"\b(qw_[a-z0-9_]+)\s*\(", text))
    return names


def test_library_exports_every_declared_symbol():
    L = q.load_lib()
    decl = declared_functions()
    assert len(decl) >= 55
    for n in decl:
        assert hasattr(L, n), "libqwgpu_hip.so lacks %s" % n
    assert decl == {n for n, _, _ in SYMBOLS}  # the ctypes table covers exactly what the headers declare


def test_reference_interface_symbols_present():
    """The 33 functions of the reference's src/gpu.h, by name."""
    ref = """qw_gpu_open qw_gpu_close qw_gpu_name qw_gpu_max_working_set qw_gpu_compile qw_kernel_get qw_kernel_max_threads
    qw_kernel_simd_width qw_buf_new qw_buf_free qw_pool_push qw_pool_pop qw_buf_wrap qw_batch_begin qw_batch_kernel qw_batch_buf
    qw_batch_bytes qw_batch_threadgroup_mem qw_batch_dispatch qw_batch_barrier qw_batch_flush qw_batch_end qw_batch_submit
    qw_batch_wait qw_batch_poll qw_gpu_set_stream qw_profile_enable qw_profile_count qw_profile_get qw_gpu_empty_commit_latency
    qw_power_desc qw_on_battery qw_now""".split()
    L = q.load_lib()
    for n in ref:
        assert hasattr(L, n)
    L.qw_now.restype = ctypes.c_double
    t0 = L.qw_now()
    assert L.qw_now() >= t0 > 0
    buf = ctypes.create_string_buffer(128)
    L.qw_power_desc(buf, 128)
    assert buf.value and not L.qw_on_battery()
    assert L.qw_pool_push() is None and q.load_lib().qw_hip_arch() == b"gfx950"


def test_no_device_is_reported_not_emulated():
    """Without a gfx950 device qw_gpu_open returns NULL and the Python wrapper raises: there is no CPU path."""
    L = q.load_lib()
    if L.qw_gpu_open():
        pytest.skip("a device is present")
    with pytest.raises(RuntimeError):
        q.Gpu()


ENGINE_MOE = "#define IQ_DQ_ONLY\n#define E 512\n#define TOPK 10\n#define D 2048\n#define I 512\n#define NB %d\n"  # src/engine.c:478


def test_define_blocks_of_the_reference_register_its_kernel_names():
    ok, err, names = compile_check("#define IQ_DQ_ONLY 1\n#define DQ_TEST 21\n// kernel text follows\n")  # tools/dqtest.c:27
    assert ok and names == ["dq_test"]
    blk = "#define IQ_DQ_ONLY 1\n#define qmv_gg qmv_gg_f21_k2048_n8_f\n#define GF 21\n#define KD 2048\n#define RB 880\n#define NB 8\n#define YT float\n"
    ok, err, names = compile_check(blk + "#include <metal_stdlib>\nkernel void qmv_gg(...)")  # src/engine.c:709-710
    assert ok and names == ["qmv_gg_f21_k2048_n8_f"]
    ok, err, names = compile_check(ENGINE_MOE % 8 + "#define GG_PART 0\n#define moe_sel_gg moe_sel_gg_n8\n#define gg_tab_init gg_tab_init_n8\n")
    assert ok and names == ["gg_tab_init_n8", "moe_sel_gg_n8"]
    ok, err, names = compile_check(ENGINE_MOE % 8 + "#define GG_PART 1\n#define FSG 21\n#define FSU 21\n#define RBF 1\n#define moe_pre_gg moe_pre_gg_21_21_r1_n8\n")
    assert ok and names == ["moe_pre_gg_21_21_r1_n8"]
    ok, err, names = compile_check(ENGINE_MOE % 4 + "#define GG_PART 2\n#define GSG 8\n#define RG 1\n#define FGU 21\n#define FSD 8\n#define moe_gu_gg moe_gu_gg_21_8_g1_n4\n")
    assert ok and names == ["moe_gu_gg_21_8_g1_n4"]
    ok, err, names = compile_check(ENGINE_MOE % 1 + "#define GG_PART 3\n#define FD 21\n#define DSGN 4\n#define moe_dn_gg moe_dn_gg_21_s4_n1\n#define moe_cmb_gg moe_cmb_gg_21_s4_n1\n")
    assert ok and names == ["moe_dn_gg_21_s4_n1", "moe_cmb_gg_21_s4_n1"]
    ok, err, names = compile_check(ENGINE_MOE % 3 + "#define GG_ROUTER\n#define moe_router_bf moe_router_bf_n3\n#define p_router_bf p_router_bf_n3\n")
    assert ok and names == ["moe_router_bf_n3"]  # the prefill routers have no gfx950 build: not registered, lookup gives NULL
    ok, err, names = compile_check(ENGINE_MOE % 16 + "#define GG_PART 0\n#define moe_sel_gg s16\n#define gg_tab_init t16\n")  # beyond the reference: 16 tokens
    assert ok and names == ["t16", "s16"]
    ok, err, names = compile_check("#include <metal_stdlib>\nkernel void something_else() {}\n")
    assert ok and names == []  # a source with no known block compiles to nothing; qw_kernel_get then returns NULL


@pytest.mark.parametrize("block,needle", [
    ("#define IQ_DQ_ONLY 1\n#define DQ_TEST 10\n", "10"),                                                    # Q2_K: no gfx950 build
    ("#define qmv_gg x\n#define GF 14\n#define KD 8192\n#define RB 6720\n#define NB 8\n", "8192"),            # K beyond the staged activations
    ("#define qmv_ggm g\n#define KD 2048\n#define NB 0\n#define NMAT 2\n#define GF0 12\n#define GF1 21\n", "21"),  # IQ3_S is not a format of the multi-matrix kernel
    ("#define qmv_ggm g\n#define KD 2000\n#define NB 0\n#define NMAT 1\n#define GF0 12\n", "KD 2000"),
    ("#define qmv_ggm g\n#define KD 2048\n#define NB 0\n#define NMAT 5\n#define GF0 12\n", "NMAT"),
    ("#define qmv_gg x\n#define GF 21\n#define KD 2048\n#define RB 881\n#define NB 8\n", "row bytes"),
    ("#define qmv_gg x\n#define GF 21\n#define KD 2048\n#define RB 880\n#define NB 17\n", "NB"),
    ("#define qmv_gg x\n#define GF 21\n#define KD 2048\n#define RB 880\n#define NB 8\n#define YT bfloat\n", "YT"),
    (ENGINE_MOE % 32 + "#define GG_PART 0\n", "NB"),
    (ENGINE_MOE % 8 + "#define GG_PART 2\n#define FGU 10\n#define FSD 21\n", "types 10"),                     # Q2_K routed rows
    (ENGINE_MOE % 8 + "#define GG_PART 2\n#define FGU 23\n#define FSD 11\n", "23/11"),                        # Q3_K shared down
    ("#define E 64\n#define TOPK 10\n#define D 2560\n#define I 640\n#define NB 8\n#define GG_PART 3\n#define FD 12\n", "I 640"),  # Q4_K rows want I a multiple of 256
    (ENGINE_MOE % 8 + "#define GG_PART 1\n#define FSG 21\n#define FSU 8\n#define RBF 1\n", "equal"),
    (ENGINE_MOE % 8 + "#define GG_PART 6\n", "GG_PART"),
    ("#define E 512\n#define TOPK 10\n#define D 2000\n#define I 512\n#define NB 8\n#define GG_PART 3\n#define FD 21\n", "D 2000"),
    ("#define E 2048\n#define TOPK 10\n#define D 2048\n#define I 512\n#define NB 8\n#define GG_PART 0\n", "E 2048"),
])
def test_unsupported_blocks_fail_with_a_message(block, needle):
    ok, err, names = compile_check(block)
    assert not ok and needle in err and names == []


@pytest.mark.parametrize("fgu,fsd,fd", [(23, 21, 23), (12, 13, 14), (20, 14, 12), (21, 12, 13), (8, 23, 20)])
def test_routed_rows_of_the_other_types_are_taken(fgu, fsd, fd):
    """kernels/moe_gg.metal:336-395 of the reference: Q4_K, Q5_K, Q6_K, IQ4_NL and IQ4_XS beside IQ3_S and Q8_0, for the
    routed rows and for the shared down rows."""
    ok, err, names = compile_check(ENGINE_MOE % 8 + "#define GG_PART 2\n#define FGU %d\n#define FSD %d\n" % (fgu, fsd))
    assert ok and names == ["moe_gu_gg"], err
    ok, err, names = compile_check(ENGINE_MOE % 8 + "#define GG_PART 3\n#define FD %d\n" % fd)
    assert ok and sorted(names) == ["moe_cmb_gg", "moe_dn_gg"], err


def test_later_definitions_win_and_whitespace_is_tolerated():
    ok, err, names = compile_check("  #define   DQ_TEST   14  \n\n#define DQ_TEST\t8\r\n#define dq_test  my_dq\n")
    assert ok and names == ["my_dq"]


def test_packing_blocks_register_the_reference_names():
    blk = "#define moe_scatter moe_scatter_x\n#define E 512\n#define TOPK 10\n#define KD 2048\n#define I 512\n#define TM 64\n"  # bench/moe_prefill.c:86-87
    ok, err, names = compile_check(blk)
    assert ok, err
    assert names == ["moe_count", "moe_plan", "moe_plan_t", "moe_scatter_x", "moe_act", "p_act2", "moe_combine", "p_zero"]
    pf = ("#define IQ_DQ_ONLY\n#define E 512\n#define TOPK 10\n#define D 2048\n#define I 512\n#define NB 1\n#define GG_PART 5\n#define PFF 21\n#define KD 2048\n"
          "#define TM 64\n#define TN 64\n#define SG 4\n#define KC 64\n#define PFS 1\n#define PFT 1\n#define PFDBG 0\n#define moe_pf_gg moe_pf_gg_21_k2048_tm64\n")  # src/engine.c:3244-3248
    ok, err, names = compile_check(pf)
    assert ok and names == ["moe_pf_gg_21_k2048_tm64"], err
    ok, err, names = compile_check(pf.replace("#define TM 64", "#define TM 128"))
    assert not ok and "TM 128" in err
    ok, err, names = compile_check(pf.replace("#define PFF 21", "#define PFF 22"))
    assert not ok and "22" in err  # IQ2_S
    ok, err, names = compile_check(pf.replace("GG_PART 5", "GG_PART 6"))
    assert not ok and "GG_PART" in err


def test_other_formats_and_the_multi_matrix_block():
    for f, rb in ((12, 1152), (13, 1408), (14, 1680), (23, 1088), (20, 1152), (30, 4096), (1, 4096)):
        ok, err, names = compile_check("#define qmv_gg q_%d\n#define GF %d\n#define KD 2048\n#define RB %d\n#define NB 4\n" % (f, f, rb))
        assert ok and names == ["q_%d" % f], err
        ok, err, names = compile_check("#define DQ_TEST %d\n" % f)
        assert ok and names == ["dq_test"], err
    # src/engine.c:738-739: NB 0 builds one kernel per token count, <name>_b<n>
    blk = "#define IQ_DQ_ONLY 1\n#define qmv_ggm qmv_ggm_k2048_m4_12_12_14_30\n#define KD 2048\n#define NB 0\n#define NMAT 4\n#define GF0 12\n#define GF1 12\n#define GF2 14\n#define GF3 30\n"
    ok, err, names = compile_check(blk)
    assert ok, err
    assert names == ["qmv_ggm_k2048_m4_12_12_14_30_b%d" % n for n in range(1, 17)]
    ok, err, names = compile_check("#define qmv_ggm one\n#define KD 512\n#define NB 3\n#define NMAT 1\n#define GF0 23\n#define YT float\n")
    assert ok and names == ["one"], err


def test_valu_gemv_is_asked_for_by_a_macro():
    blk = "#define qmv_gg q1\n#define GF 21\n#define KD 2048\n#define RB 880\n#define NB 2\n#define YT float\n#define QW_VALU 1\n"
    ok, err, names = compile_check(blk)
    assert ok and names == ["q1"]


def test_reference_clients_link_against_the_library():
    """The reference's tools/dqtest.c and tools/ggmtest.c, compiled unchanged by oracle/Makefile (`make ref`, where the
    reference tree is mounted), ask the library for nothing it does not export."""
    import subprocess
    L = q.load_lib()
    exes = [os.path.join(ROOT, "oracle", "_ref", n) for n in ("dqtest_ref", "ggmtest_ref")]
    if not os.path.isdir("/root/reference"):
        pytest.skip("no reference tree here")
    for exe in exes:
        assert os.path.exists(exe), "oracle/_ref is stale: run `make -C oracle ref` after building the library"
        und = subprocess.run(["nm", "-D", "--undefined-only", exe], stdout=subprocess.PIPE, text=True, check=True).stdout
        asked = set(re.findall(r"\b(qw_[a-z0-9_]+)", und))
        assert asked and all(hasattr(L, n) for n in asked), asked
