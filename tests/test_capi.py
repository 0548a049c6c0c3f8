"""The C ABI without a GPU: libmi355_moe.so loads, exports every function include/mi355_moe.h
declares, the ctypes mirrors have the C structs' layout, and host-only entry points answer."""
import ctypes as C
import os
import re
import subprocess

import pytest

from therock_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "mi355_moe.h")


def declared_functions():
    text = re.sub(r"/\*.*?\*/", "", open(HEADER).read(), flags=re.S)
    return sorted(set(re.findall(r"\b(mi355_\w+)\s*\(", text)))


def test_every_declared_symbol_is_exported_and_bound():
    names = declared_functions()
    assert len(names) >= 10
    lib = _lib.load()
    for n in names:
        assert n in _lib.PROTOTYPES, f"{n} has no ctypes prototype"
        assert getattr(lib, n) is not None
    assert sorted(_lib.PROTOTYPES) == names


def test_struct_layouts_match_the_header(tmp_path):
    structs = {"mi355_moe_sorting_args": _lib.SortingArgs, "mi355_fused_moe_traits": _lib.FusedMoeTraits,
               "mi355_fused_moegemm_args": _lib.FusedMoeGemmArgs, "mi355_fused_moe_args": _lib.FusedMoeArgs,
               "mi355_topk_softmax_args": _lib.TopkSoftmaxArgs, "mi355_topk_softmax_traits": _lib.TopkSoftmaxTraits,
               "mi355_moe_flatmm_args": _lib.FlatmmArgs, "mi355_moe_smoothquant_args": _lib.SmoothquantArgs,
               "mi355_moe_workspace": _lib.Workspace}
    lines = ['#include <stdio.h>', '#include <stddef.h>', f'#include "{HEADER}"', "int main(void){"]
    for cname, ct in structs.items():
        lines.append(f'printf("{cname} %zu\\n", sizeof({cname}));')
        for fname, _ in ct._fields_:
            lines.append(f'printf("{cname}.{fname} %zu\\n", offsetof({cname}, {fname}));')
    lines.append("return 0;}")
    src = tmp_path / "layout.c"
    src.write_text("\n".join(lines))
    exe = tmp_path / "layout"
    subprocess.run(["gcc", "-std=c99", "-Wall", "-Werror", str(src), "-o", str(exe)], check=True)
    out = dict(l.split() for l in subprocess.run([str(exe)], check=True, capture_output=True, text=True).stdout.splitlines())
    for cname, ct in structs.items():
        assert int(out[cname]) == C.sizeof(ct), cname
        for fname, _ in ct._fields_:
            assert int(out[f"{cname}.{fname}"]) == getattr(ct, fname).offset, f"{cname}.{fname}"


def test_argument_blocks_have_the_layout_of_the_ck_tile_structs(tmp_path):
    """mi355_fused_moegemm_args / mi355_moe_sorting_args against ck_tile's FusedMoeGemmHostArgs / MoeSortingHostArgs:
    one translation unit includes both headers and static_asserts size and every field offset."""
    import shutil
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(hipcc):
        pytest.skip("hipcc is not installed")
    src = os.path.join(ROOT, "tests", "cpp", "abi_layout_check.cpp")
    cmd = [hipcc, "-std=c++17", "--cuda-host-only", "-I/opt/rocm/include", "-Wno-everything"]
    subprocess.run(cmd + ["-fsyntax-only", src], check=True)
    pre = subprocess.run(cmd + ["-E", src], check=True, capture_output=True, text=True).stdout
    if "mi355_abi_layout_checked = 1" not in pre:
        pytest.skip("the ck_tile headers are not installed: nothing to compare with")
    # the check is live: a struct with an extra field in front of hidden_size must fail to compile
    bad = tmp_path / "bad.cpp"
    bad.write_text(open(src).read().replace('#include "../../include/mi355_moe.h"',
                                            f'#define hidden_size padding_; int32_t hidden_size\n#include "{HEADER}"\n#undef hidden_size'))
    r = subprocess.run(cmd + ["-fsyntax-only", str(bad)], capture_output=True, text=True)
    assert r.returncode != 0 and "static assertion failed" in r.stderr


def test_tile_order_of_the_large_tile_kernel_visits_every_tile_once(tmp_path):
    """blocked_tile_of (the index arithmetic a workgroup of the large-tile kernel uses to find its tile) on the host:
    a bijection for every (row tiles, column tiles) pair, with the locality it is there for."""
    import shutil
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(hipcc):
        pytest.skip("hipcc is not installed")
    exe = tmp_path / "tile_order_check"
    subprocess.run([hipcc, "-std=c++17", "--cuda-host-only", "-I/opt/rocm/include", "-Wno-everything", "-o", str(exe),
                    os.path.join(ROOT, "tests", "cpp", "tile_order_check.cpp")], check=True)
    r = subprocess.run([str(exe)], capture_output=True, text=True)
    assert r.returncode == 0 and "tile_order_check ok" in r.stdout, r.stdout


def test_sizes_out_of_range_are_rejected_on_the_host():
    """No entry point divides by or indexes with a size before checking it (0 experts used to kill the process)."""
    lib = _lib.load()
    t = _lib.FusedMoeTraits(0, 0, 0, 3, 3, 3, 3, 32, 1, 0, 0, 0)
    for shape in ((128, 0, 2, 1024, 1024), (128, 8, 0, 1024, 1024), (-1, 8, 2, 1024, 1024), (128, 8, 2, 0, 1024),
                  (128, 8, 2, 1024, -4), (128, 2000, 2, 1024, 1024), (128, 8, 300, 1024, 1024),
                  (1 << 24, 8, 2, 1024, 1024), (0xffffff, 8, 255, 1024, 1024)):  # 24-bit tokens, 32-bit row indices
        assert lib.mi355_fused_moe_workspace_size(C.byref(t), *shape) == 0, shape
        assert lib.mi355_fused_moe_tile_rows(C.byref(t), *shape) == 0, shape
        T, E, K, H, I = shape
        f = _lib.FusedMoeArgs(block_m=32, hidden_size=H, intermediate_size=I, num_tokens=T, num_experts=E, topk=K,
                              stride_token=max(H, 0))
        ws = _lib.Workspace(None, 0)
        assert lib.mi355_fused_moe(C.byref(t), C.byref(f), C.byref(ws), None) == _lib.E_INVALID, shape
        assert b"bad sizes" in lib.mi355_moe_last_error()
        g = _lib.FusedMoeGemmArgs(hidden_size=H, intermediate_size=I, num_tokens=T, num_experts=E, topk=K,
                                  stride_token=max(H, 0))
        assert lib.mi355_fused_moegemm(C.byref(t), C.byref(g), C.byref(ws), None) == _lib.E_INVALID, shape
        assert lib.mi355_fused_moegemm(C.byref(t), C.byref(g), None, None) == _lib.E_INVALID, shape
    # a valid shape without a workspace: the workspace error, before anything is launched
    f = _lib.FusedMoeArgs(block_m=32, hidden_size=1024, intermediate_size=1024, num_tokens=128, num_experts=8, topk=2,
                          stride_token=1024)
    assert lib.mi355_fused_moe(C.byref(t), C.byref(f), None, None) == _lib.E_WORKSPACE


def test_static_workspace_entry_point_rejects_oversized_problems_on_the_host():
    lib = _lib.load()
    cap = lib.mi355_fused_moe_static_ws_capacity()
    assert cap == 96 << 20
    t = _lib.FusedMoeTraits(1, 1, 0, 3, 3, 3, 3, 32, 1, 0, 0, 0)
    assert lib.mi355_fused_moe_workspace_size(C.byref(t), 8192, 256, 8, 7168, 2048) > cap
    f = _lib.FusedMoeArgs(block_m=32, hidden_size=7168, intermediate_size=2048, num_tokens=8192, num_experts=256, topk=8,
                          stride_token=7168)
    assert lib.mi355_fused_moe_static_ws(C.byref(t), C.byref(f), None) == _lib.E_WORKSPACE
    assert b"library-owned" in lib.mi355_moe_last_error()
    f.num_experts = 0
    assert lib.mi355_fused_moe_static_ws(C.byref(t), C.byref(f), None) == _lib.E_INVALID
    # the benchmark's decode regime fits
    t8 = _lib.FusedMoeTraits(2, 2, 0, 3, 3, 3, 3, 32, 1, 0, 0, 0)
    for tokens in (16, 64, 256):
        assert 0 < lib.mi355_fused_moe_workspace_size(C.byref(t8), tokens, 128, 8, 4096, 1536) <= cap


def test_flatmm_operand_types_on_the_host():
    """Which operand pairs the stand-alone GEMMs take (decided on the host, before any launch): equal 16-bit or
    8-bit types, and bf16 activations with int8 weights for the down GEMM only."""
    lib = _lib.load()
    D = _lib.DTYPES

    def ws(kind, pa, pb):
        a = _lib.FlatmmArgs()
        a.NumTokens, a.NumExperts, a.TopK, a.N, a.K, a.block_m, a.k_batch = 64, 4, 2, 256, 128, 32, 1
        a.prec_a, a.prec_b = D[pa], D[pb]
        return lib.mi355_moe_flatmm_workspace_size(kind, C.byref(a))

    for kind in (0, 1, 2):
        for p in ("bf16", "fp16", "fp8"):
            assert ws(kind, p, p) > 0, (kind, p)
        assert ws(kind, "bf16", "fp16") == 0 and ws(kind, "fp16", "bf16") == 0 and ws(kind, "fp16", "int8") == 0
        assert b"operand types" in lib.mi355_moe_last_error()
    assert ws(1, "int8", "int8") > 0 and ws(2, "bf16", "int8") > 0 and ws(2, "int8", "int8") == 0
    # the same size limits as the fused entry points
    for field, value in (("NumTokens", 1 << 24), ("NumExperts", 0), ("TopK", 256), ("N", 0), ("K", -8)):
        a = _lib.FlatmmArgs()
        a.NumTokens, a.NumExperts, a.TopK, a.N, a.K, a.block_m, a.k_batch = 64, 4, 2, 256, 128, 32, 1
        a.prec_a = a.prec_b = D["bf16"]
        setattr(a, field, value)
        assert lib.mi355_moe_flatmm_workspace_size(1, C.byref(a)) == 0 and b"bad sizes" in lib.mi355_moe_last_error(), field

    # B as ck_tile::shuffle_b lays it out for 16-row warp tiles: rows of whole 64-byte blocks, no padded K
    def ws_shuffled(prec, K, b_shuffle=1, k_pad=0):
        a = _lib.FlatmmArgs()
        a.NumTokens, a.NumExperts, a.TopK, a.N, a.K, a.block_m, a.k_batch = 64, 4, 2, 256, K, 32, 1
        a.prec_a = a.prec_b = D[prec]
        a.b_shuffle, a.k_padded_zeros = b_shuffle, k_pad
        return lib.mi355_moe_flatmm_workspace_size(1, C.byref(a))

    assert ws_shuffled("bf16", 128) > 0 and ws_shuffled("int8", 128) > 0 and ws_shuffled("bf16", 96) > 0
    assert ws_shuffled("int8", 96) == 0 and b"b_shuffle" in lib.mi355_moe_last_error()
    assert ws_shuffled("bf16", 128, b_shuffle=2) == 0 and ws_shuffled("bf16", 128, k_pad=32) == 0


def test_host_only_entry_points():
    lib = _lib.load()
    assert lib.mi355_moe_version() == _lib.header_version() >= 210
    assert lib.mi355_moe_max_num_tokens_padded(128, 8, 2, 32) == 2 * 128 + 8 * 32 - 2
    assert lib.mi355_moe_sorting_workspace_size(64, 128, 8) == 0          # one workgroup, no workspace
    assert lib.mi355_moe_sorting_workspace_size(32768, 64, 6) >= 384 * 64 * 4
    t = _lib.FusedMoeTraits(0, 0, 0, 3, 3, 3, 3, 32, 1, 0, 0, 0)
    assert lib.mi355_fused_moe_supported(C.byref(t)) == 1
    ws = lib.mi355_fused_moe_workspace_size(C.byref(t), 128, 8, 2, 1024, 1024)
    assert ws >= 510 * 1024 * 2 + 256 * 1024 * 2
    bad = _lib.FusedMoeTraits(5, 5, 0, 3, 3, 3, 3, 32, 1, 0, 0, 0)
    assert lib.mi355_fused_moe_supported(C.byref(bad)) == 0
    assert lib.mi355_fused_moe_workspace_size(C.byref(bad), 128, 8, 2, 1024, 1024) == 0
    assert lib.mi355_moe_sorting(None, None) == _lib.E_INVALID and b"null" in lib.mi355_moe_last_error()
    assert lib.mi355_fused_moe(None, None, None, None) == _lib.E_INVALID
    # traits of the reference's example API: both activations and both weight layouts have kernels
    for act, gate_only, ok in ((0, 0, 1), (1, 1, 1), (0, 1, 1), (2, 0, 0), (1, 2, 0)):
        t = _lib.FusedMoeTraits(0, 0, 0, 3, 3, 3, 3, 32, act, gate_only, 0, 0)
        assert lib.mi355_fused_moe_supported(C.byref(t)) == ok
    # fp16 operands go with an fp16 output and only with it
    for pi, po, ok in ((5, 5, 1), (5, 0, 0), (0, 5, 0)):
        t = _lib.FusedMoeTraits(pi, pi, po, 3, 3, 3, 3, 32, 1, 0, 0, 0)
        assert lib.mi355_fused_moe_supported(C.byref(t)) == ok
    # weight layouts: FusedMoeGemmWeightPermuteEnum's two values, nothing else
    for prec in (0, 1, 2):
        for wp, ok in ((0, 1), (1, 1), (2, 0), (-1, 0)):
            t = _lib.FusedMoeTraits(prec, prec, 0, 3, 3, 3, 3, 32, 1, 0, 0, 0, wp)
            assert lib.mi355_fused_moe_supported(C.byref(t)) == ok
    # fused_quant 1 / 2 (re-quantised intermediate activations) exist for int8 and fp8 and need a larger workspace
    for prec, fq, ok in ((2, 1, 1), (2, 2, 1), (2, 3, 0), (0, 2, 0), (1, 1, 1), (1, 2, 1), (5, 2, 0)):
        t = _lib.FusedMoeTraits(prec, prec, 0, 3, 3, 3, 3, 32, 1, 0, fq, 0)
        assert lib.mi355_fused_moe_supported(C.byref(t)) == ok
    w0, w2 = (lib.mi355_fused_moe_workspace_size(C.byref(_lib.FusedMoeTraits(2, 2, 0, 3, 3, 3, 3, 32, 1, 0, fq, 0)),
                                                 256, 128, 8, 4096, 1536) for fq in (0, 2))
    assert w2 >= w0 + (256 * 8) * 1536
    # rows per GEMM workgroup: decode tiles, small tiles, 320-row tiles (sort unit a multiple of 16)
    rows = lambda prec, unit, *shape: lib.mi355_fused_moe_tile_rows(
        C.byref(_lib.FusedMoeTraits(prec, prec, 0, 3, 3, 3, 3, unit, 1, 0, 0, 0)), *shape)
    assert rows(2, 32, 64, 128, 8, 4096, 1536) == 32
    assert rows(1, 32, 8192, 256, 8, 7168, 2048) == 320
    assert rows(1, 32, 1024, 256, 8, 7168, 2048) == 320 and rows(1, 32, 512, 256, 8, 7168, 2048) == 32
    assert rows(1, 8, 8192, 256, 8, 7168, 2048) == 128
    # 28 .. 56 rows per expert: 64-row tiles of the decode kernel for 16-bit and int8 operands, 320-row tiles for fp8
    assert rows(2, 32, 640, 128, 8, 4096, 1536) == 64 and rows(0, 32, 160, 8, 2, 4096, 14336) == 64
    assert rows(2, 32, 448, 128, 8, 4096, 1536) == 64 and rows(2, 32, 432, 128, 8, 4096, 1536) == 32
    assert rows(2, 32, 896, 128, 8, 4096, 1536) == 64 and rows(2, 32, 912, 128, 8, 4096, 1536) == 320
    assert rows(1, 32, 1280, 256, 8, 7168, 2048) == 320
    assert rows(2, 32, 8192, 128, 8, 4096, 1536) == 320 and rows(2, 32, 8192, 128, 8, 4096, 1504) == 128


def test_python_mirror_rejects_unknown_traits_without_touching_the_gpu():
    import therock_amd as ta
    assert ta.fused_moe(ta.fused_moe_traits(prec_i="fp16", prec_w="fp16"), ta.fused_moe_args()) == -1.0
    with pytest.raises(ValueError):
        ta.fused_moe_traits(prec_i="fp4").pod()


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    """There is no CPU fallback: without the built HIP library every entry point of the Python mirror raises."""
    import therock_amd as ta
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", str(tmp_path / "libmi355_moe.so"))
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        ta.moe_sorting_get_workspace_size(64, 8, 2)
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        ta.fused_moe(ta.fused_moe_traits(), ta.fused_moe_args())


def test_build_entry_compares_the_library_with_the_header():
    """build() must take the expected version from the header, never from a literal of its own."""
    src = open(os.path.join(ROOT, "__graft_entry__.py")).read()
    body = src[src.index("def build()"):src.index("def smoke()")]
    assert "header_version()" in body
    import re
    assert not re.search(r"mi355_moe_version\(\)\s*[=!]=\s*\d", body)


def test_bench_refuses_more_than_one_gpu():
    r = subprocess.run(["python", os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert r.returncode != 0 and "one GPU only" in r.stderr
