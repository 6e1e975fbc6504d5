"""Host-side checks that need no GPU: the library loads, exports every symbol the header declares,
the ctypes mirrors match the C struct layouts, and argument errors are reported the reference's way
(message + outputs untouched) before any device work."""
import ctypes
import os
import re
import subprocess

import numpy as np
import pytest

import helpers as hp

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CLANG = "/opt/rocm/lib/llvm/bin/clang"


def declared_functions():
    text = open(os.path.join(ROOT, "include", "ptl_api.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    names = re.findall(r"^\s*(?:const\s+)?(?:void|int|float|char|size_t)\s*\*?\s*(\w+)\s*\(", text, flags=re.M)
    return sorted(set(names))


def test_library_exports_every_declared_symbol(pkg):
    lib = pkg.load()
    names = declared_functions()
    assert len(names) > 110
    missing = [n for n in names if not hasattr(lib, n)]
    assert not missing, missing
    # and the Python lists name nothing the header does not declare
    listed = set(pkg.VOID_ENTRY_POINTS + pkg.BATCHED_ENTRY_POINTS + pkg.OTHER_ENTRY_POINTS + pkg.STEP_ENTRY_POINTS +
                 pkg.PLAIN_ENTRY_POINTS + pkg.FUSED_NORM_ENTRY_POINTS + pkg.CACHED_ENTRY_POINTS + pkg.DEFERRED_ENTRY_POINTS + pkg.STATS_ENTRY_POINTS +
                 pkg.GRAD_STATS_ENTRY_POINTS + pkg.NORMED_ENTRY_POINTS + pkg.CHAINED_ENTRY_POINTS +
                 pkg.HEAD_ENTRY_POINTS)
    assert listed == set(names)


STRUCTS = {
    "blob": "Blob", "blob_fp16": "Blob", "im2col_args": "Im2colArgs", "im2col_args_fp16": "Im2colArgs",
    "transp_args": "TranspArgs", "transp_args_fp16": "TranspArgs", "layout_args": "LayoutArgs",
    "blocktransp_args": "BlocktranspArgs", "copy_args": "CopyArgs", "set_to_value_args": "SetToValueArgs",
    "set_to_value_args_fp16": "SetToValueArgsFp16", "vect_sum_args": "VectSumArgs", "cast_16t32_args": "CastArgs",
    "cast_32t16_args": "CastArgs", "pad_args": "PadArgs", "pad_args_fp16": "PadArgs", "matMul_args": "MatMulArgs",
    "matMul_args_fp16": "MatMulArgs", "kernel_DW_args": "KernelDWArgs", "kernel_DW_args_fp16": "KernelDWArgsFp16",
    "mm_manager_args": "MMManagerArgs", "mm_manager_args_fp16": "MMManagerArgs",
    "mm_bias_add_args": "MMBiasAddArgs", "mm_bias_add_args_fp16": "MMBiasAddArgs", "Conv2D_args": "Conv2DArgs",
    "Conv2D_args_fp16": "Conv2DArgs", "PointWise_Conv_args": "PointWiseConvArgs",
    "PointWise_Conv_args_fp16": "PointWiseConvArgs", "DepthWise_Conv_args": "DepthWiseConvArgs",
    "DepthWise_Conv_args_fp16": "DepthWiseConvArgsFp16", "Linear_args": "LinearArgs", "Linear_args_fp16": "LinearArgs",
    "softmax_args": "SoftmaxArgs", "Mhsa_args": "MhsaArgs", "act_args": "ActArgs", "act_args_fp16": "ActArgs",
    "SkipConn_args": "SkipConnArgs", "SkipConn_args_fp16": "SkipConnArgs", "pool_args": "PoolArgs",
    "pool_args_fp16": "PoolArgs", "loss_args": "LossArgs", "loss_args_fp16": "LossArgs", "optim_args": "OptimArgs",
    "optim_args_fp16": "OptimArgsFp16", "BatchNorm_args_fp32": "BatchNormArgs", "BatchNorm_args_fp16": "BatchNormArgs",
    "ptl_norm_fusion_fp32": "NormFusion", "ptl_norm_fusion_fp16": "NormFusion", "ptl_conv_cache": "ConvCache", "ptl_wg_batch": "WgBatch", "ptl_norm_stats": "NormStats", "ptl_grad_post": "GradPost",
}


def test_ctypes_mirrors_match_c_layout(pkg, tmp_path):
    """sizeof and the offset of the last field of every struct, as a C compiler sees the header."""
    lines = ['#include <stdio.h>', '#include <stddef.h>', '#include "ptl_structs.h"', "int main(void){"]
    for cname, pyname in STRUCTS.items():
        last = getattr(pkg, pyname)._fields_[-1][0].rstrip("_")
        lines.append('printf("%s %%zu %%zu\\n", sizeof(struct %s), offsetof(struct %s, %s));'
                     % (cname, cname, cname, last))
    lines.append("return 0;}")
    src = tmp_path / "probe.c"
    src.write_text("\n".join(lines))
    exe = tmp_path / "probe"
    subprocess.check_call([CLANG, "-I", os.path.join(ROOT, "include"), str(src), "-o", str(exe)])
    out = subprocess.check_output([str(exe)], text=True)
    for line in out.strip().splitlines():
        cname, size, off = line.split()
        cls = getattr(pkg, STRUCTS[cname])
        assert ctypes.sizeof(cls) == int(size), cname
        assert getattr(cls, cls._fields_[-1][0]).offset == int(off), cname


def test_rejected_arguments_leave_outputs_untouched(pkg, capfd):
    lib = pkg.load()
    x = np.ones((2, 5, 5), np.float32)
    w = np.ones((3, 2, 3, 3), np.float32)
    y = np.full((3, 3, 3), 7.0, np.float32)
    # invalid layout flag: reference prints and returns (pulp_conv2d_fp32.c:162-164)
    a, keep = hp.conv2d_args(pkg, x, None, w, None, y, None, 2, 5, 5, 3, 3, 3, 3, 3, hwc=2)
    lib.pulp_conv2d_fp32_fw_cl(ctypes.byref(a))
    assert lib.ptl_last_status() == 1
    assert np.all(y == 7.0)
    # invalid algorithm selector (pulp_conv2d_fp32.c:219-221)
    a, keep = hp.conv2d_args(pkg, x, None, w, None, y, None, 2, 5, 5, 3, 3, 3, 3, 3, im2col=5)
    lib.pulp_conv2d_fp32_fw_cl(ctypes.byref(a))
    assert lib.ptl_last_status() == 1
    # naive HWC does not exist in the reference (pulp_conv2d_fp32.c:210-212)
    a, keep = hp.conv2d_args(pkg, x, None, w, None, y, None, 2, 5, 5, 3, 3, 3, 3, 3, hwc=1, im2col=0)
    lib.pulp_conv2d_fp32_fw_cl(ctypes.byref(a))
    assert lib.ptl_last_status() == 1
    # stride that does not divide the padded extent: im2row prints and returns (pulp_im2col_fp32.c:125-128)
    y2 = np.full((3, 2, 2), 7.0, np.float32)
    a, keep = hp.conv2d_args(pkg, np.ones((2, 6, 6), np.float32), None, w, None, y2, None, 2, 6, 6, 3, 3, 3, 2, 2,
                             stride=(2, 2))
    lib.pulp_conv2d_fp32_fw_cl(ctypes.byref(a))
    assert lib.ptl_last_status() == 1
    assert np.all(y2 == 7.0)
    # pointwise with a bad layout flag (pulp_conv_pw_fp32.c:87-89)
    a, keep = hp.pw_args(pkg, x, None, w, None, y, None, 2, 3, 5, 5, hwc=3)
    lib.pulp_conv_pw_fp32_fw_cl(ctypes.byref(a))
    assert lib.ptl_last_status() == 1
    # mm_manager with a layer it does not serve / an id outside the list (pulp_train_utils_fp32.c:1666-1668)
    m = hp.mm_args(pkg, x, w, y, 1, 1, 1, 0)
    man = pkg.MMManagerArgs()
    man.mm_args = ctypes.pointer(m)
    man.layer_type, man.step_type, man.matmul_type = pkg.LAYER_DW_CONV, pkg.STEP_FW, 0
    lib.mm_manager(ctypes.byref(man))
    assert lib.ptl_last_status() == 1
    man.layer_type, man.matmul_type = pkg.LAYER_CONV2D, 24
    lib.mm_manager(ctypes.byref(man))
    assert lib.ptl_last_status() == 1
    out = capfd.readouterr().out
    for msg in ("Invalid data layout format", "Invalid selection of the conv2d algorithm", "not implemented",
                "Invalid H stride", "Invalid HWC parameter", "Wrong layer_type selection", "Wrong matmul selection"):
        assert msg in out, msg
    assert np.all(y == 7.0)


def test_no_device_fails_loudly(pkg):
    import torch
    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    lib = pkg.load()
    assert lib.ptl_init(0) != 0
    assert b"no CPU fallback" in lib.ptl_last_error()
    # a compute entry point reports the failure instead of computing on the host
    A = np.ones((4, 4), np.float32)
    C = np.zeros((4, 4), np.float32)
    assert lib.ptl_mm_fp32(A.ctypes.data, A.ctypes.data, C.ctypes.data, 4, 4, 4, 0) != 0
    assert np.all(C == 0)


def test_cache_prepare_rejects_before_any_device_work(pkg):
    """ptl_conv2d_fp16_cache_prepare: no cache, a layer that reads no blocked copy, a buffer that is too small - all
    reported as argument errors (1) without touching a device."""
    lib = pkg.load()
    x = np.zeros((64, 8, 8), np.float16)
    w = np.zeros((64, 64, 3, 3), np.float16)
    y = np.zeros((64, 8, 8), np.float16)
    a, keep = hp.conv2d_args(pkg, x, None, w, None, y, None, 64, 8, 8, 64, 3, 3, 8, 8, (1, 1, 1, 1))
    assert lib.ptl_conv2d_fp16_cache_prepare(ctypes.byref(a), 4, None) == 1
    need = lib.ptl_conv2d_fp16_cache_bytes(ctypes.byref(a), 4)
    assert need == (64 // 8 * 4 * 9 * 9 + 256 + 384) * 16  # blocked, padded copy of four samples + the kernel's reach
    c = pkg.ConvCache()
    c.valid = 1
    c.buf, c.bytes = 16, need - 16
    assert lib.ptl_conv2d_fp16_cache_prepare(ctypes.byref(a), 4, ctypes.byref(c)) == 1
    assert c.valid == 0 and b"16-byte aligned" in lib.ptl_last_error()
    x32 = np.zeros((32, 8, 8), np.float16)
    w32 = np.zeros((64, 32, 3, 3), np.float16)
    a32, keep32 = hp.conv2d_args(pkg, x32, None, w32, None, y, None, 32, 8, 8, 64, 3, 3, 8, 8, (1, 1, 1, 1))
    c.bytes = 1 << 20
    assert lib.ptl_conv2d_fp16_cache_prepare(ctypes.byref(a32), 4, ctypes.byref(c)) == 1
    assert b"does not read a blocked copy" in lib.ptl_last_error()


def test_product_does_not_reference_the_oracle():
    """Nothing under the package or include/ names the oracle."""
    for base in ("pulp-trainlib_amd", "include"):
        for dirpath, _, files in os.walk(os.path.join(ROOT, base)):
            if "build" in dirpath.split(os.sep):
                continue
            for f in files:
                if f.endswith((".so", ".o", ".pyc")):
                    continue
                text = open(os.path.join(dirpath, f), errors="ignore").read()
                assert "oracle" not in text.lower() or f == "__init__.py" and "oracle" not in text, (dirpath, f)


def test_struct_fields_match_the_reference_headers():
    """include/ptl_structs.h against tests/golden/struct_fields.json, the (type, name) lists of the reference's
    own struct declarations (written by tests/golden/make_struct_fields.py from lib/include/*.h): same fields,
    same order, same types - `fp16` and `float16alt`-style spellings of the 16-bit type aside."""
    import importlib.util
    import json
    spec = importlib.util.spec_from_file_location("make_struct_fields",
                                                  os.path.join(ROOT, "tests", "golden", "make_struct_fields.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    mine = mod.struct_fields(open(os.path.join(ROOT, "include", "ptl_structs.h")).read())
    gold = json.load(open(os.path.join(ROOT, "tests", "golden", "struct_fields.json")))
    assert set(mine) == set(gold["reference_structs"]) | set(gold["extensions"])
    assert gold["extensions"] == ["BatchNorm_args_fp16", "ptl_conv_cache", "ptl_grad_post", "ptl_norm_fusion_fp16", "ptl_norm_fusion_fp32",
                                  "ptl_norm_stats", "ptl_wg_batch"]
    norm = lambda t: t.replace("unsigned int", "unsigned").strip()
    for name, ref in gold["reference_structs"].items():
        got = [[norm(t), f] for t, f in mine[name]]
        want = [[norm(t), f] for t, f in ref["fields"]]
        assert got == want, (name, ref["header"])
