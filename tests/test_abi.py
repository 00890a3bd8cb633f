"""CPU-side checks of the boundary: the library loads, exports every symbol that
include/quik_hip.h declares, rejects bad arguments before touching the GPU, and the Python
surface has the reference's names and keyword arguments.  No kernel is launched here."""
import ctypes
import inspect
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "quik_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(quik_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    from quik_amd import _lib as L
    lib = L.load()
    names = _declared_symbols()
    assert len(names) >= 14
    for n in names:
        assert hasattr(lib, n), n
    assert sorted(L.SIGNATURES) == names
    assert lib.quik_abi_version() == 1
    assert lib.quik_status_string(-1) == b"bits argument must be either 4 or 8"


def test_argument_validation_without_gpu():
    """Every entry point validates before launching; these calls return before any HIP call."""
    from quik_amd import _lib as L
    lib = L.load()
    null = ctypes.c_void_p(None)
    one = ctypes.c_void_p(16)  # never dereferenced: validation fails first
    assert lib.quik_colmap_bytes(8192, 7936, 256) > 0
    assert lib.quik_colmap_bytes(8192, 7936, 255) == 0
    # idx16 layout: src_col (2 B each), fp_col, one mask bit per column, one u32 per 8-column group, one u32 per
    # possible dirty group (at most one per outlier), one u16 per possible dirty group, the in-place order (one u16
    # per integer column) and its patch list (one u32 per outlier column), the 16-column units of the int8 operand
    # buffers (one u16 per unit, one u16 and 16 source columns per unit that may need a gather: at most one per
    # outlier column), flags; every section 16-byte aligned
    assert lib.quik_colmap_bytes(8192, 7936, 256) == (7936 * 2 + 512 + 1024 + 4096 + 1024 + 512 + 7936 * 2 + 1024 +
                                                      7936 // 16 * 2 + 512 + 256 * 32 + 16)
    a16 = lambda v: (v + 15) // 16 * 16
    assert lib.quik_colmap_bytes(70000, 69000, 1000) == 69000 * 4 + a16(4000) + a16((70000 + 31) // 32 * 4) + 16
    assert lib.quik_asym_quantize(one, 0, 4, 64, one, 62, 2, 5, one, one, one, null) == -1
    assert lib.quik_asym_quantize(one, 0, 4, 64, one, 60, 2, 4, one, one, one, null) == -2
    assert lib.quik_asym_quantize(one, 0, 4, 64, one, 61, 3, 4, one, one, one, null) == -4
    assert lib.quik_asym_quantize(one, 7, 4, 64, one, 62, 2, 4, one, one, one, null) == -3
    assert lib.quik_asym_quantize(null, 0, 4, 64, one, 62, 2, 4, one, one, one, null) == -5
    assert lib.quik_asym_quantize(one, 0, 0, 64, one, 62, 2, 4, one, one, one, null) == 0     # empty batch
    assert lib.quik_int4_matmul(one, one, one, 4, 4, 48, null) == -4      # K % 32
    assert lib.quik_int4_matmul(one, one, one, 4, 4, 131072, null) == -6  # accumulator headroom
    assert lib.quik_int8_matmul(one, one, one, 4, 4, 24, null) == -4      # K % 16
    assert lib.quik_int8_matmul(null, one, one, 4, 4, 32, null) == -5
    assert lib.quik_int4_matmul(one, one, one, 0, 4, 32, null) == 0
    assert lib.quik_asym_dequantize(one, one, one, one, one, 0, 4, 4, 3, one, null) == -1
    assert lib.quik_sym_dequantize(one, 4, one, one, one, 4, 4, one, null) == -1
    assert lib.quik_sym_quantize(one, one, 4, 4, 16, one, null) == -1
    assert lib.quik_mixed_linear_fwd(one, one, one, one, one, one, one, null, 0, 4, 4, 32, 12, 4, one, null) == -4
    assert lib.quik_mixed_linear_fwd(one, one, null, one, one, one, one, null, 0, 4, 4, 32, 8, 4, one, null) == -5


def test_tile_ordered_entry_points_validate_without_gpu():
    """The entry points that write or read tile-ordered operand buffers reject shapes, alignments and NULL
    pointers before any HIP call (the column map's streaming flag lives on the device: a map that does not
    stream makes the kernel write nothing, and the Python wrappers refuse it before launching)."""
    from quik_amd import _lib as L
    lib = L.load()
    null = ctypes.c_void_p(None)
    one = ctypes.c_void_p(256)  # aligned, never dereferenced
    odd = ctypes.c_void_p(264)  # 8 mod 256
    f = ctypes.c_float
    assert lib.quik_fp6_operand_bytes(2048, 7936, 256) == 32 * (124 + 16) * 3072 + 2048 * 4
    assert lib.quik_fp6_operand_bytes(2048, 7936 + 64, 256) == 0           # K % 128
    assert lib.quik_tile8_operand_bytes(2048, 28416, 256) == 32 * (888 + 16) * 2048
    assert lib.quik_tile8_operand_bytes(2048, 28416, 8) == 0               # F % 32
    assert lib.quik_asym_quantize_fp6(one, 0, 64, 8192, one, 7936 - 64, 256 + 64, one, one, null) == -4
    assert lib.quik_asym_quantize_fp6(one, 0, 64, 8192, one, 7936, 256, odd, one, null) == -4
    assert lib.quik_asym_quantize_fp6(one, 0, 64, 8192, null, 7936, 256, one, one, null) == -5
    assert lib.quik_asym_quantize_fp6(one, 3, 64, 8192, one, 7936, 256, one, one, null) == -3
    assert lib.quik_asym_quantize_fp6(one, 0, 64, 8192, one, 7936, 250, one, one, null) == -2
    assert lib.quik_asym_quantize_fp6(one, 0, 0, 8192, one, 7936, 256, one, one, null) == 0     # empty batch
    assert lib.quik_asym_quantize_tile8(one, 0, 64, 8192, one, 8192 - 32, 32, one, one, null) == -4   # K % 64
    assert lib.quik_asym_quantize_tile8(one, 0, 64, 8192, one, 7936, 256, one, null, null) == -5
    assert lib.quik_sym_quantize_mapped(one, 64, 8192, one, 7936, 256, 5, f(4.0), 1, one, one, null, null) == -1
    assert lib.quik_sym_quantize_mapped(one, 64, 8192, one, 7936, 256, 4, f(0.0), 1, one, one, null, null) == -2
    assert lib.quik_sym_quantize_mapped(one, 64, 8190, one, 7934, 256, 4, f(4.0), 0, one, one, one, null) == -2
    assert lib.quik_sym_quantize_mapped(one, 64, 8192, one, 7936, 256, 4, f(4.0), 0, one, one, null, null) == -5
    assert lib.quik_sym_quantize_mapped(one, 64, 8192, one, 7936, 256, 4, f(4.0), 1, odd, one, null, null) == -4
    assert lib.quik_mixed_linear_fwd_fp6(one, one, one, one, one, null, 0, -1, 256, 7936, 256, one, null) == -2
    assert lib.quik_mixed_linear_fwd_fp6(one, odd, one, one, one, null, 0, 64, 256, 7936, 256, one, null) == -4
    assert lib.quik_mixed_linear_fwd_fp6(one, one, one, one, one, null, 0, 64, 256, 74496 + 128, 256, one, null) == -6
    assert lib.quik_mixed_linear_fwd_tile8(one, one, null, one, one, null, 0, 64, 256, 28416, 256, one, null) == -5
    assert lib.quik_splitk_workspace_bytes(64, 8192, 28416, 8) > 4096
    assert lib.quik_splitk_workspace_bytes(2048, 28672, 7936, 4) == 0
    assert lib.quik_sim_act_fake_quant(one, 0, 4, 64, one, 1, one, null) == -1
    assert lib.quik_sim_act_fake_quant(one, 0, 4, 64, one, 9, one, null) == -1
    assert lib.quik_sim_act_fake_quant(one, 2, 4, 64, one, 4, one, null) == -3
    assert lib.quik_sim_act_fake_quant(one, 0, 4, 0, one, 4, one, null) == -2
    assert lib.quik_sim_act_fake_quant(one, 0, 4, 64, null, 4, one, null) == -5
    assert lib.quik_sim_act_fake_quant(one, 0, 0, 64, one, 4, one, null) == 0


def test_python_surface_matches_reference_names():
    """Names and keyword arguments of the pybind module (src/asymmetric/asymmetric.cpp:144-180,
    src/symmetric/symmetric.cpp:120-136, src/matmul/matmul.cpp:85,109 of the reference)."""
    import quik
    from quik._C import asymmetric, matmul, symmetric
    assert quik.__all__ == ['matmul', 'symmetric', 'asymmetric']
    sig = lambda f: list(inspect.signature(f).parameters)
    assert sig(asymmetric.quantize) == ["src", "int_indices", "fp_indices", "bits"]
    assert sig(asymmetric.dequantize) == ["x", "meta", "scale_col", "wReduced", "y", "bits"]
    assert sig(asymmetric.find_meta) == ["src", "bits"]
    assert sig(asymmetric.quantizeOld) == ["src", "meta", "bits"]
    assert sig(symmetric.quantize) == ["src", "scale", "bits"]
    assert sig(symmetric.dequantize) == ["x", "scale_row", "scale_col", "y", "bits"]
    assert sig(matmul.int4Matmul) == ["A", "B"] and sig(matmul.int8Matmul) == ["A", "B"]
    # fused GEMM + dequantize ops (src/asymmetric/asymmetric.cpp:182-211, src/symmetric/symmetric.cpp:120-136)
    for f in (asymmetric.int4FusedDequantize, asymmetric.int8FusedDequantize):
        assert sig(f) == ["A", "B", "scale_row", "scale_col", "shift_value", "zero_row", "w_reduced", "y"]
    for f in (symmetric.int4FusedDequantize, symmetric.int8FusedDequantize):
        assert sig(f) == ["A", "B", "scale_row", "scale_col", "y"]
    from quik_amd import qlinear
    assert sig(qlinear.MixedQLinear.from_float)[:7] == ["module", "weight_matrix", "weights_scales", "shared_input",
                                                         "fp_indices", "symm", "bits"]
    assert sig(qlinear.MixedQLinear.__init__)[1:8] == ["in_features", "out_features", "shared_input",
                                                        "fp_features_num", "symm", "bits", "dtype"]


def test_typed_stubs_describe_the_modules():
    """quik/_C/*.pyi (the reference ships the same three, quik/_C/{asymmetric,matmul,symmetric}.pyi): every function a
    stub declares exists in the module with the same parameter names in the same order."""
    import ast
    import importlib
    for name in ("asymmetric", "matmul", "symmetric"):
        mod = importlib.import_module("quik_amd." + name)
        tree = ast.parse(open(os.path.join(ROOT, "quik", "_C", name + ".pyi")).read())
        funcs = [n for n in tree.body if isinstance(n, ast.FunctionDef)]
        assert len(funcs) >= 2
        for f in funcs:
            assert [a.arg for a in f.args.args] == list(inspect.signature(getattr(mod, f.name)).parameters), f.name
        for public in mod.__all__:
            if public != "check_mapped_args":
                assert public in {f.name for f in funcs}, (name, public)


def test_ops_reject_cpu_tensors_and_bad_bits():
    import torch

    import quik
    x = torch.zeros(4, 64, dtype=torch.float16)
    ii, fi = torch.arange(62), torch.tensor([62, 63])
    with pytest.raises(RuntimeError, match="CUDA"):
        quik.asymmetric.quantize(x, ii, fi, 4)
    with pytest.raises(RuntimeError, match="either 4 or 8"):
        quik.asymmetric.quantize(x, ii, fi, 3)
    with pytest.raises(RuntimeError, match="CUDA"):
        quik.matmul.int4Matmul(torch.zeros(4, 16, dtype=torch.uint8), torch.zeros(4, 16, dtype=torch.uint8))
    with pytest.raises(RuntimeError, match="CUDA"):   # device check precedes the bits switch, as in the reference
        quik.symmetric.quantize(x, x[:, :1].contiguous(), 16)


def test_from_float_buffers_on_cpu():
    """from_float's packing is host/torch work and must match the oracle without a GPU."""
    import numpy as np
    import torch

    from oracle import quik_oracle as qo
    from quik_amd.qlinear import MixedQLinear, SharedQuantizedInput, pack_to_i4
    rng = np.random.default_rng(0)
    N, n_in, F = 48, 256, 32
    fi = rng.permutation(n_in)[:F].astype(np.int64)
    mask = np.ones(n_in, bool)
    mask[fi] = False
    ii = np.arange(n_in)[mask]
    for bits in (4, 8):
        lo, hi = (-8, 8) if bits == 4 else (-127, 128)
        codes = rng.integers(lo, hi, (N, n_in - F))
        s_w = rng.uniform(0.001, 0.01, (N, 1)).astype(np.float16)
        W = np.zeros((N, n_in), np.float16)
        W[:, ii] = (codes * s_w.astype(np.float32)).astype(np.float16)
        W[:, fi] = (0.02 * rng.standard_normal((N, F))).astype(np.float16)
        lin = torch.nn.Linear(n_in, N, bias=False)
        mod = MixedQLinear.from_float(lin, torch.from_numpy(W), torch.from_numpy(s_w), SharedQuantizedInput(1),
                                      torch.from_numpy(fi), bits=bits)
        o = qo.from_float(W, s_w, fi, bits)
        assert np.array_equal(mod.int_weight.numpy(), o["int_weight"])
        assert np.array_equal(mod.reduced_w.numpy(), o["reduced_w"])
        assert np.array_equal(mod.fp_weight.numpy(), o["fp_weight"])
        assert np.array_equal(mod.int_indices.numpy(), o["int_indices"]) and mod.bias is None
        assert set(mod.state_dict()) == {"weights_scales", "int_weight", "int_indices", "fp_indices", "fp_weight",
                                         "reduced_w"}
    assert pack_to_i4(torch.tensor([[-8, 7]])).tolist() == [[0x78]]
    # a converted module computes in the type its buffers now have (the integer buffers keep theirs)
    assert mod.dtype == torch.float16
    mod = mod.to(torch.bfloat16)
    assert mod.dtype == torch.bfloat16 and mod.weights_scales.dtype == torch.bfloat16
    assert mod.int_weight.dtype == torch.int8 and mod.int_indices.dtype == torch.int64
    assert mod.half().dtype == torch.float16
    with pytest.raises(AssertionError, match="duplication"):
        MixedQLinear.from_float(lin, torch.from_numpy(W), torch.from_numpy(s_w), None, torch.tensor([1, 1]), bits=4)


def test_layer_forward_validates_without_gpu():
    """quik_layer_forward / quik_layer_workspace_bytes check the descriptor, the pointers, their alignment and the
    workspace size before any HIP call."""
    from quik_amd import _lib as L
    lib = L.load()
    null = ctypes.c_void_p(None)
    one, odd = ctypes.c_void_p(256), ctypes.c_void_p(264)

    def layer(**kw):
        d = L.QuikLayer()
        d.struct_bytes = ctypes.sizeof(L.QuikLayer)
        d.bits, d.dtype, d.symmetric = 4, L.QUIK_F16, 0
        d.in_features, d.num_int, d.num_fp, d.out_features = 8192, 7936, 256, 1024
        d.sym_divisor, d.colmap_streams, d.tiled_min_rows = 4.0, 1, 33
        d.colmap = d.int_weight = d.weights_scales = d.reduced_w = d.fp_weight = 256
        for k, v in kw.items():
            setattr(d, k, v)
        return d

    fwd = lambda d, x=one, rows=64, ws=one, nb=1 << 30, out=one: lib.quik_layer_forward(
        ctypes.byref(d), x, rows, ws, nb, null, 0, out, null, null)
    a256 = lambda v: (v + 255) // 256 * 256
    # row-major plan: packed codes, (scale, zero) per row, outlier values; every section 256-byte aligned
    d = layer()
    assert lib.quik_layer_workspace_bytes(ctypes.byref(d), 20) == a256(20 * 7936 // 2) + a256(20 * 4) + a256(20 * 256 * 2)
    assert lib.quik_layer_workspace_bytes(ctypes.byref(d), 64) == a256(64 * 7936 // 2) + a256(64 * 4) + a256(64 * 256 * 2)
    # tile-ordered plan once the layer has a tile-ordered weight copy and enough rows: operand buffer + (scale, zero)
    t = layer(tiled_weight=256)
    assert lib.quik_layer_workspace_bytes(ctypes.byref(t), 64) == \
        a256(lib.quik_fp6_operand_bytes(64, 7936, 256)) + a256(64 * 4)
    assert lib.quik_layer_workspace_bytes(ctypes.byref(t), 32) == lib.quik_layer_workspace_bytes(ctypes.byref(d), 32)
    t8 = layer(bits=8, tiled_weight=256, in_features=28672, num_int=28416)
    assert lib.quik_layer_workspace_bytes(ctypes.byref(t8), 64) == \
        a256(lib.quik_tile8_operand_bytes(64, 28416, 256)) + a256(64 * 4)
    assert lib.quik_layer_workspace_bytes(ctypes.byref(layer(struct_bytes=8)), 64) == 0
    assert lib.quik_layer_workspace_bytes(ctypes.byref(d), 0) == 0
    assert fwd(layer(struct_bytes=8)) == -2                  # a descriptor of another layout
    assert fwd(layer(bits=5)) == -2
    assert fwd(layer(num_fp=255)) == -2                      # num_int + num_fp != in_features
    assert fwd(d, rows=-1) == -2
    assert fwd(d, rows=0) == 0                               # empty batch
    assert fwd(d, x=null) == -5
    assert fwd(d, out=null) == -5
    assert fwd(layer(reduced_w=None)) == -5                  # asymmetric needs the reduced weights
    assert fwd(layer(fp_weight=None)) == -5
    assert fwd(layer(int_weight=None)) == -5                 # ... only a layer whose every call is tile-ordered may
    assert fwd(layer(int_weight=None, tiled_weight=256), rows=20) == -5
    assert fwd(d, x=ctypes.c_void_p(264)) == -4
    assert fwd(d, ws=odd) == -4
    assert fwd(d, nb=1024) == -6                             # workspace too small
    assert fwd(layer(symmetric=1, dtype=L.QUIK_BF16)) == -3  # symmetric activations are fp16
