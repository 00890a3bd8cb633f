"""MixedQLinear for MI355X: the module interface of the reference's experiments/qlinear.py.

Same constructor, buffers, `from_float` signature and `SharedQuantizedInput` protocol as the
reference (experiments/qlinear.py:21-199), so `llama_replace_with_kernels`
(experiments/llama.py:394-440) can use it unchanged.  Differences, all deliberate:

* forward runs two launches by default: one quantize kernel (cached column map) and one fused
  GEMM kernel (integer GEMM + outlier GEMM + dequantize).  `fused=False` replays the
  reference's op sequence (F.linear, int GEMM, dequantize) with the stand-alone ops.
* a 3-D input (B, S, in) is flattened to (B*S, in) and the result has shape (B, S, N); the
  reference keeps only batch element 0 (qlinear.py:89-90) and returns (1, S, N), which is
  the same thing for B == 1.
* the symmetric branch works: the reference calls the symmetric ops without their `bits`
  argument and hands a [N, 1] scale where [1, N] is checked (qlinear.py:103,142), so it raises
  at HEAD.  Its activation scale divisor `1 << (bits - 1) - 1` parses as 1 << ((bits-1)-1)
  = 4 for bits=4; that value is kept (`sym_divisor`) so codes match what the expression says.
"""
from __future__ import annotations

import ctypes
import weakref

import torch
from torch import Tensor

from . import _lib as L
from . import asymmetric, matmul, symmetric
from ._lib import device_guard

__all__ = ["MixedQLinear", "SharedQuantizedInput", "FusedMixedQLinearGroup", "Linear4bit", "Linear8bit", "pack_to_i4",
           "two_compl"]


def two_compl(x: Tensor, bits: int) -> Tensor:
    return torch.where(x < 0, 2 ** bits + x, x)


def pack_to_i4(X: Tensor) -> Tensor:
    """Signed int4 codes [R, K] (K even) -> uint8 [R, K/2], even element in the low nibble."""
    u = two_compl(X.to(dtype=torch.int8), 4).to(torch.uint8)
    return u[:, 0::2] | (u[:, 1::2] << 4)


class _PerObjectCache(dict):
    """A cache that copies of its owner do not inherit (it holds ctypes structures with raw pointers)."""

    def __copy__(self):
        return _PerObjectCache()

    def __deepcopy__(self, memo):
        return _PerObjectCache()


class SharedQuantizedInput:
    """Quantized activation shared by the layers of one group (q/k/v, gate/up): the first
    member quantizes, the others reuse, the last one clears (qlinear.py:21-37).

    The reference shares only the quantized activation and still runs one GEMM per member.  Here the members
    register with the group when they are built; when the first member of a complete, compatible group is called
    (same input size, outlier columns, bits, symmetry, dtype, bias or no bias), the group runs ONE quantize and
    ONE GEMM over the members' weights concatenated along the output dimension, hands the caller its columns of
    the result and keeps the other members' columns until they are called (they then compute nothing), as the
    shared quantized activation is kept in the reference.  The per-column arithmetic is the members', so every
    output has the bits the member alone would give.  `MixedQLinear.fuse_shared_groups = False` switches this off."""

    def __init__(self, group_size):
        self.qint_x = None
        self.fp_x = None
        self.qscale_x = None
        self.meta = None
        self.x6 = None  # activation as a tile-ordered operand buffer (codes and outlier values), see MixedQLinear
        self.group_size = group_size
        self.cur_group_elem = 0
        self._members = []      # weak references, in the order the members were built
        self._fused = None      # the concatenated layer (built by the first call), or False: this group cannot be fused
        self._fused_key = None
        self._outs = None       # column views of the group's result, one per member, until the last member was called

    def __getstate__(self):     # (weak references and device tensors of a forward in flight do not travel)
        state = dict(self.__dict__)
        state.update(_members=[], _fused=None, _fused_key=None, _outs=None, qint_x=None, fp_x=None, qscale_x=None,
                     meta=None, x6=None, cur_group_elem=0)
        return state

    def register(self, module):
        self._members = [r for r in self._members if r() is not None and r() is not module]
        self._members.append(weakref.ref(module))
        self._fused = None

    def finish(self):
        self.cur_group_elem += 1
        if self.cur_group_elem == self.group_size:
            self.qint_x = None
            self.qscale_x = None
            self.meta = None
            self.fp_x = None
            self.x6 = None
            self._outs = None
            self.cur_group_elem = 0

    def _members_key(self, mods):
        return tuple((id(m), m.int_weight.data_ptr(), m.int_weight._version, m.weights_scales.data_ptr(),
                      m.int_indices._version, m.fp_indices._version, bool(m.six_bit_path), m.six_bit_min_rows,
                      m.tile8_min_rows) for m in mods)

    def _fused_layer(self):
        """The members' weights as one MixedQLinear (None when the group is not complete or not compatible).  Built
        once; afterwards the members' buffers are row slices of the concatenated buffers, so the group holds one
        copy of the reference's buffers, and the tile-ordered copy exists once, for the whole group."""
        mods = [r() for r in self._members]
        if len(mods) != self.group_size or any(m is None for m in mods) or self.group_size < 2:
            return None
        if self._fused is not None and self._fused is not False and self._fused_key == self._members_key(mods):
            return self._fused
        if self._fused is False and self._fused_key == self._members_key(mods):
            return None
        first = mods[0]
        ok = all(m.fused and not m._row_major_released and m.int_features_num > 0 and m.int_weight.is_cuda and
                 m.int_weight.device == first.int_weight.device and m.in_features == first.in_features and
                 m.bits == first.bits and m.symmetric == first.symmetric and m.dtype == first.dtype and
                 m.fp_features_num == first.fp_features_num and (m.bias is None) == (first.bias is None) and
                 m.sym_divisor == first.sym_divisor and m.six_bit_path == first.six_bit_path and
                 m.six_bit_min_rows == first.six_bit_min_rows and m.tile8_min_rows == first.tile8_min_rows
                 for m in mods)
        ok = ok and all(torch.equal(m.fp_indices, first.fp_indices) and torch.equal(m.int_indices, first.int_indices)
                        for m in mods[1:])
        if not ok:
            self._fused, self._fused_key = False, self._members_key(mods)
            return None
        fused = _concatenate_layers(mods)
        fused.six_bit_path = first.six_bit_path
        fused.six_bit_min_rows, fused.tile8_min_rows = first.six_bit_min_rows, first.tile8_min_rows
        fused.sym_divisor = first.sym_divisor
        fused.transient_tiled_copy = first.transient_tiled_copy
        # the members' buffers become row slices (contiguous) of the concatenated ones: no second copy
        lo = 0
        for m in mods:
            hi = lo + m.out_features
            m.int_weight = fused.int_weight[lo:hi]
            m.weights_scales = fused.weights_scales[lo:hi]
            if m.fp_features_num > 0:
                m.fp_weight = fused.fp_weight[lo:hi]
            if not m.symmetric:
                m.reduced_w = fused.reduced_w[:, lo:hi]
            if m.bias is not None:
                m.bias = fused.bias[lo:hi]
            m._w6 = m._w6_key = None      # a member's own tile-ordered copy is not read while the group serves it
            m._descs.clear()
            lo = hi
        self._fused, self._fused_key = fused, self._members_key(mods)
        self._split = [m.out_features for m in mods]
        return fused

    def group_forward(self, member, x2):
        """Output [rows, member.out_features] of `member` for the 2-D input x2 through the fused group, or None when
        this call is not served that way (the caller then takes the member's own path)."""
        if self.cur_group_elem == 0:
            self._outs = None
            fused = self._fused_layer()
            if fused is None:
                return None
            with device_guard(x2.device):
                whole = fused._forward_one_call(x2)
            if whole is None:
                return None
            mods = [r() for r in self._members]
            self._outs = {id(m): o for m, o in zip(mods, whole.split(self._split, dim=-1))}
        if self._outs is None or id(member) not in self._outs:
            return None
        out = self._outs[id(member)]
        self.finish()
        return out


def _concatenate_layers(layers):
    """MixedQLinear whose output columns are those of `layers` (same input, outlier columns, bits, symmetry and
    dtype), one after the other."""
    first = layers[0]
    total = sum(m.out_features for m in layers)
    fused = MixedQLinear(first.in_features, total, None, fp_features_num=first.fp_features_num,
                         symm=first.symmetric, bits=first.bits, dtype=first.dtype, fused=True, allocate=False)
    fused.int_weight = torch.cat([m.int_weight for m in layers], dim=0).contiguous()
    fused.weights_scales = torch.cat([m.weights_scales for m in layers], dim=0).contiguous()
    fused.int_indices = first.int_indices.clone()
    fused.fp_indices = first.fp_indices.clone()
    if first.fp_features_num > 0:
        fused.fp_weight = torch.cat([m.fp_weight for m in layers], dim=0).contiguous()
    if not first.symmetric:
        fused.reduced_w = torch.cat([m.reduced_w for m in layers], dim=1).contiguous()
    fused.bias = None if first.bias is None else torch.cat([m.bias for m in layers], dim=0).contiguous()
    return fused


class MixedQLinear(torch.nn.Module):
    """The reference's layer (qlinear.py:40-145) on the HIP kernels.

    Asymmetric calls with at least `six_bit_min_rows` token rows (everything above decode size) read both
    operands in tile order (`tiled_path`; the quantize kernel writes the activation that way, the weights
    get a second, repacked copy on first use), so every operand cache line is fetched once per tile.
    W4A4: the int4 products run on the 6-bit (E2M3) matrix-core instructions, which have twice the int8 rate:
    levels code + 8 are exact E2M3 numbers and the integer accumulator is recovered exactly (needs
    int_features % 128 == 0; 0.75 bytes per weight).  W8A8: int8 MFMA as before (int_features % 64 == 0;
    1 byte per weight).  Both need fp_features % 32 == 0 and ascending int_indices and give the output bits
    of the row-major kernels; `six_bit_path = False` turns them off."""

    # Profiling hook: a torch.cuda.Event (created, i.e. recorded once before) stored here is recorded between the
    # quantize launch and the GEMM launch of the next forward that goes through the one-call path, then cleared.
    mid_event = None

    six_bit_min_rows = 33    # up to 32 rows the weight-streaming decode kernel on the packed int4 weights is the right one
    tile8_min_rows = 33      # the same switch for 8 bits (the tile-ordered kernel itself takes any row count)
    fuse_shared_groups = True   # members of a SharedQuantizedInput group run as one quantize + one GEMM (see there)
    # Memory policy: True = the tile-ordered weight copy is NOT kept.  Every call of more than 32 rows repacks the
    # reference's buffers into a temporary operand buffer (one launch, the buffer goes back to torch's allocator
    # behind the GEMM, so consecutive layers reuse the same block) and runs the same tile-ordered GEMM: output bits
    # unchanged, weights resident once (the reference's layout), each such call longer by the repacking
    # (see weight_bytes(); set on the class for every layer or on single modules).
    transient_tiled_copy = False

    def __init__(self, in_features, out_features, shared_input=None,
                 fp_features_num=0, symm=False, bits=4, dtype=torch.float16, fused=True, allocate=True):
        """allocate=False: the buffers are registered empty (the caller assigns them); otherwise as in the reference."""
        super().__init__()
        self.six_bit_path = True
        self._w6 = None
        self._w6_key = None
        self._row_major_released = False
        self._streams = None
        self.fp_features_num = fp_features_num
        self.int_features_num = in_features - fp_features_num
        self.in_features = in_features
        self.out_features = out_features
        self.symmetric = symm
        self.bits = bits
        self.shared_input = shared_input
        self.dtype = dtype
        self.fused = fused
        self.sym_divisor = 1 << ((bits - 1) - 1)
        rows = out_features if allocate else 0
        self.register_buffer('weights_scales', torch.zeros((rows, 1), dtype=dtype))
        if bits == 4:
            self.register_buffer('int_weight', torch.zeros((rows, self.int_features_num // 2), dtype=torch.uint8))
        else:
            self.register_buffer('int_weight', torch.zeros((rows, self.int_features_num), dtype=torch.int8))
        self.register_buffer('bias', torch.zeros((rows,), dtype=dtype))
        self.register_buffer('int_indices', torch.zeros((self.int_features_num if allocate else 0,), dtype=torch.long))
        self.register_buffer('fp_indices', torch.zeros((fp_features_num if allocate else 0,), dtype=torch.long))
        if fp_features_num > 0:
            self.register_buffer('fp_weight', torch.zeros((rows, fp_features_num), dtype=dtype))
        if not symm:
            self.register_buffer('reduced_w', torch.zeros((1, rows), dtype=dtype))
        self._colmap = None
        self._colmap_key = None
        self._descs = _PerObjectCache()
        if shared_input is not None and hasattr(shared_input, "register"):
            shared_input.register(self)

    def _apply(self, fn, recurse=True):
        """`.to()` / `.half()` / `.bfloat16()` convert the floating-point buffers; `dtype` (a plain attribute in the
        reference, qlinear.py:52, fixed at construction) follows them, so that a converted module computes in the
        type its buffers now have instead of failing on the mismatch."""
        out = super()._apply(fn, recurse)
        if self.weights_scales.dtype in (torch.float16, torch.bfloat16):
            self.dtype = self.weights_scales.dtype
        return out

    # -- cached column map: rebuilt when the index buffers move or are written in place
    def _column_map(self):
        key = (self.int_indices.data_ptr(), self.fp_indices.data_ptr(), self.int_indices._version,
               self.fp_indices._version, self.int_indices.device)
        if self._colmap is None or self._colmap_key != key:
            self._colmap = asymmetric.build_colmap(self.int_indices, self.fp_indices, self.in_features)
            self._colmap_key = key
            self._streams = None
        return self._colmap

    # -- 6-bit matrix-core path: eligibility and the cached weight operand
    def _six_bit_ok(self, rows):
        """True if this call takes the tile-ordered path (6-bit matrix-core GEMM for 4 bits, int8 for 8 bits)."""
        if not (self.six_bit_path and self.fused and self.bits in (4, 8)):
            return False
        if self.symmetric and self.dtype != torch.float16:      # symmetric activations are fp16 (as in the reference)
            return False
        k_multiple = 128 if self.bits == 4 else 64
        min_rows = self.six_bit_min_rows if self.bits == 4 else self.tile8_min_rows
        if rows < min_rows or self.int_features_num % k_multiple != 0 or self.fp_features_num % 32 != 0:
            return False
        if self.bits == 4 and self.int_features_num > 74496:   # the 6-bit path's fp32 sums are exact up to here
            return False
        return self._streams_flag()

    def _weight6(self):
        if self._row_major_released:
            return self._w6
        fp_w = self.fp_weight if self.fp_features_num > 0 else \
            torch.empty((self.out_features, 0), dtype=self.dtype, device=self.int_weight.device)
        if self.transient_tiled_copy:    # a fresh buffer per call, never kept
            self._w6 = self._w6_key = None
            if self.bits == 4:
                return matmul.pack_weight_fp6(self.int_weight, fp_w, self._column_map())
            return matmul.pack_weight_tile8(self.int_weight, fp_w)
        key = (self.int_weight.data_ptr(), self.int_weight._version, fp_w.data_ptr(), fp_w._version,
               self.int_weight.device, self._column_map().data_ptr())
        if self._w6 is None or self._w6_key != key:
            if self.bits == 4:    # in the column map's in-place order, as the activation is quantized
                self._w6 = matmul.pack_weight_fp6(self.int_weight, fp_w, self._column_map())
            else:
                self._w6 = matmul.pack_weight_tile8(self.int_weight, fp_w)
            self._w6_key = key
        return self._w6

    # -- which copies of the weights stay resident
    def weight_bytes(self):
        """Bytes of weight storage this module holds on its device: the reference's buffers (int_weight + fp_weight,
        qlinear.py:53-78 of the reference) and the tile-ordered copy the prefill GEMMs read (made by the first call
        that takes that path; 0.75 byte per int4 weight, 1 per int8 weight, outlier columns included)."""
        fp = self.fp_weight if self.fp_features_num > 0 else None
        row_major = self.int_weight.numel() * self.int_weight.element_size() + \
            (fp.numel() * fp.element_size() if fp is not None else 0)
        tiled = self._w6.numel() * self._w6.element_size() if self._w6 is not None else 0
        packed = self.out_features * (self.int_features_num * self.bits // 8 +
                                      self.fp_features_num * self.weights_scales.element_size())
        return {"row_major": row_major, "tiled": tiled, "reference_layout": packed}

    def release_tiled_weights(self):
        """Drop the tile-ordered copy and stop using the tile-ordered paths: every call reads the reference's
        buffers (int8-MFMA GEMM above 32 rows: same output bits, about half the 6-bit path's rate for W4A4)."""
        if self._row_major_released:
            raise RuntimeError("the tile-ordered copy is the only one this module holds")
        self.six_bit_path = False
        self._w6 = self._w6_key = None
        self._descs.clear()

    def release_row_major_weights(self):
        if self.transient_tiled_copy:
            raise RuntimeError("transient_tiled_copy repacks the row-major weights on every call: they cannot be released")
        return self._release_row_major_weights()

    def _release_row_major_weights(self):
        """Keep only the tile-ordered copy: int_weight and fp_weight become empty tensors and EVERY call, down to
        one row, takes the tile-ordered path (same output bits above 32 rows; up to 32 rows equal within rounding
        of the fp32 sums, and slower than the weight-streaming kernel, which reads the packed nibbles).  The
        module can no longer be saved in the reference's checkpoint format or moved to another device."""
        if not self._six_bit_ok(max(self.six_bit_min_rows, self.tile8_min_rows)):
            raise RuntimeError("this layer does not take the tile-ordered path (shape, dtype or column map)")
        w6 = self._weight6()
        self._row_major_released = True
        self.six_bit_min_rows = self.tile8_min_rows = 1
        dev = self.int_weight.device
        self.int_weight = torch.empty((0,), dtype=self.int_weight.dtype, device=dev)
        if self.fp_features_num > 0:
            self.fp_weight = torch.empty((0,), dtype=self.dtype, device=dev)
        self._descs.clear()
        assert self._weight6() is w6

    def _streams_flag(self):
        """True if the column map selects the streaming quantize kernel (cached; one synchronisation per map)."""
        colmap = self._column_map()
        if self._streams is None:
            flag = getattr(colmap, "_quik_streams", None)
            if flag is None:
                flag = asymmetric.colmap_streams(colmap, self.int_features_num, self.fp_features_num)
            # the ops that need the streaming kernel look for the answer on the tensor (asymmetric.check_mapped_args)
            colmap._quik_shape = (self.in_features, self.int_features_num, self.fp_features_num)
            colmap._quik_streams = flag
            self._streams = flag
        return self._streams

    # -- one library call per forward (quik_layer_forward): the layer's buffers described once
    def _descriptor(self, tiled):
        """(ctypes quik_layer, workspace sizes by row count) for this module, with or without the tile-ordered weight
        copy; cached, rebuilt when a buffer moves or is written in place."""
        bufs = (self.int_weight, self.weights_scales, self.int_indices, self.fp_indices,
                self.reduced_w if not self.symmetric else None, self.fp_weight if self.fp_features_num > 0 else None,
                self.bias)
        # (the scalar switches below are baked into the descriptor too: changing one after a forward rebuilds it)
        key = tuple((b.data_ptr(), b._version) if b is not None else None for b in bufs) + \
            (self.six_bit_min_rows, self.tile8_min_rows, float(self.sym_divisor), bool(self.six_bit_path))
        transient = tiled and self.transient_tiled_copy and not self._row_major_released
        if transient:
            # the cached descriptor of the row-major form, copied, with this call's temporary operand buffer
            base, sizes = self._descriptor(False)
            d = L.QuikLayer.from_buffer_copy(base)
            w6 = self._weight6()
            d.tiled_weight = w6.data_ptr()
            d._keep = w6     # (alive until the caller drops the descriptor, i.e. behind the launch)
            return d, self._descs.setdefault("transient_sizes", {})
        entry = self._descs.get(tiled)
        if entry is None or entry[0] != key:
            w6 = self._weight6() if tiled else None
            colmap = self._column_map()
            d = L.QuikLayer()
            d.struct_bytes = ctypes.sizeof(L.QuikLayer)
            d.bits, d.symmetric = self.bits, int(self.symmetric)
            d.dtype = L.QUIK_F16 if self.dtype == torch.float16 else L.QUIK_BF16
            d.in_features, d.num_int, d.num_fp = self.in_features, self.int_features_num, self.fp_features_num
            d.out_features = self.out_features
            d.sym_divisor = float(self.sym_divisor)
            d.colmap_streams = int(self._streams_flag())
            d.tiled_min_rows = self.six_bit_min_rows if self.bits == 4 else self.tile8_min_rows
            d.colmap, d.weights_scales = colmap.data_ptr(), bufs[1].data_ptr()
            d.int_weight = bufs[0].data_ptr() if bufs[0].numel() > 0 else None
            d.reduced_w = bufs[4].data_ptr() if bufs[4] is not None else None
            d.fp_weight = bufs[5].data_ptr() if bufs[5] is not None and bufs[5].numel() > 0 else None
            d.bias = bufs[6].data_ptr() if bufs[6] is not None and bufs[6].numel() > 0 else None
            d.tiled_weight = w6.data_ptr() if w6 is not None else None
            entry = self._descs[tiled] = (key, d, {}, (colmap, w6))   # the tensors the pointers refer to stay alive
        return entry[1], entry[2]

    def _forward_one_call(self, x2):
        """quantize + fused GEMM through quik_layer_forward; None when this call is not one it serves."""
        if x2.dtype != self.dtype or x2.data_ptr() % 16 != 0 or self.dtype not in (torch.float16, torch.bfloat16):
            return None
        if self.symmetric and not (self.dtype == torch.float16 and self._streams_flag()):
            return None
        rows = x2.shape[0]
        if rows == 0:
            return None
        tiled = self._six_bit_ok(rows)
        desc, ws_bytes = self._descriptor(tiled)
        lib = L.load()
        nbytes = ws_bytes.get(rows)
        if nbytes is None:
            nbytes = ws_bytes[rows] = lib.quik_layer_workspace_bytes(ctypes.byref(desc), rows)
        ws = torch.empty((nbytes,), dtype=torch.uint8, device=x2.device)
        out = torch.empty((rows, self.out_features), dtype=self.dtype, device=x2.device)
        sk, sk_bytes = matmul._splitk_workspace(x2.device, rows, self.out_features, self.int_features_num, self.bits) \
            if tiled else (None, 0)
        mid = None
        if self.mid_event is not None:   # profiling hook, see the class comment
            mid, self.mid_event = self.mid_event.cuda_event, None
        L.check(lib.quik_layer_forward(ctypes.byref(desc), x2.data_ptr(), rows, ws.data_ptr(), nbytes, L.ptr(sk),
                                       sk_bytes, out.data_ptr(), mid, L.stream()), "MixedQLinear.forward")
        return out

    def _quantize_input(self, x, shared_input):
        if self.symmetric and x.dtype == torch.float16 and x.data_ptr() % 16 == 0 and self._streams_flag():
            # the op sequence of the next branch in one kernel, same bits
            shared_input.qint_x, shared_input.qscale_x, shared_input.fp_x = symmetric.quantize_mapped(
                x, self._column_map(), self.int_features_num, self.fp_features_num, self.bits, self.sym_divisor, False)
            if self.fp_features_num == 0:
                shared_input.fp_x = None
        elif self.symmetric:
            if self.fp_features_num > 0:
                int_x = x[:, self.int_indices].contiguous()
                shared_input.fp_x = x[:, self.fp_indices].contiguous()
            else:
                int_x = x
                shared_input.fp_x = None
            shared_input.qscale_x = (torch.max(torch.abs(int_x), dim=1)[0].unsqueeze(1) /
                                     self.sym_divisor).to(torch.float16)
            shared_input.qint_x = symmetric.quantize(int_x, shared_input.qscale_x, self.bits)
        else:
            shared_input.qint_x, shared_input.meta, shared_input.fp_x = asymmetric.quantize_mapped(
                x, self._column_map(), self.int_features_num, self.fp_features_num, self.bits)

    def forward(self, x):
        if self.int_features_num <= 0:
            return torch.nn.functional.linear(x, self.fp_weight, self.bias)
        if not x.is_cuda:
            raise RuntimeError("MixedQLinear.forward needs a tensor on the GPU; there is no CPU path")
        lead = x.shape[:-1] if x.dim() == 3 else (1, x.shape[0])
        x2 = x.reshape(-1, x.shape[-1])
        if not x2.is_contiguous():
            x2 = x2.contiguous()
        if self.fused and (self.shared_input is None or self.shared_input.group_size == 1):
            with device_guard(x.device):
                output = self._forward_one_call(x2)
            if output is not None:
                return output.reshape(*lead, self.out_features)
        if self.fused and self.fuse_shared_groups and self.shared_input is not None and \
                self.shared_input.group_size > 1 and hasattr(self.shared_input, "group_forward"):
            output = self.shared_input.group_forward(self, x2)    # one quantize + one GEMM for the whole group
            if output is not None:
                return output.reshape(*lead, self.out_features)
        shared_input = self.shared_input if self.shared_input is not None else SharedQuantizedInput(1)
        with device_guard(x.device):
            if x2.data_ptr() % 16 == 0 and (not self.symmetric or x2.dtype == torch.float16) \
                    and self._six_bit_ok(x2.shape[0]):
                quantize6 = asymmetric.quantize_mapped_fp6 if self.bits == 4 else asymmetric.quantize_mapped_tile8
                linear6 = matmul.mixed_linear_fp6 if self.bits == 4 else matmul.mixed_linear_tile8
                if shared_input.x6 is None:
                    if self.symmetric:
                        shared_input.x6, shared_input.qscale_x, _ = symmetric.quantize_mapped(
                            x2, self._column_map(), self.int_features_num, self.fp_features_num, self.bits,
                            self.sym_divisor, True)
                    else:
                        shared_input.x6, shared_input.meta = quantize6(
                            x2, self._column_map(), self.int_features_num, self.fp_features_num)
                output = linear6(shared_input.x6, self._weight6(),
                                 shared_input.qscale_x if self.symmetric else shared_input.meta,
                                 self.weights_scales, None if self.symmetric else self.reduced_w, self.bias,
                                 x2.shape[0], self.out_features, self.int_features_num, self.fp_features_num,
                                 self.dtype)
                shared_input.finish()
                return output.reshape(*lead, self.out_features)
            if self._row_major_released:
                raise RuntimeError("this call needs the row-major weights, which release_row_major_weights() dropped "
                                   "(input dtype / alignment, or fused / six_bit_path switched off)")
            if shared_input.qint_x is None:
                self._quantize_input(x2, shared_input)
            if self.fused:
                output = matmul.mixed_linear(
                    shared_input.qint_x, self.int_weight,
                    shared_input.qscale_x if self.symmetric else shared_input.meta,
                    self.weights_scales, None if self.symmetric else self.reduced_w,
                    shared_input.fp_x if self.fp_features_num > 0 else None,
                    self.fp_weight if self.fp_features_num > 0 else None,
                    self.bias, self.bits, self.dtype)
            else:
                output = self._forward_unfused(shared_input)
        shared_input.finish()
        return output.reshape(*lead, self.out_features)

    def _forward_unfused(self, shared_input):
        """The reference's op sequence (qlinear.py:122-145)."""
        rows = shared_input.qint_x.shape[0]
        if self.fp_features_num > 0:
            fp_result = torch.nn.functional.linear(shared_input.fp_x, self.fp_weight, self.bias)
        elif self.bias is not None:
            fp_result = self.bias.repeat(rows, 1)
        else:
            fp_result = torch.zeros((rows, self.out_features), dtype=self.dtype, device=self.int_weight.device)
        if self.bits == 4:
            int_result = matmul.int4Matmul(shared_input.qint_x, self.int_weight)
        else:
            int_result = matmul.int8Matmul(shared_input.qint_x, self.int_weight)
        if self.symmetric:
            return symmetric.dequantize(int_result, shared_input.qscale_x,
                                        self.weights_scales.reshape(1, -1).contiguous(), fp_result.contiguous(), 32)
        return asymmetric.dequantize(int_result, shared_input.meta, self.weights_scales, self.reduced_w,
                                     fp_result.contiguous(), self.bits)

    @staticmethod
    def from_float(module: torch.nn.Linear, weight_matrix, weights_scales, shared_input=None,
                   fp_indices=None, symm=False, bits=4, fused=True):
        """Build a MixedQLinear from a float Linear (qlinear.py:150-199).

        `weight_matrix` [out, in] holds the fake-quantized weights (codes * scale on the int
        columns), `weights_scales` [out, 1] the per-output-channel scales, `fp_indices` the
        outlier input columns.  Integer columns are the ascending complement of fp_indices."""
        assert weights_scales.shape == (module.out_features, 1), 'weights_scales should have shape (out_features, 1)'
        assert weight_matrix.shape == (module.out_features, module.in_features)
        assert (symm and bits == 4) or not symm, "Symmetric quantization with 8 bits is not supported"
        int_indices = torch.arange(module.in_features)
        if fp_indices is None or len(fp_indices) == 0:
            fp_indices = torch.tensor([], dtype=int_indices.dtype)
        else:
            fp_indices = fp_indices.to(device='cpu', dtype=int_indices.dtype)
            int_indices = int_indices[~torch.isin(int_indices, fp_indices)]
        assert torch.numel(int_indices) + torch.numel(fp_indices) == module.in_features, \
            'There are some duplication in the fp_indices!'

        mod = MixedQLinear(module.in_features, module.out_features, shared_input,
                           fp_features_num=torch.numel(fp_indices), symm=symm, bits=bits,
                           dtype=weight_matrix.dtype, fused=fused)
        if torch.cuda.is_available():
            weight_matrix = weight_matrix.cuda()
        dev = weight_matrix.device
        mod.weights_scales.copy_(weights_scales.to(weight_matrix.dtype))
        w_int = weight_matrix[:, int_indices.to(dev)]
        rounded = (w_int / weights_scales.to(dev)).round()
        if bits == 4:
            mod.int_weight.copy_(pack_to_i4(rounded.to(torch.int8)).cpu())
        else:
            mod.int_weight.copy_(rounded.to(torch.int8).cpu())
        if not symm:
            reduced_w = torch.sum(w_int.float(), dim=1, keepdim=True).to(weight_matrix.dtype)
            mod.reduced_w.copy_(reduced_w.t().cpu())
        if module.bias is not None:
            mod.bias.copy_(module.bias)
        else:
            mod.bias = None
        mod.int_indices.copy_(int_indices)
        mod.fp_indices.copy_(fp_indices)
        if mod.fp_features_num > 0:
            mod.fp_weight.copy_(weight_matrix[:, fp_indices.to(dev)].to(weight_matrix.dtype))
        return mod


class FusedMixedQLinearGroup(torch.nn.Module):
    """One quantize and ONE GEMM for layers that read the same input (q/k/v, gate/up).

    The reference shares only the quantized activation between such layers
    (SharedQuantizedInput, qlinear.py:21-37; experiments/llama.py:402-411) and still runs one
    GEMM per layer.  Here their packed weights are concatenated along the output dimension, so
    narrow members (Llama-2-70B k/v: 1024 columns) ride in the tiles of the wide one.  The
    per-column arithmetic is that of the member layers, so the outputs are bit-identical to theirs.
    forward(x) returns one tensor per member, views of a single [.., sum(out_features)] result."""

    def __init__(self, layers):
        super().__init__()
        layers = list(layers)
        first = layers[0]
        for m in layers[1:]:
            same = (m.in_features == first.in_features and m.bits == first.bits and m.symmetric == first.symmetric
                    and m.dtype == first.dtype and m.fp_features_num == first.fp_features_num
                    and torch.equal(m.fp_indices.cpu(), first.fp_indices.cpu())
                    and (m.bias is None) == (first.bias is None))
            if not same:
                raise ValueError("FusedMixedQLinearGroup: members must agree in input size, outlier columns, "
                                 "bits, symmetry, dtype and presence of a bias")
        self.split_sizes = [m.out_features for m in layers]
        self.fused = _concatenate_layers(layers)

    def forward(self, x):
        return self.fused(x).split(self.split_sizes, dim=-1)


class Linear8bit(torch.nn.Module):
    """Plain int8 GEMM layer of the reference's benchmark scaffolding (qlinear.py:202-228)."""

    def __init__(self, in_features, out_features, bias=None):
        super().__init__()
        self.in_features = in_features
        self.out_features = out_features
        self.register_buffer('int_weight', torch.zeros((out_features, in_features), dtype=torch.int8))
        self.register_buffer('bias', torch.zeros((out_features,), dtype=torch.float16))
        if bias is not None:
            self.bias.copy_(bias)
        else:
            self.bias = None

    def forward(self, x):
        if x.dim() == 3:
            x = x[0]
        out = matmul.int8Matmul(x.to(torch.int8).contiguous(), self.int_weight).to(torch.float16)
        return out if self.bias is None else out.add(self.bias)


class Linear4bit(torch.nn.Module):
    """Plain int4 GEMM layer of the reference's benchmark scaffolding (qlinear.py:231-256)."""

    def __init__(self, in_features, out_features, bias=None):
        super().__init__()
        self.in_features = in_features
        self.out_features = out_features
        self.register_buffer('int_weight', torch.zeros((out_features, in_features // 2), dtype=torch.uint8))
        self.register_buffer('bias', torch.zeros((out_features,), dtype=torch.float16))
        if bias is not None:
            self.bias.copy_(bias)
        else:
            self.bias = None

    def forward(self, x):
        if x.dim() == 3:
            x = x[0]
        x_int4 = x[:, :x.size(1) // 2].to(torch.uint8).contiguous()
        out = matmul.int4Matmul(x_int4, self.int_weight).to(torch.float16)
        return out if self.bias is None else out.add(self.bias)
