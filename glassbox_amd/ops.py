"""Python bindings of the device kernels (csrc/hip/*.hip), through ctypes.

Each function checks devices, dtypes, contiguity and shapes, then passes raw
pointers and the current HIP stream to the kernel's C entry point.  There is no
CPU path and no library fallback: a missing GPU or a library that cannot be
built raises.  Tensors are torch tensors only because torch is the allocator
and stream owner; no torch operator computes anything here.
"""
from __future__ import annotations

import ctypes as C
import functools
import struct
from typing import List, Optional, Sequence

import torch

from . import build

F32, BF16 = 0, 1
_vp, _i, _f = C.c_void_p, C.c_int, C.c_float


class KernelError(RuntimeError):
    pass


def require_gpu() -> None:
    if not torch.cuda.is_available():
        raise KernelError("no GPU is visible: glassbox_amd runs on a gfx950 GPU only and has no CPU path")


def dtype_code(t: torch.Tensor) -> int:
    if t.dtype == torch.float32:
        return F32
    if t.dtype == torch.bfloat16:
        return BF16
    raise KernelError(f"unsupported element type {t.dtype}")


_SIGS = {
    "elementwise": {
        "gb_embed": [_vp, _i, _vp, _vp, _i, _i, _i, _f, _i, _vp],
        "gb_rmsnorm": [_vp, _vp, _i, _vp, _vp, _i, _i, _i, _f, _vp],
        "gb_rope_table": [_vp, _vp, _vp, _vp, _i, _i, _vp],
        # qkv, dtype, stride, cos, sin, slots, k, v, n, nh, nkv, hd, page, rotate, v_rows, q_start, q_len, pos0,
        # seq_base, n_seqs, max_q_len, stream
        "gb_rope_store": [_vp, _i, _i, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _vp, _vp, _vp, _i, _i, _i, _vp],
        "gb_silu_mul": [_vp, _vp, _i, _i, _i, _vp],
        "gb_copy_rows": [_vp, C.c_longlong, _vp, _vp, _i, _vp],
        # qk, dtype, stride, bias_q, bias_k, w_q, w_k, eps, slots, k, v, n, nh, nkv, hd, page, v_off, stream
        "gb_qk_norm_store": [_vp, _i, _i, _vp, _vp, _vp, _vp, _f, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _vp],
        "gb_add_bias": [_vp, _vp, _i, _i, _vp],
        "gb_scale_rows": [_vp, _f, C.c_longlong, _vp],
        # a, lda, w, ldw, c, ldc, operand dtype, result dtype, M, N, K, accumulate, stream
        "gb_gemm_plain": [_vp, _i, _vp, _i, _vp, _i, _i, _i, _i, _i, _i, _i, _vp],
        # table, pairs, dtype, ids, x, n, d, vocab, buckets, mul_prev, mul_cur, tok_seq, q_start, q_len, pos0, state slots,
        # prev, copies, stream
        "gb_embed_pairs": [_vp, _vp, _i, _vp, _vp, _i, _i, _i, _i, C.c_longlong, C.c_longlong, _vp, _vp, _vp, _vp, _vp, _vp,
                           _i, _vp],
        # gate_up, its dtype, ld, act, its dtype, n, inter, limit, alpha, stream
        "gb_glu_clamped": [_vp, _i, _i, _vp, _i, _i, _i, _f, _f, _vp],
        # x, y, alpha, bias, n, d, stream
        "gb_axpy_rows": [_vp, _vp, _f, _vp, _i, _i, _vp],
    },
    "shortconv": {
        # proj, dtype, stride, wconv, taps, state, tok_seq, q_start, pos0, state slots, cos, sin, rot, eps, norm, out,
        # out stride, hd, slots, k, v, page, n, nh, nkv, dim, vdim, update_state, stream
        "gb_conv_heads": [_vp, _i, _i, _vp, _i, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _f, _i, _vp, _i, _i, _vp, _vp, _vp, _i,
                          _i, _i, _i, _i, _i, _i, _vp],
        # proj, dtype, stride, state, q_start, q_len, state slots, requests, channels, taps, stream
        "gb_conv_state": [_vp, _i, _i, _vp, _vp, _vp, _vp, _i, _i, _i, _vp],
    },
    "headmix": {
        # x, ldx, w, taps, state, tok_seq, q_start, pos0, state slots, out, dtype, ldo, n, d, single, stream
        "gb_time_conv": [_vp, _i, _vp, _i, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _vp],
        # in, dtype, ld, n, eps, (col, d, gamma, out, ldo) twice, stream
        "gb_norm_slices": [_vp, _i, _i, _i, _f, _i, _i, _vp, _vp, _i, _i, _i, _vp, _vp, _i, _vp],
        # q, ldq, kv, ldkv, krot, ldr, dtype, cos, sin, rot, out, ldo, hd, slots, k, v, page, n, H, dim, rot_dim, vdim, stream
        "gb_latent_heads": [_vp, _i, _vp, _i, _vp, _i, _i, _vp, _vp, _i, _vp, _i, _i, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _vp],
        # proj, dtype, ld, wq, wk, eps, coef, every, positions, out, ldo, hd, slots, k, v, page, n, H, G, dim, vdim, stream
        "gb_diff_heads": [_vp, _i, _i, _vp, _vp, _f, _f, _i, _vp, _vp, _i, _i, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _vp],
        # att, its dtype, lda, hd, lambda, mult, eps, out, its dtype, ldo, n, H, vdim, stream
        "gb_diff_combine": [_vp, _i, _i, _i, _vp, _f, _f, _vp, _i, _i, _i, _i, _i, _vp],
        # att, lda, hd, gate, ldg, dtype, out, ldo, n, H, vdim, stream
        "gb_gate_heads": [_vp, _i, _i, _vp, _i, _i, _vp, _i, _i, _i, _i, _vp],
        # z, ldz, coef, eps, out, ldo, dtype, n, d, stream
        "gb_poly_norm": [_vp, _i, _vp, _f, _vp, _i, _i, _i, _i, _vp],
        # x, y, slices, slice stride, g, eps, rounded, dtype, n, d, conv w, taps, state, tok_seq, pos0, state slots, stream
        "gb_norm_add": [_vp, _vp, _i, C.c_longlong, _vp, _f, _vp, _i, _i, _i, _vp, _i, _vp, _vp, _vp, _vp, _vp],
    },
    "tanhmix": {
        # x, ldx, rows, alpha, w, b, out, its dtype, ldo, n, d, stream
        "gb_tanh_norm": [_vp, _i, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _vp],
        # x, y, slices, slice stride, alpha, w, b, next alpha, w, b, h, its dtype, n, d, stream
        "gb_tanh_norm_add": [_vp, _vp, _i, C.c_longlong, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _vp],
        # proj, dtype, ld, bias, wconv, sums, state, tok_seq, q_start, pos0, state slots, flags and taps, wq, wk, eps, cos, sin,
        # rot, mag, out, ldo, hd, slots, k, v, page, n, H, G, dk, dv, stream
        "gb_qk_heads": [_vp, _i, _i, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _vp, _vp, _f, _vp, _vp, _i, _f, _vp, _i,
                        _i, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _vp],
        # proj, dtype, ld, bias, state, q_start, q_len, state slots, requests, channels, taps, stream
        "gb_qk_conv_state": [_vp, _i, _i, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _vp],
        # att, lda, hd, gate, ldg, one gate a head, dtype, out, ldo, n, H, dv, stream
        "gb_gate_rows": [_vp, _i, _i, _vp, _i, _i, _i, _vp, _i, _i, _i, _i, _vp],
    },
    "moe": {        # z, ldz, n, experts, correction, top, scale, shared, combine, ids, weights, stream
        "gb_moe_route": [_vp, _i, _i, _i, _vp, _i, _f, _i, _vp, _vp, _vp, _vp],
        # z, ldz, n, experts, correction, top, scale, shared (0, 1 gate, 2 whole), softmax, renorm, groups, kept groups,
        # combine, ids, weights, stream
        "gb_moe_route_by": [_vp, _i, _i, _i, _vp, _i, _f, _i, _i, _i, _i, _i, _vp, _vp, _vp, _vp],
        # z, its dtype, ld, combine, its columns, act, its dtype, lda, n, inter, experts, ff, stream
        "gb_moe_relu2_units": [_vp, _i, _i, _vp, _i, _vp, _i, _i, _i, _i, _i, _i, _vp],
        # gate_up, its dtype, ld, combine, its columns, act, its dtype, n, inter, experts, ff, stream
        "gb_moe_gated_units": [_vp, _i, _i, _vp, _i, _vp, _i, _i, _i, _i, _i, _vp],
        # ids, n, top, experts, rows a tile, tiles, counts, rows, pos, map, stream
        "gb_moe_sort": [_vp, _i, _i, _i, _i, _i, _vp, _vp, _vp, _vp, _vp],
        # y, ldy, pos, weights, top, y_shared, its stride, gates, their stride, out, ldo, accumulate, n, d, rows of y, stream
        "gb_moe_combine": [_vp, _i, _vp, _vp, _i, _vp, _i, _vp, _i, _vp, _i, _i, _i, _i, _i, _vp],
    },
    "streams": {
        # X, stream stride, streams, w_in, gamma, gamma dtype, rows, out, out dtype, sum, m, d, eps, mix, w_out, y, stream
        "gb_streams_norm": [_vp, C.c_longlong, _i, _vp, _vp, _i, _vp, _vp, _i, _vp, _i, _i, _f, _vp, _vp, _vp, _vp],
        "gb_streams_mix": [_vp, C.c_longlong, _i, _vp, _vp, _vp, C.c_longlong, _vp],
    },
    "linear_attention": {
        # q, k, decays, head decays, v, v dtype, v stride, out, state, q_start, q_len, pos0, state slots, requests, heads,
        # dk, dv, state columns a head, decay a head (0/1), segments, rows a segment, workspace, its floats, stream
        "gb_linear_scan": [_vp, _vp, _vp, _vp, _vp, _i, _i, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _i, _vp,
                           C.c_longlong, _vp],
        # z, ldz, bias_i, bias_f, cap, coef, state, floats a head, where m lies, q_start, q_len, pos0, state slots,
        # requests, heads, rows, every request one row (0/1), stream
        "gb_mlstm_gates": [_vp, _i, _vp, _vp, _f, _vp, _vp, C.c_longlong, C.c_longlong, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _vp],
        # proj, dtype, stride, q_off, k_off, v_off, coef, q32, k32, decay, vext, n, heads, dk, dv, q_scale, stream
        "gb_mlstm_prep": [_vp, _i, _i, _i, _i, _i, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _f, _vp],
        # o, coef, gate, dtype, gate stride, w, out, n, heads, dv, eps, stream
        "gb_mlstm_out": [_vp, _vp, _vp, _i, _i, _vp, _vp, _i, _i, _i, _f, _vp],
        # proj, dtype, stride, q_off, k_off, cos, sin, q32, k32, n, heads, dk, rot, k_scale, stream
        "gb_retention_prep": [_vp, _i, _i, _i, _i, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _f, _vp],
        # proj, dtype, stride, q_off, k_off, low_off, a2, z, a2 bias, q32, k32, decay, n, width, rank, q_scale, 1/tau, stream
        "gb_gla_prep": [_vp, _i, _i, _i, _i, _i, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _f, _f, _vp],
        # o, gate, dtype, gate stride, w, out, n, heads, dv, eps, stream
        "gb_head_norm_gate": [_vp, _vp, _i, _i, _vp, _vp, _i, _i, _i, _f, _vp],
    },
    "gemm_f32": {
        "gb_gemm_f32": [_vp, _i, _vp, _i, _vp, _i, _i, _i, _i, _i, _vp],
        "gb_gemm_f32_by": [_vp, _i, _vp, _i, _vp, _i, _i, _i, _i, _i, _i, _vp],
    },
    "gemm_bf16": {
        # a, lda, w, ldw, c, ldc, c_dtype, M, N, K, epilogue, gamma, gamma_dtype, eps,
        # emit_gamma, emit_gamma_dtype, emit_h, emit_ldh, emit_ss, parts, n_parts, split_ws, split_ws_floats, stream
        "gb_gemm_bf16": [_vp, _i, _vp, _i, _vp, _i, _i, _i, _i, _i, _i, _vp, _i, _f, _vp, _i, _vp, _i, _vp, _vp, _i, _vp,
                         C.c_longlong, _vp],
        # a, lda, rows, w, ldw, distance between groups, up_off, c, ldc, c_dtype, map, tiles, rows a tile, N, K, epilogue, stream
        "gb_gemm_bf16_grouped": [_vp, _i, _vp, _vp, _i, C.c_longlong, _i, _vp, _i, _i, _vp, _i, _i, _i, _i, _i, _vp],
        # a, lda, w, ldw, c, ldc, M, N, K, limit, alpha, plus, stream
        "gb_gemm_bf16_glu": [_vp, _i, _vp, _i, _vp, _i, _i, _i, _i, _f, _f, _f, _vp],
        "gb_gemm_bf16_split_floats": [_i, _i, _i],
        "gb_gemm_bf16_slices": [_i, _i, _i],
        # a, lda, w, ldw, workspace, its floats, M, N, K, stream
        "gb_gemm_bf16_partial": [_vp, _i, _vp, _i, _vp, C.c_longlong, _i, _i, _i, _vp],
        "gb_gemm_bf16_emit_parts": [_i, _i],
        "gb_gemm_bf16_emit_mode": [_i, _i, _i],
        # a, lda, w, ldw, c, ldc, M, N, K, gamma, gamma_dtype, eps, parts, n_parts, cos, sin, slots, k, v,
        # nh, nkv, hd, page, stream
        "gb_gemm_bf16_rope": [_vp, _i, _vp, _i, _vp, _i, _i, _i, _i, _vp, _i, _f, _vp, _i, _vp, _vp, _vp, _vp, _vp,
                              _i, _i, _i, _i, _vp],
    },
    "attention_plain": {
        # q, q_stride, out, out_stride, dtype, positions, tok_seq, tables, table_stride, k, v, n, nh, nkv, hd, page,
        # scale, window, workspace, workspace floats, max_context, stream
        # scale, window, kept first keys, workspace, workspace floats, max_context, grouped, stream
        # scale, window, kept first keys, run of positions, cap, sinks, workspace, workspace floats, max_context, grouped, stream
        "gb_attention_plain": [_vp, _i, _vp, _i, _i, _vp, _vp, _vp, _i, _vp, _vp, _i, _i, _i, _i, _i, _f, _i, _i, _i, _f, _vp,
                               _vp, C.c_longlong, _i, _i, _vp],
        "gb_attention_plain_split_floats": [_i, _i, _i, _i, _i, _i],
    },
    "attention_bf16": {
        # q, q_stride, out, out_stride, ws_acc, ws_ml, positions, tables, table_stride, k, v,
        # n_decode, nh, nkv, hd, page, scale, window, chunk, max_context, stream
        "gb_attention_decode_bf16": [_vp, _i, _vp, _i, _vp, _vp, _vp, _vp, _i, _vp, _vp, _i, _i, _i, _i, _i, _f, _i,
                                     _i, _i, _vp],
        # q, q_stride, out, out_stride, q_start, q_len, pos0, seq_base, n_seqs, max_q_len, max_context, tables,
        # table_stride, k, v, nh, nkv, hd, page, scale, window, first_row, n_rows, part_ws, part_floats, stream
        "gb_attention_prefill_bf16": [_vp, _i, _vp, _i, _vp, _vp, _vp, _i, _i, _i, _i, _vp, _i, _vp, _vp, _i, _i, _i, _i,
                                      _f, _i, _i, _i, _vp, C.c_longlong, _vp],
        "gb_attention_prefill_parts": [_i, _i, _i, _i, _i],
        # q, q_stride, out, out_stride, out32, ws_acc, ws_ml, positions, tables, table_stride, k, v, n_decode, nh, nkv, hd,
        # page, scale, window, kept first keys, run of positions, cap, sinks, chunk, max_context, stream
        "gb_attention_decode_bf16_by": [_vp, _i, _vp, _i, _i, _vp, _vp, _vp, _vp, _i, _vp, _vp, _i, _i, _i, _i, _i, _f, _i, _i,
                                        _i, _f, _vp, _i, _i, _vp],
        # q, q_stride, out, out_stride, out32, q_start, q_len, pos0, seq_base, n_seqs, max_q_len, max_context, tables,
        # table_stride, k, v, nh, nkv, hd, page, scale, window, kept first keys, run of positions, cap, sinks, first_row,
        # n_rows, part_ws, part_floats, stream
        "gb_attention_prefill_bf16_by": [_vp, _i, _vp, _i, _i, _vp, _vp, _vp, _i, _i, _i, _i, _vp, _i, _vp, _vp, _i, _i, _i, _i,
                                         _f, _i, _i, _i, _f, _vp, _i, _i, _vp, C.c_longlong, _vp],
        # the same two with the number of kept first keys after the window
        "gb_attention_decode_bf16_keep": [_vp, _i, _vp, _i, _vp, _vp, _vp, _vp, _i, _vp, _vp, _i, _i, _i, _i, _i, _f, _i, _i,
                                          _i, _i, _vp],
        "gb_attention_prefill_bf16_keep": [_vp, _i, _vp, _i, _vp, _vp, _vp, _i, _i, _i, _i, _vp, _i, _vp, _vp, _i, _i, _i, _i,
                                           _f, _i, _i, _i, _i, _vp, C.c_longlong, _vp],
        # the same two with float32 result rows
        "gb_attention_decode_bf16_out32": [_vp, _i, _vp, _i, _vp, _vp, _vp, _vp, _i, _vp, _vp, _i, _i, _i, _i, _i, _f, _i, _i,
                                           _i, _i, _vp],
        "gb_attention_prefill_bf16_out32": [_vp, _i, _vp, _i, _vp, _vp, _vp, _i, _i, _i, _i, _vp, _i, _vp, _vp, _i, _i, _i, _i,
                                            _f, _i, _i, _i, _i, _vp, C.c_longlong, _vp],
    },
    "sampling": {
        "gb_argmax": [_vp, _vp, _i, _i, _vp],
        "gb_penalize": [_vp, _i, _vp, _vp, _vp, _vp, _i, _vp],
        "gb_sample": [_vp, _i, _i, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp],
    },
}
_libs = {}


def _lib(name: str):
    lib = _libs.get(name)
    if lib is None:
        require_gpu()
        lib = build.load(name)
        for fn, args in _SIGS[name].items():
            f = getattr(lib, fn)
            f.argtypes = args
            f.restype = C.c_int
        lib.gb_last_error.restype = C.c_char_p
        _libs[name] = lib
    return lib


def _launch(lib, entry, *args) -> None:
    """Calls a kernel's entry point; every launch of a step goes through here, which is where a layer's
    launches are recorded (``start_tape``)."""
    if entry(*args) != 0:
        raise KernelError(lib.gb_last_error().decode())
    if _tape is not None:
        _tape.add(lib, entry, args)


# ------------------------------------------------------------------ recorded launches
# The layers of a model mostly differ in nothing but their tensors.  A step walks the first of a kind through the
# parts' Python while the launches it makes are recorded, and makes the same launches again for every later layer
# of that kind from native code, with the recorded layer's tensors replaced by the later layer's
# (csrc/host/launch_tape.cpp).  ``parts.model.DecoderModel.forward`` decides which layers are of a kind.
TAPE_COUNTS = {"recorded_layers": 0, "replayed_layers": 0, "replayed_launches": 0}
_tape: Optional["LaunchTape"] = None
_tape_entries: dict = {}
_host = None


def _host_lib():
    global _host
    if _host is None:
        lib = build.load("host")
        lib.gbh_tape_run.argtypes = [_vp, _i, _vp, _vp, _vp, _i]
        lib.gbh_tape_run.restype = _i
        if lib.gbh_tape_entry_bytes() != 24 + 8 * lib.gbh_tape_max_args():
            raise KernelError("the host library's recorded launches are not laid out as the bindings pack them")
        _host = lib
    return _host


def _tape_entry(lib, entry):
    """How to pack a launch of ``entry``: (struct, address of its taped form, pointer mask), or False if the
    library has no taped form of it."""
    held = _tape_entries.get(id(entry))   # ctypes functions do not hash; the entry is held so that its id stays its own
    hit = held[1] if held is not None and held[0] is entry else None
    if hit is None:
        max_args = _host_lib().gbh_tape_max_args()
        try:
            taped = getattr(lib, entry.__name__ + "_taped")
        except AttributeError:
            taped = None
        if taped is None or len(entry.argtypes) > max_args:
            hit = False
        else:
            codes, mask = "", 0
            for i, t in enumerate(entry.argtypes):
                if t is _vp:
                    codes += "Q"
                    mask |= 1 << i
                elif t is _f:
                    codes += "f4x"      # the float's bits in the low half of the slot
                else:
                    codes += "q"
            pad = 8 * (max_args - len(entry.argtypes))
            hit = (struct.Struct("<QQII" + codes + (f"{pad}x" if pad else "")), C.cast(taped, _vp).value, mask,
                   len(entry.argtypes))
        _tape_entries[id(entry)] = (entry, hit)
    return hit


class LaunchTape:
    """The launches made between ``start_tape()`` and ``stop_tape()``, packed as the native runner reads them."""

    def __init__(self):
        self.data = bytearray()
        self.libs: list = []          # the library of each launch: it holds the message if a replay refuses
        self.names: List[str] = []    # the entry point of each launch
        self.usable = True            # False once a launch was made that cannot be made again natively
        self._c = None

    def __len__(self):
        return len(self.libs)

    def add(self, lib, entry, args) -> None:
        how = _tape_entry(lib, entry)
        if how is False:
            self.usable = False
            return
        st, address, mask, n = how
        self.data += st.pack(address, mask, n, 0, *[0 if a is None else a for a in args])
        self.libs.append(lib)
        self.names.append(entry.__name__)

    def pointer(self):
        if self._c is None:
            self._c = (C.c_char * max(1, len(self.data))).from_buffer(self.data)
        return C.addressof(self._c)


class TapeOperands:
    """The tensors of a layer, in a fixed order, as the address ranges the native runner maps between layers."""

    def __init__(self, tensors: Sequence[torch.Tensor]):
        n = len(tensors)
        ptrs, sizes = [], []
        for t in tensors:
            span = 1 + sum((s - 1) * st for s, st in zip(t.shape, t.stride())) if t.numel() else 0
            ptrs.append(t.data_ptr())
            sizes.append(span * t.element_size())
        self.sizes = tuple(sizes)
        self.ptrs = (C.c_uint64 * max(1, n))(*ptrs)
        self.bytes = (C.c_uint64 * max(1, n))(*sizes)
        self.count = n
        self.keep = list(tensors)
        # pairs of ranges that overlap or coincide (a tensor that the layer holds in two places): a pointer into such a
        # place has two ranges to be moved by
        order = sorted((i for i in range(n) if sizes[i]), key=lambda i: ptrs[i])
        self.overlaps = [(a, b) for k, a in enumerate(order) for b in order[k + 1:] if ptrs[b] < ptrs[a] + sizes[a]]

    def maps_onto(self, target: "TapeOperands") -> bool:
        """Whether every pointer into these tensors has one place in ``target``'s: ranges that overlap here must be
        moved by the same distance (the runner takes the first range that holds a pointer)."""
        for a, b in self.overlaps:
            if target.ptrs[a] - self.ptrs[a] != target.ptrs[b] - self.ptrs[b]:
                return False
        return True


def start_tape() -> LaunchTape:
    global _tape
    if _tape is not None:
        raise KernelError("launches are being recorded already")
    _host_lib()
    _tape = LaunchTape()
    return _tape


def stop_tape() -> None:
    global _tape
    _tape = None


def run_tape(tape: LaunchTape, recorded: TapeOperands, target: TapeOperands) -> None:
    """Makes the recorded launches again with the tensors of ``recorded`` replaced, one for one, by those of ``target``."""
    if not tape.usable or recorded.sizes != target.sizes or not recorded.maps_onto(target):
        raise KernelError("run_tape: the layer's tensors do not match those of the recorded layer")
    rc = _host_lib().gbh_tape_run(tape.pointer(), len(tape), C.addressof(recorded.ptrs), C.addressof(recorded.bytes),
                                  C.addressof(target.ptrs), recorded.count)
    if rc != 0:
        raise KernelError(tape.libs[rc - 1].gb_last_error().decode())
    TAPE_COUNTS["replayed_layers"] += 1
    TAPE_COUNTS["replayed_launches"] += len(tape)


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)
_get_device = getattr(torch._C, "_cuda_getDevice", torch.cuda.current_device)   # CUDA is up by the time a kernel is launched


def _stream():
    # every kernel launch asks for the stream: the raw handle costs a fraction of a Stream object
    if _raw_stream is not None:
        return _raw_stream(_get_device())
    return torch.cuda.current_stream().cuda_stream


def _dev(*tensors: Optional[torch.Tensor]) -> None:
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise KernelError("operands must be on the GPU")


def _p(t: Optional[torch.Tensor]):
    return None if t is None else t.data_ptr()


def _rows(t: torch.Tensor, what: str) -> int:
    """Row stride of a 2-d tensor whose rows are dense."""
    if t.dim() != 2 or t.stride(1) != 1:
        raise KernelError(f"{what} must be 2-d with dense rows, got shape {tuple(t.shape)} strides {t.stride()}")
    return t.stride(0)


def _i32(t: Optional[torch.Tensor], what: str, n: Optional[int] = None) -> None:
    if t is None:
        return
    if t.dtype != torch.int32 or not t.is_contiguous():
        raise KernelError(f"{what} must be a contiguous int32 tensor")
    if n is not None and t.numel() < n:
        raise KernelError(f"{what} holds {t.numel()} entries, {n} are needed")


def key_piece(head_dim: int) -> int:
    """Elements of one piece of a key in its page: 8 for head sizes that are a multiple of 8."""
    return 8 if head_dim % 8 == 0 else 4 if head_dim % 4 == 0 else 2 if head_dim % 2 == 0 else 1


def key_pages_shape(pages: int, n_kv_heads: int, page_size: int, head_dim: int) -> tuple:
    """Key pages hold a head's dimensions in pieces, and of each piece the page's slots side by side:
    [pages, kv heads, head size / piece, page size, piece].  The lanes that take neighbouring keys for a
    matrix-core operand then read neighbouring addresses."""
    piece = key_piece(head_dim)
    return (pages, n_kv_heads, head_dim // piece, page_size, piece)


def pack_keys(keys: torch.Tensor) -> torch.Tensor:
    """[pages, kv heads, page size, head size] to the layout of key pages."""
    p, h, s, d = keys.shape
    piece = key_piece(d)
    return keys.reshape(p, h, s, d // piece, piece).permute(0, 1, 3, 2, 4).contiguous()


def unpack_keys(k_pages: torch.Tensor) -> torch.Tensor:
    """Key pages to [pages, kv heads, page size, head size]."""
    p, h, n, s, piece = k_pages.shape
    return k_pages.permute(0, 1, 3, 2, 4).reshape(p, h, s, n * piece)


def _check_pages(k_pages, v_pages, dtype, what: str):
    """Key pages as ``key_pages_shape`` says; value pages transposed, [pages, kv heads, head size, page size];
    both contiguous and of the activations' type.  Returns (pages, kv heads, page size, head size)."""
    if k_pages is None or v_pages is None or k_pages.dim() != 5 or v_pages.dim() != 4:
        raise KernelError(f"{what}: key pages must be 5-d [pages, kv heads, head size / piece, page size, piece] "
                          f"and value pages 4-d")
    p, h, n, s, piece = k_pages.shape
    d = n * piece
    if piece != key_piece(d):
        raise KernelError(f"{what}: key pages of head size {d} are kept in pieces of {key_piece(d)}, not {piece}")
    if tuple(v_pages.shape) != (p, h, d, s):
        raise KernelError(f"{what}: value pages must be [pages, kv heads, head size, page size] = "
                          f"{(p, h, d, s)}, got {tuple(v_pages.shape)}")
    if not k_pages.is_contiguous() or not v_pages.is_contiguous() or k_pages.dtype != dtype or v_pages.dtype != dtype:
        raise KernelError(f"{what}: pages must be contiguous and of the activations' type")
    return p, h, s, d


# ------------------------------------------------------------------ elementwise
def embed(table: torch.Tensor, ids: torch.Tensor, out: torch.Tensor, scale: float = 1.0) -> None:
    """out[i, :] = table[ids[i], :] * scale as 32-bit floats; an out of [copies, n, d] receives that many copies."""
    _dev(table, ids, out)
    copies = out.shape[0] if out.dim() == 3 else 1
    n, d = out.shape[-2:]
    _i32(ids, "ids", n)
    if out.dtype != torch.float32 or not out.is_contiguous() or not table.is_contiguous() or table.shape[1] != d:
        raise KernelError("embed: out must be contiguous float32 [n, d] or [copies, n, d] and table [vocab, d]")
    lib = _lib("elementwise")
    _launch(lib, lib.gb_embed, _p(table), dtype_code(table), _p(ids), _p(out), n, d, table.shape[0], float(scale),
            int(copies), _stream())


def rmsnorm(x: torch.Tensor, gamma: torch.Tensor, eps: float, out: torch.Tensor,
            rows: Optional[torch.Tensor] = None) -> None:
    """out[r] = gamma * (x[rows[r] or r] / sqrt(mean(x^2) + eps)); x is float32."""
    _dev(x, gamma, out, rows)
    m, d = out.shape
    if x.dtype != torch.float32 or not x.is_contiguous() or x.shape[1] != d or not out.is_contiguous():
        raise KernelError("rmsnorm: x must be contiguous float32 [n, d] and out contiguous [m, d]")
    if gamma.numel() != d or not gamma.is_contiguous():
        raise KernelError(f"rmsnorm: gamma has {gamma.numel()} entries, the rows have {d}")
    if rows is None and x.shape[0] < m:
        raise KernelError("rmsnorm: fewer input rows than output rows")
    _i32(rows, "rows", m)
    lib = _lib("elementwise")
    _launch(lib, lib.gb_rmsnorm, _p(x), _p(gamma), dtype_code(gamma), _p(rows), _p(out), dtype_code(out), m, d,
                               float(eps), _stream())


def rope_table(positions: torch.Tensor, inv_freq: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> None:
    _dev(positions, inv_freq, cos, sin)
    n, half = cos.shape
    _i32(positions, "positions", n)
    for t in (inv_freq, cos, sin):
        if t.dtype != torch.float32 or not t.is_contiguous():
            raise KernelError("rope_table: tables must be contiguous float32")
    if inv_freq.numel() != half or sin.shape != cos.shape:
        raise KernelError("rope_table: table shapes do not match")
    lib = _lib("elementwise")
    _launch(lib, lib.gb_rope_table, _p(positions), _p(inv_freq), _p(cos), _p(sin), n, half, _stream())


def rope_store(qkv: torch.Tensor, cos: Optional[torch.Tensor], sin: Optional[torch.Tensor],
               slots: Optional[torch.Tensor], k_pages: Optional[torch.Tensor], v_pages: Optional[torch.Tensor],
               n_heads: int, n_kv_heads: int, head_dim: int, rotate: bool = True, portions=None) -> None:
    """Rotate the query and key heads of each stacked row in place and write keys and values
    to the pages at ``slots``.  ``slots`` None: nothing is stored.

    ``portions = (first_row, q_start, q_len, pos0, seq_base, n_seqs, max_q_len)`` says that the rows from
    first_row on are prompt portions of requests seq_base .. seq_base + n_seqs - 1 (device arrays indexed
    by request): their values are then written to the transposed pages sixteen positions at a time."""
    _dev(qkv, cos, sin, slots, k_pages, v_pages)
    n = qkv.shape[0]
    stride = _rows(qkv, "qkv")
    page_size = 0
    if slots is not None:
        _i32(slots, "slots", n)
        _, p_heads, page_size, p_hd = _check_pages(k_pages, v_pages, qkv.dtype, "rope_store")
        if (p_heads, p_hd) != (n_kv_heads, head_dim):
            raise KernelError("rope_store: pages do not have this layer's kv heads and head size")
    if rotate:
        if cos is None or sin is None or cos.shape != (n, head_dim // 2) and cos.shape[0] < n:
            raise KernelError("rope_store: rotation needs cos/sin tables of [n, head_dim/2]")
        if cos.shape[1] != head_dim // 2 or cos.dtype != torch.float32 or not cos.is_contiguous() \
                or not sin.is_contiguous():
            raise KernelError("rope_store: cos/sin must be contiguous float32 [n, head_dim/2]")
    v_rows, q_start, q_len, pos0, seq_base, n_seqs, max_q_len = n, None, None, None, 0, 0, 0
    if portions is not None and slots is not None:
        v_rows, q_start, q_len, pos0, seq_base, n_seqs, max_q_len = portions
        _dev(q_start, q_len, pos0)
        for name, t in (("q_start", q_start), ("q_len", q_len), ("pos0", pos0)):
            if t.dtype != torch.int32 or not t.is_contiguous() or t.numel() < seq_base + n_seqs:
                raise KernelError(f"rope_store: {name} must be contiguous int32, one entry per request")
        if not 0 <= v_rows <= n:
            raise KernelError("rope_store: the first portion row lies outside the batch")
    lib = _lib("elementwise")
    _launch(lib, lib.gb_rope_store, _p(qkv), dtype_code(qkv), stride, _p(cos), _p(sin), _p(slots), _p(k_pages),
                                  _p(v_pages), n, n_heads, n_kv_heads, head_dim, page_size, 1 if rotate else 0,
                                  int(v_rows), _p(q_start), _p(q_len), _p(pos0), int(seq_base), int(n_seqs),
                                  int(max_q_len), _stream())


def silu_mul(gate_up: torch.Tensor, out: torch.Tensor) -> None:
    _dev(gate_up, out)
    n, inter = out.shape
    if gate_up.shape != (n, 2 * inter) or not gate_up.is_contiguous() or not out.is_contiguous() \
            or gate_up.dtype != out.dtype:
        raise KernelError("silu_mul: gate_up must be contiguous [n, 2I] and out [n, I] of one type")
    lib = _lib("elementwise")
    _launch(lib, lib.gb_silu_mul, _p(gate_up), _p(out), dtype_code(out), n, inter, _stream())


def copy_rows(base: torch.Tensor, src: torch.Tensor, dst: torch.Tensor) -> None:
    """base[dst[i]] = base[src[i]] along the first dimension."""
    _dev(base, src, dst)
    if not base.is_contiguous():
        raise KernelError("copy_rows: base must be contiguous")
    count = src.numel()
    _i32(src, "src", count)
    _i32(dst, "dst", count)
    row_bytes = base[0].numel() * base.element_size()
    lib = _lib("elementwise")
    _launch(lib, lib.gb_copy_rows, _p(base), row_bytes, _p(src), _p(dst), count, _stream())


def qk_norm_store(qk: torch.Tensor, bias_q: Optional[torch.Tensor], bias_k: Optional[torch.Tensor],
                  w_q: Optional[torch.Tensor], w_k: Optional[torch.Tensor], eps: float, slots: Optional[torch.Tensor],
                  k_pages: Optional[torch.Tensor], v_pages: Optional[torch.Tensor], n_heads: int, n_kv_heads: int,
                  head_dim: int, values_in_rows: bool = False) -> None:
    """Rows of query heads then key heads: adds the biases, writes each key head as it then is to the value pages
    (the values of such a layer are its keys as projected), RMS-norms every head over its dimensions with the weight
    that the heads of its kind share (None: the head stays as it is), and leaves queries in place and keys in the key
    pages at ``slots`` (None: nothing is stored).  Biases and weights are float32.  ``values_in_rows`` (without
    ``slots``): the rows have room for the value heads behind the key heads; the normed keys stay in place, the values
    are written behind them, and ``rope_store`` without rotation takes both to the pages."""
    _dev(qk, bias_q, bias_k, w_q, w_k, slots, k_pages, v_pages)
    n = qk.shape[0]
    stride = _rows(qk, "qk")
    for t, size, what in ((bias_q, n_heads * head_dim, "bias_q"), (bias_k, n_kv_heads * head_dim, "bias_k"),
                          (w_q, head_dim, "w_q"), (w_k, head_dim, "w_k")):
        if t is not None and (t.dtype != torch.float32 or not t.is_contiguous() or t.numel() != size):
            raise KernelError(f"qk_norm_store: {what} must be contiguous float32 of {size} entries")
    if qk.shape[1] < (n_heads + (2 if values_in_rows else 1) * n_kv_heads) * head_dim or (values_in_rows and slots is not None):
        raise KernelError("qk_norm_store: rows shorter than the heads, or values in the rows together with cache rows")
    page_size = 0
    if slots is not None:
        _i32(slots, "slots", n)
        _, p_heads, page_size, p_hd = _check_pages(k_pages, v_pages, qk.dtype, "qk_norm_store")
        if (p_heads, p_hd) != (n_kv_heads, head_dim):
            raise KernelError("qk_norm_store: pages do not have this layer's kv heads and head size")
    lib = _lib("elementwise")
    _launch(lib, lib.gb_qk_norm_store, _p(qk), dtype_code(qk), stride, _p(bias_q), _p(bias_k), _p(w_q), _p(w_k), float(eps),
            _p(slots), _p(k_pages), _p(v_pages), n, n_heads, n_kv_heads, head_dim, page_size,
            (n_heads + n_kv_heads) * head_dim if values_in_rows else -1, _stream())


def add_bias(x: torch.Tensor, bias: torch.Tensor) -> None:
    """x[r, :] += bias, both float32."""
    _dev(x, bias)
    n, d = x.shape
    if x.dtype != torch.float32 or not x.is_contiguous() or bias.dtype != torch.float32 or bias.numel() != d \
            or not bias.is_contiguous():
        raise KernelError("add_bias: x must be contiguous float32 [n, d] and bias float32 [d]")
    lib = _lib("elementwise")
    _launch(lib, lib.gb_add_bias, _p(x), _p(bias), n, d, _stream())


def scale_rows(x: torch.Tensor, s: float) -> None:
    """x *= s, float32."""
    _dev(x)
    if x.dtype != torch.float32 or not x.is_contiguous():
        raise KernelError("scale_rows: x must be contiguous float32")
    lib = _lib("elementwise")
    _launch(lib, lib.gb_scale_rows, _p(x), float(s), x.numel(), _stream())


# ------------------------------------------------------------------- residual streams
MAX_STREAMS = 8   # streams.hip keeps a row's streams in registers


def _streams(X: torch.Tensor, what: str):
    if X.dim() != 3 or X.dtype != torch.float32 or not X.is_contiguous() or not 1 <= X.shape[0] <= MAX_STREAMS:
        raise KernelError(f"{what}: the streams must be contiguous float32 [streams <= {MAX_STREAMS}, n, d]")
    return X.shape


def streams_norm(X: torch.Tensor, w_in: Optional[torch.Tensor], gamma: torch.Tensor, eps: float, out: torch.Tensor,
                 rows: Optional[torch.Tensor] = None, total: Optional[torch.Tensor] = None, update: Optional[tuple] = None) -> None:
    """out[r] = gamma * u / sqrt(mean(u^2) + eps), u = sum_s w_in[s] X[s][rows[r] or r] (``w_in`` None: the plain sum of
    the streams); ``total`` (float32 [m, d]) receives u as well.  ``update=(mix, w_out, y)``: the streams are first
    updated as ``streams_mix`` does, in the same pass, and u is taken from the new ones (every row, no ``rows``)."""
    _dev(X, w_in, gamma, out, rows, total)
    mix = w_out = y = None
    if update is not None:
        mix, w_out, y = update
        _dev(mix, w_out, y)
        S0, n0, d0 = X.shape
        if rows is not None or out.shape[0] != n0 or y.dtype != torch.float32 or y.shape != (n0, d0) or not y.is_contiguous() \
                or mix.dtype != torch.float32 or mix.shape != (S0, S0) or not mix.is_contiguous() \
                or w_out.dtype != torch.float32 or w_out.numel() != S0 or not w_out.is_contiguous():
            raise KernelError("streams_norm: update=(mix [S, S], w_out [S], y [n, d]) in float32, on every row")
    S, n, d = _streams(X, "streams_norm")
    m = out.shape[0]
    if out.shape != (m, d) or not out.is_contiguous() or gamma.numel() != d or not gamma.is_contiguous():
        raise KernelError("streams_norm: out must be contiguous [m, d] and gamma hold d entries")
    if w_in is not None and (w_in.dtype != torch.float32 or w_in.numel() != S or not w_in.is_contiguous()):
        raise KernelError("streams_norm: w_in must be float32, one weight a stream")
    if rows is None and n < m:
        raise KernelError("streams_norm: fewer input rows than output rows")
    if total is not None and (total.dtype != torch.float32 or total.shape != (m, d) or not total.is_contiguous()):
        raise KernelError("streams_norm: total must be contiguous float32 [m, d]")
    _i32(rows, "rows", m)
    lib = _lib("streams")
    _launch(lib, lib.gb_streams_norm, _p(X), X.stride(0), S, _p(w_in), _p(gamma), dtype_code(gamma), _p(rows), _p(out),
            dtype_code(out), _p(total), m, d, float(eps), _p(mix), _p(w_out), _p(y), _stream())


def streams_mix(X: torch.Tensor, mix: torch.Tensor, w_out: torch.Tensor, y: torch.Tensor) -> None:
    """In place, all streams at once from the old ones: X[t] = sum_s mix[s, t] X[s] + w_out[t] y."""
    _dev(X, mix, w_out, y)
    S, n, d = _streams(X, "streams_mix")
    if y.dtype != torch.float32 or y.shape != (n, d) or not y.is_contiguous():
        raise KernelError("streams_mix: y must be contiguous float32 [n, d]")
    if mix.dtype != torch.float32 or mix.shape != (S, S) or not mix.is_contiguous() or w_out.dtype != torch.float32 \
            or w_out.numel() != S or not w_out.is_contiguous():
        raise KernelError("streams_mix: mix must be float32 [streams, streams] and w_out float32 [streams]")
    lib = _lib("streams")
    _launch(lib, lib.gb_streams_mix, _p(X), X.stride(0), S, _p(mix), _p(w_out), _p(y), n * d, _stream())


# ------------------------------------------------------------------- linear attention
LINEAR_MAX_KEY_DIM = 256   # linear_attention.hip: a lane holds at most 32 rows of its column of the state


def _f32_rows(t: torch.Tensor, shape, what: str) -> None:
    if t.dtype != torch.float32 or tuple(t.shape) != tuple(shape) or not t.is_contiguous():
        raise KernelError(f"{what} must be contiguous float32 {tuple(shape)}")


def retention_prep(proj: torch.Tensor, q_off: int, k_off: int, cos: Optional[torch.Tensor], sin: Optional[torch.Tensor],
                   q32: torch.Tensor, k32: torch.Tensor, n_heads: int, key_dim: int, rot: int, k_scale: float) -> None:
    """q32, k32 (float32 [n, heads * key_dim]) from the query and key heads at columns ``q_off`` and ``k_off`` of the
    projection's rows: the first ``rot`` dimensions of each head turned in rotate-half pairs by the rows' angles
    (``cos``, ``sin`` float32 [n, rot / 2]), the keys then times ``k_scale``."""
    _dev(proj, cos, sin, q32, k32)
    n = proj.shape[0]
    stride = _rows(proj, "proj")
    _f32_rows(q32, (n, n_heads * key_dim), "q32")
    _f32_rows(k32, (n, n_heads * key_dim), "k32")
    if rot:
        for t in (cos, sin):
            if t is None or t.dtype != torch.float32 or not t.is_contiguous() or t.shape[1] != rot // 2 or t.shape[0] < n:
                raise KernelError("retention_prep: cos/sin must be contiguous float32 [n, rot / 2]")
    if max(q_off, k_off) + n_heads * key_dim > proj.shape[1]:
        raise KernelError("retention_prep: the heads lie beyond the projection's rows")
    lib = _lib("linear_attention")
    _launch(lib, lib.gb_retention_prep, _p(proj), dtype_code(proj), stride, int(q_off), int(k_off), _p(cos) if rot else None,
            _p(sin) if rot else None, _p(q32), _p(k32), n, n_heads, key_dim, int(rot), float(k_scale), _stream())


def gla_prep(proj: torch.Tensor, q_off: int, k_off: int, low_off: int, a2: torch.Tensor, a2_bias: Optional[torch.Tensor],
             q32: torch.Tensor, k32: torch.Tensor, decay: torch.Tensor, q_scale: float, tau: float,
             z: Optional[torch.Tensor] = None) -> None:
    """q32 = q * q_scale, k32 = k, decay = sigmoid(z)^(1/tau) with z = a2 . low + a2_bias, all float32 [n, width], from
    the projection's rows (queries, keys and the low-rank rows at the given columns; ``a2`` [width, rank] in the
    projection's type).  ``z`` (float32 [n, width]): the products a2 . low, where a matrix product has made them."""
    _dev(proj, a2, a2_bias, q32, k32, decay, z)
    if z is not None:
        _f32_rows(z, (proj.shape[0], a2.shape[0]), "z")
    n = proj.shape[0]
    stride = _rows(proj, "proj")
    width, rank = a2.shape
    for t, what in ((q32, "q32"), (k32, "k32"), (decay, "decay")):
        _f32_rows(t, (n, width), what)
    if a2.dtype != proj.dtype or not a2.is_contiguous():
        raise KernelError("gla_prep: a2 must be contiguous and of the projection's type")
    if a2_bias is not None:
        _f32_rows(a2_bias, (width,), "a2_bias")
    if max(q_off, k_off) + width > proj.shape[1] or low_off + rank > proj.shape[1]:
        raise KernelError("gla_prep: the heads lie beyond the projection's rows")
    lib = _lib("linear_attention")
    _launch(lib, lib.gb_gla_prep, _p(proj), dtype_code(proj), stride, int(q_off), int(k_off), int(low_off), _p(a2), _p(z),
            _p(a2_bias), _p(q32), _p(k32), _p(decay), n, width, rank, float(q_scale), 1.0 / float(tau), _stream())


LINEAR_SEGMENT = 128          # rows of a segment of a long portion
LINEAR_SEGMENT_FROM = 256     # portions up to here run token after token from the request's state: no bit depends on the cut


def linear_scan_segments(max_q_len: int) -> int:
    """Into how many segments ``linear_scan`` cuts the portions of a step whose longest one has ``max_q_len`` rows."""
    return 1 if max_q_len <= LINEAR_SEGMENT_FROM else -(-max_q_len // LINEAR_SEGMENT)


def linear_scan(q32: torch.Tensor, k32: torch.Tensor, v: torch.Tensor, out: torch.Tensor, state: torch.Tensor, ctx,
                n_heads: int, key_dim: int, value_dim: int, decay: Optional[torch.Tensor] = None,
                head_decay: Optional[torch.Tensor] = None, segments: int = 1,
                workspace: Optional[torch.Tensor] = None, token_decay: Optional[torch.Tensor] = None) -> None:
    """The recurrence S <- diag(a) S + k v^T, o = S^T q over each request's rows of the step, in their order, from the
    state in the request's slot (empty for a request at position 0) and back into it.  ``decay`` float32
    [n, heads * key_dim] (a decay a key channel and token) or ``head_decay`` float32 [heads]; ``v`` rows of
    heads * value_dim in the activations' type (may be a view into wider rows); ``out`` float32 [n, heads * value_dim];
    ``state`` float32 [slots, heads, value_dim, key_dim].  ``segments`` > 1 (``linear_scan_segments`` of the step's
    longest portion, with a float32 ``workspace`` of requests * segments * heads * (value_dim + 1) * key_dim elements): long
    portions run as segments of ``LINEAR_SEGMENT`` rows side by side and a second kernel joins them; what a token gets then
    differs from the token-by-token sums by rounding.  ``token_decay`` float32 [n, heads], in place of the other two: a
    decay a token and head, the same for all key channels.  ``state`` may hold more than value_dim columns a head
    ([slots, heads, columns, key_dim]): the recurrence keeps the first value_dim, the rest are the caller's."""
    _dev(q32, k32, v, out, state, decay, head_decay, token_decay)
    a_head = token_decay is not None
    if a_head:
        if decay is not None or head_decay is not None:
            raise KernelError("linear_scan: a decay a head, a key channel, or a token and head: one of the three")
        _f32_rows(token_decay, (q32.shape[0], n_heads), "token_decay")
        decay = token_decay
    n = q32.shape[0]
    _f32_rows(q32, (n, n_heads * key_dim), "q32")
    _f32_rows(k32, (n, n_heads * key_dim), "k32")
    _f32_rows(out, (n, n_heads * value_dim), "out")
    if (decay is None) == (head_decay is None):
        raise KernelError("linear_scan: a decay a head or a decay a key channel, one of the two")
    if a_head:
        pass
    elif decay is not None:
        _f32_rows(decay, (n, n_heads * key_dim), "decay")
    else:
        _f32_rows(head_decay, (n_heads,), "head_decay")
    if v.shape != (n, n_heads * value_dim):
        raise KernelError("linear_scan: v must be [n, heads * value_dim]")
    if (state.dtype != torch.float32 or not state.is_contiguous() or state.dim() != 4 or state.shape[1] != n_heads
            or state.shape[2] < value_dim or state.shape[3] != key_dim):
        raise KernelError("linear_scan: state must be contiguous float32 [slots, heads, value_dim or more, key_dim]")
    if key_dim > LINEAR_MAX_KEY_DIM:
        raise KernelError(f"linear_scan: a key size of {key_dim} is above {LINEAR_MAX_KEY_DIM}")
    if segments > 1:
        _dev(workspace)
        need = ctx.num_seqs * segments * n_heads * (value_dim + 1) * key_dim
        if workspace is None or workspace.dtype != torch.float32 or not workspace.is_contiguous() or workspace.numel() < need:
            raise KernelError(f"linear_scan: {segments} segments need a contiguous float32 workspace of {need} elements")
    lib = _lib("linear_attention")
    _launch(lib, lib.gb_linear_scan, _p(q32), _p(k32), _p(decay), _p(head_decay), _p(v), dtype_code(v), _rows(v, "v"), _p(out),
            _p(state), _p(ctx.q_start), _p(ctx.q_len), _p(ctx.pos0), _p(ctx.state_slots), ctx.num_seqs, n_heads, key_dim,
            value_dim, int(state.shape[2]), 1 if a_head else 0, int(segments), LINEAR_SEGMENT, _p(workspace) if segments > 1 else None,
            workspace.numel() if segments > 1 else 0, _stream())


def head_norm_gate(o: torch.Tensor, gate: torch.Tensor, weight: Optional[torch.Tensor], out: torch.Tensor, n_heads: int,
                   value_dim: int, eps: float) -> None:
    """out[t, h] = weight * o[t, h] / sqrt(mean(o[t, h]^2) + eps) * silu(gate[t, h]) (``weight`` float32 [value_dim] shared
    by the heads, or None); o float32, gate and out in the activations' type."""
    _dev(o, gate, weight, out)
    n = o.shape[0]
    _f32_rows(o, (n, n_heads * value_dim), "o")
    if gate.shape != (n, n_heads * value_dim) or out.shape != (n, n_heads * value_dim) or gate.dtype != out.dtype \
            or not out.is_contiguous():
        raise KernelError("head_norm_gate: gate and out must be [n, heads * value_dim] of one type, out contiguous")
    if weight is not None:
        _f32_rows(weight, (value_dim,), "weight")
    lib = _lib("linear_attention")
    _launch(lib, lib.gb_head_norm_gate, _p(o), _p(gate), dtype_code(out), _rows(gate, "gate"), _p(weight), _p(out), n, n_heads,
            value_dim, float(eps), _stream())


# ------------------------------------------------------------------- matrix memory with exponential gates
def mlstm_gates(z: torch.Tensor, bias_i: Optional[torch.Tensor], bias_f: Optional[torch.Tensor], cap: float,
                coef: torch.Tensor, state: torch.Tensor, m_row: int, ctx, n_heads: int) -> None:
    """coef[t, h] = (a, b, exp(-m)) float32 [n, heads, 3] from the gates' projections ``z`` float32 [n, 2 * heads] (input
    gates, then forget gates) and their biases (float32 [heads]): i = cap tanh(z_i / cap), f = log sigmoid(cap tanh(z_f /
    cap)), m_t = max(f_t + m_(t-1), i_t), a = exp(f + m_(t-1) - m), b = exp(i - m), over each request's rows in their
    order.  m before a request's first token is 0; between steps it lives in element 0 of row ``m_row`` of the head's
    block of ``state`` ([slots, heads, rows, key size] float32)."""
    _dev(z, bias_i, bias_f, coef, state)
    n = z.shape[0]
    if z.dtype != torch.float32 or z.dim() != 2 or z.stride(1) != 1 or z.shape[1] < 2 * n_heads:
        raise KernelError("mlstm_gates: z must be float32 [n, 2 * heads] with dense rows")
    _f32_rows(coef, (n, n_heads, 3), "coef")
    for b in (bias_i, bias_f):
        if b is not None:
            _f32_rows(b, (n_heads,), "gate bias")
    if (state.dtype != torch.float32 or not state.is_contiguous() or state.dim() != 4 or state.shape[1] != n_heads
            or not 0 <= m_row < state.shape[2]):
        raise KernelError("mlstm_gates: state must be contiguous float32 [slots, heads, rows, key size] and hold the row of m")
    lib = _lib("linear_attention")
    _launch(lib, lib.gb_mlstm_gates, _p(z), z.stride(0), _p(bias_i), _p(bias_f), float(cap), _p(coef), _p(state),
            int(state.shape[2] * state.shape[3]), int(m_row * state.shape[3]), _p(ctx.q_start), _p(ctx.q_len), _p(ctx.pos0),
            _p(ctx.state_slots), ctx.num_seqs, n_heads, n, 1 if int(ctx.host["max_q_len"]) == 1 and n == ctx.num_seqs else 0,
            _stream())


def mlstm_prep(proj: torch.Tensor, q_off: int, k_off: int, v_off: int, coef: torch.Tensor, q32: torch.Tensor,
               k32: torch.Tensor, decay: torch.Tensor, vext: torch.Tensor, n_heads: int, key_dim: int, value_dim: int,
               q_scale: float) -> None:
    """The recurrence's operands from the projection's rows and ``mlstm_gates``' coefficients: q32 = q * q_scale,
    k32 = k * b (float32 [n, heads * key_dim]), decay = a (float32 [n, heads]), vext = (v, 1) a head
    ([n, heads * (value_dim + 1)] in the projection's type: the normaliser is one more value channel)."""
    _dev(proj, coef, q32, k32, decay, vext)
    n = proj.shape[0]
    stride = _rows(proj, "proj")
    _f32_rows(coef, (n, n_heads, 3), "coef")
    _f32_rows(q32, (n, n_heads * key_dim), "q32")
    _f32_rows(k32, (n, n_heads * key_dim), "k32")
    _f32_rows(decay, (n, n_heads), "decay")
    if vext.shape != (n, n_heads * (value_dim + 1)) or vext.dtype != proj.dtype or not vext.is_contiguous():
        raise KernelError("mlstm_prep: vext must be contiguous [n, heads * (value_dim + 1)] of the projection's type")
    if max(q_off, k_off) + n_heads * key_dim > proj.shape[1] or v_off + n_heads * value_dim > proj.shape[1]:
        raise KernelError("mlstm_prep: the heads lie beyond the projection's rows")
    lib = _lib("linear_attention")
    _launch(lib, lib.gb_mlstm_prep, _p(proj), dtype_code(proj), stride, int(q_off), int(k_off), int(v_off), _p(coef), _p(q32),
            _p(k32), _p(decay), _p(vext), n, n_heads, key_dim, value_dim, float(q_scale), _stream())


def mlstm_out(o: torch.Tensor, coef: torch.Tensor, gate: torch.Tensor, weight: Optional[torch.Tensor], out: torch.Tensor,
              n_heads: int, value_dim: int, eps: float) -> None:
    """out[t, h] = weight[h] * y / sqrt(mean(y^2) + eps) * sigmoid(gate[t, h]) with y = o[t, h, :value_dim] /
    (max(|o[t, h, value_dim]|, exp(-m)) + 1e-6): ``o`` float32 [n, heads * (value_dim + 1)] as the recurrence leaves it
    (the last sum of a head is the normaliser's), ``weight`` float32 [heads * value_dim] or None, gate and out in the
    activations' type."""
    _dev(o, coef, gate, weight, out)
    n = o.shape[0]
    _f32_rows(o, (n, n_heads * (value_dim + 1)), "o")
    _f32_rows(coef, (n, n_heads, 3), "coef")
    if gate.shape != (n, n_heads * value_dim) or out.shape != (n, n_heads * value_dim) or gate.dtype != out.dtype \
            or not out.is_contiguous():
        raise KernelError("mlstm_out: gate and out must be [n, heads * value_dim] of one type, out contiguous")
    if weight is not None:
        _f32_rows(weight, (n_heads * value_dim,), "weight")
    lib = _lib("linear_attention")
    _launch(lib, lib.gb_mlstm_out, _p(o), _p(coef), _p(gate), dtype_code(out), _rows(gate, "gate"), _p(weight), _p(out), n,
            n_heads, value_dim, float(eps), _stream())


# ------------------------------------------------------------------- short convolution before attention
CONV_MAX_TAPS = 8   # shortconv.hip keeps a channel's slot in registers


def conv_heads(proj: torch.Tensor, wconv: Optional[torch.Tensor], state: Optional[torch.Tensor], ctx,
               cos: Optional[torch.Tensor], sin: Optional[torch.Tensor], rot: int, eps: float, norm: bool, out: torch.Tensor,
               head_cols: int, slots: Optional[torch.Tensor], k_pages: Optional[torch.Tensor], v_pages: Optional[torch.Tensor],
               n_heads: int, n_kv_heads: int, dim: int, vdim: int) -> None:
    """The heads of a step's stacked projections made ready for attention.  ``proj`` [n, heads * dim + kv heads * (dim +
    vdim)]: query heads, key heads, value heads.  ``wconv`` float32 [channels, taps] (None: no convolution): every
    channel is convolved over its request's tokens, y_t = sum_j w[:, j] u_(t - taps + 1 + j), zeros before the first
    token; the last taps - 1 projections of each request live in ``state`` (float32 [slots, taps - 1, channels]) and are
    moved on by this call.  Then the first ``rot`` channels of every query and key head are turned in neighbouring pairs
    by the rows' angles (``cos``, ``sin`` float32 [n, rot / 2]) and, with ``norm``, every query and key head is divided
    by its root mean square.  ``out`` [n, (heads + 2 kv heads) * head_cols] receives the heads, each filled up with
    zeros to ``head_cols`` columns; with ``slots`` keys and values also go to the pages (heads of ``head_cols``)."""
    _dev(proj, wconv, state, cos, sin, out, slots, k_pages, v_pages)
    n = proj.shape[0]
    channels = (n_heads + n_kv_heads) * dim + n_kv_heads * vdim
    taps = 1
    if wconv is not None:
        taps = wconv.shape[1]
        _f32_rows(wconv, (channels, taps), "wconv")
        if taps > CONV_MAX_TAPS:
            raise KernelError(f"conv_heads: {taps} taps are above {CONV_MAX_TAPS}")
        if taps > 1 and (state is None or state.dtype != torch.float32 or not state.is_contiguous()
                         or tuple(state.shape[1:]) != (taps - 1, channels)):
            raise KernelError("conv_heads: state must be contiguous float32 [slots, taps - 1, channels]")
    if proj.shape[1] < channels or out.shape != (n, (n_heads + 2 * n_kv_heads) * head_cols) or out.dtype != proj.dtype \
            or not out.is_contiguous():
        raise KernelError("conv_heads: out must be contiguous [n, (heads + 2 kv heads) * head_cols] of the projection's type")
    if rot:
        for t in (cos, sin):
            if t is None or t.dtype != torch.float32 or not t.is_contiguous() or t.shape[1] != rot // 2 or t.shape[0] < n:
                raise KernelError("conv_heads: cos/sin must be contiguous float32 [n, rot / 2]")
    page_size = 0
    if slots is not None:
        _i32(slots, "slots", n)
        _, p_heads, page_size, p_hd = _check_pages(k_pages, v_pages, proj.dtype, "conv_heads")
        if (p_heads, p_hd) != (n_kv_heads, head_cols):
            raise KernelError("conv_heads: pages do not have this layer's kv heads and head size")
    single = int(ctx.host["max_q_len"]) == 1
    lib = _lib("shortconv")
    _launch(lib, lib.gb_conv_heads, _p(proj), dtype_code(proj), _rows(proj, "proj"), _p(wconv), taps, _p(state),
            _p(ctx.tok_seq), _p(ctx.q_start), _p(ctx.pos0), _p(ctx.state_slots), _p(cos) if rot else None,
            _p(sin) if rot else None, int(rot), float(eps), 1 if norm else 0, _p(out), out.stride(0), int(head_cols),
            _p(slots), _p(k_pages) if slots is not None else None, _p(v_pages) if slots is not None else None, page_size, n,
            n_heads, n_kv_heads, dim, vdim, 1 if single else 0, _stream())
    if wconv is not None and taps > 1 and not single:
        _launch(lib, lib.gb_conv_state, _p(proj), dtype_code(proj), _rows(proj, "proj"), _p(state), _p(ctx.q_start),
                _p(ctx.q_len), _p(ctx.state_slots), ctx.num_seqs, channels, taps, _stream())


# --------------------------------------------------------- sublayers with normed outputs; latent and differential heads
TIME_CONV_MAX_TAPS = 8   # headmix.hip keeps a channel's slot in registers


def _act_rows(t: torch.Tensor, dtype, cols: int, what: str) -> int:
    """Row stride of a 2-d tensor of the activations' type with dense rows of at least ``cols`` columns."""
    if t.dtype != dtype or t.dim() != 2 or t.stride(1) != 1 or t.shape[1] < cols:
        raise KernelError(f"{what} must be 2-d {dtype} with dense rows of at least {cols} columns, got {tuple(t.shape)} {t.dtype}")
    return t.stride(0)


def time_conv(x: torch.Tensor, w: Optional[torch.Tensor], state: Optional[torch.Tensor], ctx, out: torch.Tensor) -> None:
    """out = x + conv(x) in the type of ``out``: x float32 [n, d] (the residual), ``w`` float32 [taps, d], a row a tap (None: out is x
    rounded), conv(x)[t] = sum_j w[j] x[t - taps + 1 + j] over the request's own tokens, zeros before its first.  The
    request's last taps - 1 rows of x live in ``state`` (float32 [slots, taps - 1, d]) and are moved on by this call, so
    it must come before x changes."""
    _dev(x, w, state, out)
    n, d = x.shape
    _f32_rows(x, (n, d), "x")
    taps = 0
    if w is not None:
        taps = w.shape[0]
        _f32_rows(w, (taps, d), "w")
        if taps > TIME_CONV_MAX_TAPS:
            raise KernelError(f"time_conv: {taps} taps are above {TIME_CONV_MAX_TAPS}")
        if taps > 1 and (state is None or state.dtype != torch.float32 or not state.is_contiguous()
                         or tuple(state.shape[1:]) != (taps - 1, d)):
            raise KernelError("time_conv: state must be contiguous float32 [slots, taps - 1, d]")
    ldo = _act_rows(out, out.dtype, d, "out")
    if out.shape[0] != n:
        raise KernelError("time_conv: out must have x's rows")
    single = int(ctx.host["max_q_len"]) == 1
    lib = _lib("headmix")
    _launch(lib, lib.gb_time_conv, _p(x), x.stride(0), _p(w), taps, _p(state) if taps > 1 else None, _p(ctx.tok_seq),
            _p(ctx.q_start), _p(ctx.pos0), _p(ctx.state_slots), _p(out), dtype_code(out), ldo, n, d, 1 if single else 0,
            _stream())
    if taps > 1 and not single:
        conv = _lib("shortconv")
        _launch(conv, conv.gb_conv_state, _p(x), F32, x.stride(0), _p(state), _p(ctx.q_start), _p(ctx.q_len),
                _p(ctx.state_slots), ctx.num_seqs, d, taps, _stream())


def norm_slices(rows: torch.Tensor, eps: float, first, second=None) -> None:
    """RMS norms with a weight over runs of columns of ``rows``: ``first`` and ``second`` are (column, gamma float32 [d],
    out [n, >= d] of the rows' type); out = gamma * v / sqrt(mean(v^2) + eps) over the run's d columns."""
    n = rows.shape[0]
    ld = _act_rows(rows, rows.dtype, 1, "rows")
    args = []
    for item in (first, second):
        if item is None:
            args += [0, 0, None, None, 0]
            continue
        col, gamma, out = item
        d = gamma.numel()
        _dev(rows, gamma, out)
        _f32_rows(gamma, (d,), "gamma")
        if col < 0 or col + d > rows.shape[1] or out.shape[0] != n:
            raise KernelError("norm_slices: a run of columns beyond the rows")
        args += [int(col), d, _p(gamma), _p(out), _act_rows(out, rows.dtype, d, "out")]
    lib = _lib("headmix")
    _launch(lib, lib.gb_norm_slices, _p(rows), dtype_code(rows), ld, n, float(eps), *args, _stream())


def _store_args(slots, k_pages, v_pages, dtype, n: int, kv_heads: int, head_cols: int, what: str):
    if slots is None:
        return None, None, None, 0
    _dev(slots, k_pages, v_pages)
    _i32(slots, "slots", n)
    _, p_heads, page_size, p_hd = _check_pages(k_pages, v_pages, dtype, what)
    if (p_heads, p_hd) != (kv_heads, head_cols):
        raise KernelError(f"{what}: pages do not have this layer's kv heads and head size")
    return _p(slots), _p(k_pages), _p(v_pages), page_size


def latent_heads(q: torch.Tensor, kv: torch.Tensor, k_rot: torch.Tensor, cos: Optional[torch.Tensor],
                 sin: Optional[torch.Tensor], rot: int, out: torch.Tensor, head_cols: int, slots: Optional[torch.Tensor],
                 k_pages: Optional[torch.Tensor], v_pages: Optional[torch.Tensor], n_heads: int, dim: int, rot_dim: int,
                 vdim: int) -> None:
    """Heads for attention through latents.  ``q`` [n, heads * (dim + rot_dim)]; ``kv`` [n, heads * dim + heads * vdim] (the
    heads' own key parts, then their values); ``k_rot`` [n, rot_dim], the key part all heads share.  The first ``rot`` of
    the rot_dim columns of every query head and of the shared part are turned in half-split pairs (i, i + rot / 2) by
    the rows' angles (``cos``, ``sin`` float32 [n, rot / 2]).  ``out`` [n, 3 * heads * head_cols]: query heads, key heads
    [own part | shared part], value heads, each filled up with zeros; with ``slots`` keys and values also go to the pages."""
    _dev(q, kv, k_rot, cos, sin, out)
    n, dt = q.shape[0], q.dtype
    ldq = _act_rows(q, dt, n_heads * (dim + rot_dim), "q")
    ldkv = _act_rows(kv, dt, n_heads * (dim + vdim), "kv")
    ldr = _act_rows(k_rot, dt, rot_dim, "k_rot") if rot_dim else max(1, k_rot.stride(0))
    ldo = _act_rows(out, dt, 3 * n_heads * head_cols, "out")
    if rot:
        for t in (cos, sin):
            if t is None or t.dtype != torch.float32 or not t.is_contiguous() or t.shape[1] != rot // 2 or t.shape[0] < n:
                raise KernelError("latent_heads: cos/sin must be contiguous float32 [n, rot / 2]")
    store = _store_args(slots, k_pages, v_pages, dt, n, n_heads, head_cols, "latent_heads")
    lib = _lib("headmix")
    _launch(lib, lib.gb_latent_heads, _p(q), ldq, _p(kv), ldkv, _p(k_rot), ldr, dtype_code(q), _p(cos) if rot else None,
            _p(sin) if rot else None, int(rot), _p(out), ldo, int(head_cols), *store, n, n_heads, dim, rot_dim, vdim, _stream())


def diff_heads(proj: torch.Tensor, w_q: torch.Tensor, w_k: torch.Tensor, eps: float, coef: float, every: int,
               positions: torch.Tensor, out: torch.Tensor, head_cols: int, slots: Optional[torch.Tensor],
               k_pages: Optional[torch.Tensor], v_pages: Optional[torch.Tensor], n_heads: int, n_kv_heads: int, dim: int,
               vdim: int) -> None:
    """Heads for differential attention.  ``proj`` [n, heads * 2 dim + kv heads * 2 dim + kv heads * vdim]: every query
    and key head holds two maps of dim columns.  Each map is divided by its root mean square and multiplied by ``w_q``
    (``w_k``), float32 [dim]; query maps also by 1 + coef * ln(floor((position + 1) / every) + 1) (``every`` 0: not).
    ``out`` [n, (2 heads + 2 kv heads) * head_cols]: query heads [q1 | 0], [0 | q2] for each head, key heads [k1 | k2],
    value heads, filled up with zeros; with ``slots`` keys and values also go to the pages (kv heads of head_cols)."""
    _dev(proj, w_q, w_k, positions, out)
    n, dt = proj.shape[0], proj.dtype
    ld = _act_rows(proj, dt, (n_heads + n_kv_heads) * 2 * dim + n_kv_heads * vdim, "proj")
    ldo = _act_rows(out, dt, (2 * n_heads + 2 * n_kv_heads) * head_cols, "out")
    _f32_rows(w_q, (dim,), "w_q")
    _f32_rows(w_k, (dim,), "w_k")
    _i32(positions, "positions", n)
    store = _store_args(slots, k_pages, v_pages, dt, n, n_kv_heads, head_cols, "diff_heads")
    lib = _lib("headmix")
    _launch(lib, lib.gb_diff_heads, _p(proj), dtype_code(proj), ld, _p(w_q), _p(w_k), float(eps), float(coef), int(every),
            _p(positions), _p(out), ldo, int(head_cols), *store, n, n_heads, n_kv_heads, dim, vdim, _stream())


def diff_combine(att: torch.Tensor, head_cols: int, lam: torch.Tensor, mult: float, eps: float, out: torch.Tensor,
                 n_heads: int, vdim: int) -> None:
    """out[:, h] = mult * o / sqrt(mean(o^2) + eps), o = a1 - lam * a2, where a1, a2 are heads 2 h and 2 h + 1 of ``att``
    ([n, 2 heads * head_cols], of out's type or float32) cut to vdim columns and ``lam`` is one float32 on the device;
    ``out`` [n, heads * vdim]."""
    _dev(att, lam, out)
    n, dt = att.shape[0], out.dtype
    if att.dtype not in (dt, torch.float32):
        raise KernelError("diff_combine: att must have out's type or be float32")
    lda = _act_rows(att, att.dtype, 2 * n_heads * head_cols, "att")
    ldo = _act_rows(out, dt, n_heads * vdim, "out")
    _f32_rows(lam, (1,), "lam")
    lib = _lib("headmix")
    _launch(lib, lib.gb_diff_combine, _p(att), dtype_code(att), lda, int(head_cols), _p(lam), float(mult), float(eps),
            _p(out), dtype_code(out), ldo, n, n_heads, vdim, _stream())


def gate_heads(att: torch.Tensor, head_cols: int, gate: torch.Tensor, out: torch.Tensor, n_heads: int, vdim: int) -> None:
    """out[:, h, c] = att[:, h, c] * sigmoid(gate[:, h, c]) for c < vdim: ``att`` [n, heads * head_cols], ``gate`` and
    ``out`` [n, heads * vdim]."""
    _dev(att, gate, out)
    n, dt = att.shape[0], att.dtype
    lib = _lib("headmix")
    _launch(lib, lib.gb_gate_heads, _p(att), _act_rows(att, dt, n_heads * head_cols, "att"), int(head_cols), _p(gate),
            _act_rows(gate, dt, n_heads * vdim, "gate"), dtype_code(att), _p(out), _act_rows(out, dt, n_heads * vdim, "out"),
            n, n_heads, vdim, _stream())


def poly_norm(z: torch.Tensor, coef: torch.Tensor, eps: float, out: torch.Tensor) -> None:
    """out = a N(z) + b N(z^2) + c N(z^3) + e over every row, powers element by element, N(v) = v / sqrt(mean(v^2) + eps);
    ``coef`` float32 [4] = a, b, c, e."""
    _dev(z, coef, out)
    n, d = z.shape
    _f32_rows(coef, (4,), "coef")
    if out.shape != z.shape:
        raise KernelError("poly_norm: out must have z's shape")
    lib = _lib("headmix")
    _launch(lib, lib.gb_poly_norm, _p(z), _act_rows(z, z.dtype, d, "z"), _p(coef), float(eps), _p(out),
            _act_rows(out, z.dtype, d, "out"), dtype_code(z), n, d, _stream())


NORM_ADD_ROWS_MAX = 8192   # the widest row that headmix.hip keeps in registers (slices of y, the convolution after)


def norm_add_takes_rows(d: int) -> bool:
    """Whether ``norm_add`` takes y in slices, or does the next convolution, for rows of d columns."""
    return d % 4 == 0 and d <= NORM_ADD_ROWS_MAX


def norm_add(x: torch.Tensor, y: torch.Tensor, g: torch.Tensor, eps: float, rounded: Optional[torch.Tensor] = None,
             slices: int = 1, conv: Optional[tuple] = None, ctx=None) -> None:
    """x += g * y / sqrt(mean(y^2) + eps) row by row: x float32 [n, d], ``g`` one float32 on the device.  y is float32
    [n, d], or with ``slices`` > 1 float32 [slices, n, d] whose sum over the slices it is (what a product that divides k
    leaves, ``gemm_slices``).  ``rounded`` ([n, d], any activations' type) receives the new x; with ``conv=(w, state)``, w [taps, d] as ``time_conv`` takes it
    (a step in which every request brings one row; ``ctx`` the step) it receives new x + conv(new x) instead, the rows
    the next mixer reads, and the requests' slots in ``state`` move on as in ``time_conv``."""
    _dev(x, y, g, rounded)
    n, d = x.shape
    _f32_rows(x, (n, d), "x")
    if slices > 1:
        if y.dtype != torch.float32 or not y.is_contiguous() or y.numel() < slices * n * d or not norm_add_takes_rows(d):
            raise KernelError("norm_add: slices of y must be contiguous float32 [slices, n, d], d a multiple of 4 up to "
                              f"{NORM_ADD_ROWS_MAX}")
    else:
        _f32_rows(y, (n, d), "y")
    _f32_rows(g, (1,), "g")
    if rounded is not None and (tuple(rounded.shape) != (n, d) or not rounded.is_contiguous()):
        raise KernelError("norm_add: rounded must be contiguous [n, d]")
    w = state = None
    taps = 0
    if conv is not None:
        w, state = conv
        _dev(w, state)
        taps = w.shape[0]
        _f32_rows(w, (taps, d), "conv w")
        if (rounded is None or ctx is None or int(ctx.host["max_q_len"]) != 1 or not norm_add_takes_rows(d)
                or not 1 <= taps <= TIME_CONV_MAX_TAPS):
            raise KernelError("norm_add: the convolution after it goes with a step of single rows, a result and rows of a "
                              f"multiple of 4 up to {NORM_ADD_ROWS_MAX} columns")
        if taps > 1 and (state is None or state.dtype != torch.float32 or not state.is_contiguous()
                         or tuple(state.shape[1:]) != (taps - 1, d)):
            raise KernelError("norm_add: state must be contiguous float32 [slots, taps - 1, d]")
    lib = _lib("headmix")
    _launch(lib, lib.gb_norm_add, _p(x), _p(y), int(slices), n * d, _p(g), float(eps), _p(rounded),
            dtype_code(rounded) if rounded is not None else F32, n, d, _p(w), taps, _p(state) if taps > 1 else None,
            _p(ctx.tok_seq) if conv is not None else None, _p(ctx.pos0) if conv is not None else None,
            _p(ctx.state_slots) if conv is not None else None, _stream())


# ------------------------------------------------------------------- routed experts
MOE_MAX_EXPERTS = 512   # moe.hip: a lane of the routing wave holds eight experts
MOE_MAX_TOP = 16


def moe_route(z: torch.Tensor, n_experts: int, correction: Optional[torch.Tensor], top: int, scale: float, shared,
              combine: torch.Tensor, ids: torch.Tensor, weights: torch.Tensor, softmax: bool = False, renorm: bool = True,
              groups: int = 0, keep_groups: int = 0) -> None:
    """From router logits ``z`` (float32 [n, experts (+ 1)]): scores sigmoid(z), or with ``softmax`` the softmax over all
    experts; the ``top`` experts with the largest score + correction (of equal ones the lower index), with ``groups`` only
    out of the ``keep_groups`` runs of experts / groups neighbours whose best score + correction is largest; their weights
    score * scale, with ``renorm`` divided by (the sum of the chosen scores + 1e-20).
    ``ids`` int32 and ``weights`` float32 [n, top] receive the choice, ``combine`` float32 [n, experts (+ 1)] a row of
    weights with zeros for the others; with ``shared`` one more column for an expert that every token uses: sigmoid of
    z's last column (True, "gate"), or 1 ("whole")."""
    _dev(z, correction, combine, ids, weights)
    n = z.shape[0]
    cols = n_experts + (1 if shared else 0)
    if z.dtype != torch.float32 or z.dim() != 2 or z.stride(1) != 1 or z.shape[1] < n_experts + (1 if shared and shared != "whole" else 0):
        raise KernelError("moe_route: z must be float32 [n, experts (+ 1)] with dense rows")
    _f32_rows(combine, (n, cols), "combine")
    _f32_rows(weights, (n, top), "weights")
    _i32(ids, "ids", n * top)
    if correction is not None:
        _f32_rows(correction, (n_experts,), "correction")
    lib = _lib("moe")
    if softmax or not renorm or groups or shared == "whole":
        _launch(lib, lib.gb_moe_route_by, _p(z), z.stride(0), n, n_experts, _p(correction), int(top), float(scale),
                2 if shared == "whole" else 1 if shared else 0, 1 if softmax else 0, 1 if renorm else 0, int(groups),
                int(keep_groups), _p(combine), _p(ids), _p(weights), _stream())
        return
    _launch(lib, lib.gb_moe_route, _p(z), z.stride(0), n, n_experts, _p(correction), int(top), float(scale),
            1 if shared else 0, _p(combine), _p(ids), _p(weights), _stream())


def moe_relu2_units(z: torch.Tensor, combine: Optional[torch.Tensor], out: torch.Tensor, n_experts: int, ff: int) -> None:
    """out[t, j] = relu(z[t, j])^2 * combine[t, expert of column j] for units of one up matrix: columns e * ff .. of ``z``
    and ``out`` ([n, I]) are expert e's, those from experts * ff on the shared expert's (weight in the last column of
    ``combine``).  Without ``combine`` every weight is 1 (rows that are one expert's own)."""
    _dev(z, combine, out)
    n, inter = out.shape
    if z.shape != (n, inter) or z.stride(1) != 1 or out.stride(1) != 1:
        raise KernelError("moe_relu2_units: z and out must be [n, I] with dense rows")
    if combine is not None and (combine.dtype != torch.float32 or not combine.is_contiguous() or combine.shape[0] != n):
        raise KernelError("moe_relu2_units: combine must be contiguous float32 [n, experts (+ 1)]")
    lib = _lib("moe")
    _launch(lib, lib.gb_moe_relu2_units, _p(z), dtype_code(z), z.stride(0), _p(combine), combine.shape[1] if combine is not None else 0,
            _p(out), dtype_code(out), out.stride(0), n, inter, n_experts, ff, _stream())


def moe_gated_units(gate_up: torch.Tensor, combine: torch.Tensor, out: torch.Tensor, n_experts: int, ff: int) -> None:
    """out[t, j] = silu(gate) * up * combine[t, expert of column j]: ``gate_up`` [n, 2 * I] holds the experts' gate columns, the
    experts' up columns, then the shared expert's gate columns and its up columns; columns e * ff .. of ``out`` are expert
    e's, those from experts * ff on the shared expert's (weight in the last column of ``combine``)."""
    _dev(gate_up, combine, out)
    n, inter = out.shape
    if gate_up.shape != (n, 2 * inter) or gate_up.stride(1) != 1 or not out.is_contiguous():
        raise KernelError("moe_gated_units: gate_up must be [n, 2 I] and out contiguous [n, I]")
    if combine.dtype != torch.float32 or not combine.is_contiguous() or combine.shape[0] != n:
        raise KernelError("moe_gated_units: combine must be contiguous float32 [n, experts (+ 1)]")
    lib = _lib("moe")
    _launch(lib, lib.gb_moe_gated_units, _p(gate_up), dtype_code(gate_up), gate_up.stride(0), _p(combine), combine.shape[1],
            _p(out), dtype_code(out), n, inter, n_experts, ff, _stream())


# ------------------------------------------------------------------- small residual operations
def moe_sort_tiles(entries: int, n_experts: int, tile_rows: int) -> int:
    """Row tiles that ``moe_sort`` may need: every expert's last tile may be short."""
    return entries // tile_rows + n_experts


def moe_sort(ids: torch.Tensor, n_experts: int, tile_rows: int, counts: torch.Tensor, rows: torch.Tensor, pos: torch.Tensor,
             tile_map: torch.Tensor) -> None:
    """Orders the entries of ``ids`` (int32 [n, top]) by expert, entries of an expert in the order of the tokens:
    ``rows`` [n * top] receives the token behind each sorted row, ``pos`` [n, top] the sorted row of each entry, and
    ``tile_map`` [tiles, 3] cuts the sorted rows into tiles of at most ``tile_rows`` rows of one expert (expert, first row,
    end of the expert's rows; expert -1 for the tiles left over).  ``counts`` [experts] is scratch."""
    _dev(ids, counts, rows, pos, tile_map)
    n, top = ids.shape
    _i32(ids, "ids", n * top)
    _i32(counts, "counts", n_experts)
    _i32(rows, "rows", n * top)
    _i32(pos, "pos", n * top)
    tiles = tile_map.shape[0]
    _i32(tile_map, "tile_map", tiles * 3)
    lib = _lib("moe")
    _launch(lib, lib.gb_moe_sort, _p(ids), n, top, n_experts, tile_rows, tiles, _p(counts), _p(rows), _p(pos), _p(tile_map), _stream())


def moe_combine(y: torch.Tensor, pos: torch.Tensor, weights: torch.Tensor, y_shared: Optional[torch.Tensor],
                gates: Optional[torch.Tensor], out: torch.Tensor, accumulate: bool) -> None:
    """out[t] (+)= sum over k of weights[t, k] * y[pos[t, k]] + gates[t] * y_shared[t], all float32; ``gates`` may be a
    column of a wider tensor."""
    _dev(y, pos, weights, y_shared, gates, out)
    n, top = weights.shape
    d = out.shape[1]
    for t, what in ((y, "y"), (out, "out"), (y_shared, "y_shared")):
        if t is not None and (t.dtype != torch.float32 or t.dim() != 2 or t.stride(1) != 1 or t.shape[1] != d):
            raise KernelError(f"moe_combine: {what} must be float32 [rows, {d}] with dense rows")
    if out.shape[0] != n or y.shape[0] < n * top or (y_shared is not None and (y_shared.shape[0] != n or gates is None or gates.shape[0] != n)):
        raise KernelError("moe_combine: y holds a row for every entry, out, y_shared and gates a row for every token")
    _f32_rows(weights, (n, top), "weights")
    _i32(pos, "pos", n * top)
    lib = _lib("moe")
    _launch(lib, lib.gb_moe_combine, _p(y), y.stride(0), _p(pos), _p(weights), top, _p(y_shared),
            y_shared.stride(0) if y_shared is not None else 0, _p(gates), gates.stride(0) if gates is not None else 0,
            _p(out), out.stride(0), 1 if accumulate else 0, n, d, y.shape[0], _stream())


def gemm_grouped_takes(a: torch.Tensor, w: torch.Tensor, group_stride: int) -> bool:
    """Whether ``gemm_grouped`` serves these operands: bfloat16, 16-byte aligned rows and groups."""
    return (a.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and a.shape[1] % 8 == 0 and a.stride(0) % 8 == 0
            and w.stride(0) % 8 == 0 and group_stride % 8 == 0 and a.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0)


def gemm_grouped(a: torch.Tensor, rows: Optional[torch.Tensor], w: torch.Tensor, group_stride: int, n_out: int,
                 tile_map: torch.Tensor, tile_rows: int, out: torch.Tensor, silu_mul: bool = False, up_offset: int = 0) -> None:
    """Products of groups of rows with a matrix of their own each.  Sorted row r of the product reads row ``rows[r]`` of
    ``a`` (row r without ``rows``); ``tile_map`` (as ``moe_sort`` writes it) names each row tile's group and rows; group g
    uses the ``n_out`` rows of ``w`` that begin ``g * group_stride`` elements into it.  ``silu_mul``: the group's rows
    are n_out / 2 gate rows, with the up row of each ``up_offset`` rows behind it, and out = silu(gate) * up."""
    _dev(a, rows, w, tile_map, out)
    K = a.shape[1]
    cols = n_out // 2 if silu_mul else n_out
    if not gemm_grouped_takes(a, w, group_stride) or a.stride(1) != 1 or w.stride(1) != 1 or w.shape[1] < K:
        raise KernelError("gemm_grouped: operands must be bfloat16 with dense, 16-byte aligned rows")
    if out.dim() != 2 or out.stride(1) != 1 or out.shape[1] != cols or (silu_mul and out.dtype != torch.bfloat16):
        raise KernelError(f"gemm_grouped: out must be [rows, {cols}] with dense rows (bfloat16 behind silu(gate) * up)")
    tiles = tile_map.shape[0]
    _i32(tile_map, "tile_map", tiles * 3)
    if rows is not None:
        _i32(rows, "rows")
    lib = _lib("gemm_bf16")
    _launch(lib, lib.gb_gemm_bf16_grouped, _p(a), a.stride(0), _p(rows), _p(w), w.stride(0), int(group_stride), int(up_offset),
            _p(out), out.stride(0), dtype_code(out), _p(tile_map), tiles, tile_rows, n_out, K, 2 if silu_mul else 0, _stream())


def embed_pairs(table: torch.Tensor, pairs: torch.Tensor, ctx, out: torch.Tensor, buckets: int, mul_prev: int, mul_cur: int,
                prev: torch.Tensor) -> None:
    """out[i] = table[id_i] + pairs[(id_(i-1) * mul_prev + id_i * mul_cur) mod buckets], row ``buckets`` of ``pairs`` for
    a request's first token; float32 [n, d] or [copies, n, d].  ``prev`` int32 [slots, 1]: the last token of each
    request's earlier steps, read for the first row of a request that goes on and left for the next step."""
    _dev(table, pairs, out, prev)
    copies = out.shape[0] if out.dim() == 3 else 1
    n, d = out.shape[-2:]
    if out.dtype != torch.float32 or not out.is_contiguous() or not table.is_contiguous() or table.shape[1] != d \
            or not pairs.is_contiguous() or tuple(pairs.shape) != (buckets + 1, d) or pairs.dtype != table.dtype:
        raise KernelError("embed_pairs: out must be contiguous float32 [n, d], table [vocab, d], pairs [buckets + 1, d]")
    if prev.dtype != torch.int32 or not prev.is_contiguous() or prev[0].numel() != 1:
        raise KernelError("embed_pairs: prev must be contiguous int32, one entry a slot")
    lib = _lib("elementwise")
    _launch(lib, lib.gb_embed_pairs, _p(table), _p(pairs), dtype_code(table), _p(ctx.token_ids), _p(out), n, d, table.shape[0],
            int(buckets), int(mul_prev), int(mul_cur), _p(ctx.tok_seq), _p(ctx.q_start), _p(ctx.q_len), _p(ctx.pos0),
            _p(ctx.state_slots), _p(prev), int(copies), _stream())


def glu_clamped(gate_up: torch.Tensor, out: torch.Tensor, limit: float, alpha: float) -> None:
    """out = g * sigmoid(alpha * g) * (u + 1) with g = min(gate, limit), u = clamp(up, -limit, limit); ``gate_up`` [n, 2 I]
    (gate columns, then up columns) in float32 or the result's type."""
    _dev(gate_up, out)
    n, inter = out.shape
    if gate_up.shape != (n, 2 * inter) or gate_up.stride(1) != 1 or not out.is_contiguous():
        raise KernelError("glu_clamped: gate_up must be [n, 2 I] and out contiguous [n, I]")
    lib = _lib("elementwise")
    _launch(lib, lib.gb_glu_clamped, _p(gate_up), dtype_code(gate_up), gate_up.stride(0), _p(out), dtype_code(out), n, inter,
            float(limit), float(alpha), _stream())


def axpy_rows(x: torch.Tensor, y: Optional[torch.Tensor] = None, alpha: float = 1.0, bias: Optional[torch.Tensor] = None) -> None:
    """x[r, :] += alpha * y[r, :] + bias, all float32; ``y`` or ``bias`` may be None."""
    _dev(x, y, bias)
    n, d = x.shape
    if x.dtype != torch.float32 or not x.is_contiguous():
        raise KernelError("axpy_rows: x must be contiguous float32 [n, d]")
    if y is not None and (y.dtype != torch.float32 or not y.is_contiguous() or y.shape != x.shape):
        raise KernelError("axpy_rows: y must be contiguous float32 of x's shape")
    if bias is not None and (bias.dtype != torch.float32 or not bias.is_contiguous() or bias.numel() != d):
        raise KernelError("axpy_rows: bias must be contiguous float32 [d]")
    lib = _lib("elementwise")
    _launch(lib, lib.gb_axpy_rows, _p(x), _p(y), float(alpha), _p(bias), n, d, _stream())


# ------------------------------------------------------------------------ products
FUSED_NORM_MAX_ROWS = 16   # measured: beyond one 16-row block the re-reading of float32 rows costs more than a norm pass
HEAD_PREPARED_MAX_ROWS = 16   # beyond, the vocabulary product goes through tiles that take whole rows only


def head_takes_parts(rows: int) -> bool:
    """Whether a vocabulary product of ``rows`` rows can scale by the partial sums that the product before it left
    (``gemm(..., rms_parts=)``) instead of reading rows that a norm kernel wrote."""
    return rows <= HEAD_PREPARED_MAX_ROWS


def parts_stride(rows: int) -> int:
    """Floats a tile of partial sums holds (``gemm(..., emit=)`` / ``rms_parts=``): one per row, 8 for up to 8 rows,
    64 beyond."""
    return 8 if rows <= 8 else 64


@functools.lru_cache(maxsize=4096)   # a pure function of the sizes, asked for at every product
def gemm_emit_parts(rows: int, n: int) -> int:
    """How many partial sums an accumulating bfloat16 product of ``rows`` rows and ``n`` columns writes when
    asked to prepare the norm that follows (``gemm(..., emit=...)``); 0 if that product cannot."""
    return int(_lib("gemm_bf16").gb_gemm_bf16_emit_parts(int(rows), int(n)))


@functools.lru_cache(maxsize=4096)   # a pure function of the sizes, asked for at every product
def gemm_emit_mode(rows: int, n: int, k: int) -> int:
    """What an accumulating bfloat16 product of these sizes can do for the RMS norm that reads the residual after
    it: 0 nothing; 1 the operand and partial sums (``gemm(..., emit=(gamma, h, parts))``, see ``gemm_emit_parts``);
    2 the whole norm (``gemm(..., emit=(gamma, h, eps), workspace=...)``: h receives the normed rows)."""
    return int(_lib("gemm_bf16").gb_gemm_bf16_emit_mode(int(rows), int(n), int(k)))


@functools.lru_cache(maxsize=4096)   # a pure function of the sizes, asked for at every product
def gemm_split_floats(rows: int, n: int, k: int) -> int:
    """Floats of workspace with which a bfloat16 product of these sizes would divide k over workgroups
    (``gemm(..., workspace=)``); 0 if it would not: only products with few tiles do."""
    f = _lib("gemm_bf16").gb_gemm_bf16_split_floats
    f.restype = C.c_longlong
    return int(f(int(rows), int(n), int(k)))


def gemm_slices(rows: int, n: int, k: int) -> int:
    """Slices into which ``gemm_partial`` divides k for a bfloat16 product of these sizes (1: it does not)."""
    return int(_lib("gemm_bf16").gb_gemm_bf16_slices(int(rows), int(n), int(k)))


def gemm_partial(a: torch.Tensor, w: torch.Tensor, workspace: torch.Tensor) -> int:
    """The first pass alone of a bfloat16 product that divides k (``gemm_slices`` > 1): ``workspace`` (float32, at least
    ``gemm_split_floats`` elements) receives [slices, rows, out features], slice z the product over the z-th run of k;
    whoever reads them adds them in their order (``norm_add(slices=)``).  Returns the number of slices."""
    _dev(a, w, workspace)
    M, K = a.shape
    N = w.shape[0]
    if a.dtype != torch.bfloat16 or w.dtype != torch.bfloat16 or w.shape[1] != K:
        raise KernelError(f"gemm_partial: bfloat16 operands of one inner size, got a {tuple(a.shape)} {a.dtype}, w {tuple(w.shape)} {w.dtype}")
    if workspace.dtype != torch.float32 or not workspace.is_contiguous():
        raise KernelError("gemm_partial: the workspace must be contiguous float32")
    slices = gemm_slices(M, N, K)
    lib = _lib("gemm_bf16")
    _launch(lib, lib.gb_gemm_bf16_partial, _p(a), _rows(a, "a"), _p(w), _rows(w, "w"), _p(workspace), workspace.numel(), M, N, K,
            _stream())
    return slices


def gemm(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor, accumulate: bool = False, silu_mul: bool = False,
         rms: Optional[tuple] = None, emit: Optional[tuple] = None, rms_parts: Optional[tuple] = None,
         workspace: Optional[torch.Tensor] = None) -> None:
    """out (+)= a . w^T with w in the [out features, in features] layout.
    float32 operands take the true 32-bit kernel; bfloat16 operands the matrix-core kernels,
    with out in bfloat16 or float32 (float32 when accumulating into the residual).
    ``silu_mul`` (bfloat16): w stacks gate rows over up rows and out[m, j] =
    silu(a . gate_j) * (a . up_j), of half as many columns.
    ``rms=(gamma, eps)`` (bfloat16 w and out, at most 64 rows): a is the float32 residual and the
    product is that of its RMS-normed rows, the norm computed inside the product's kernel.
    ``emit=(gamma, h, parts)`` (accumulating bfloat16 product with ``gemm_emit_mode(M, N, K) == 1``: at most 64
    rows): besides the new residual r in out, h[m, n] = bf16(gamma[n] r[m, n]) and float32 parts[tile, m] of
    sum(r^2) over the tile's columns are written (``gemm_emit_parts`` tiles, ``parts_stride(M)`` floats a tile):
    the work of the RMS norm that reads the residual next.
    ``emit=(gamma, h, eps)`` with a number as the third entry (``gemm_emit_mode(M, N, K) == 2``, with the
    workspace): h receives the rows of that norm itself, gamma * r / sqrt(mean(r^2) + eps).
    ``rms_parts=(parts, n_parts, eps)`` (at most 64 rows): a is such an h, and the product is scaled by
    1 / sqrt(sum(parts[:, m]) / K + eps) to that of the normed rows.
    ``workspace`` (float32, at least ``gemm_split_floats(M, N, K)`` elements): lets a bfloat16 product of
    more than 16 rows and few tiles divide k over workgroups; their sums are added in a fixed order."""
    _dev(a, w, out)
    M, K = a.shape
    N = w.shape[0]
    if w.shape[1] != K or out.shape != (M, N // 2 if silu_mul else N):
        raise KernelError(f"gemm: shapes do not match: a {tuple(a.shape)}, w {tuple(w.shape)}, out {tuple(out.shape)}")
    if silu_mul and (w.dtype != torch.bfloat16 or accumulate or N % 16):
        raise KernelError("gemm: the fused SiLU-multiply takes bfloat16 operands and gate/up stacks of a "
                          "multiple of 8 rows each")
    lda, ldw, ldc = _rows(a, "a"), _rows(w, "w"), _rows(out, "out")
    if rms is not None:
        gamma, eps = rms
        if (a.dtype != torch.float32 or w.dtype != torch.bfloat16 or out.dtype != torch.bfloat16 or accumulate
                or M > 64 or gamma.numel() != K or not gamma.is_contiguous()):
            raise KernelError("gemm: the fused RMS norm takes float32 rows (at most 64), bfloat16 weights and result")
        if emit is not None or rms_parts is not None:
            raise KernelError("gemm: one way of fusing the norm at a time")
        lib = _lib("gemm_bf16")
        _launch(lib, lib.gb_gemm_bf16, _p(a), lda, _p(w), ldw, _p(out), ldc, BF16, M, N, K, 2 if silu_mul else 0,
                                     _p(gamma), dtype_code(gamma), float(eps), None, 0, None, 0, None, None, 0,
                                     None, 0, _stream())
    elif a.dtype == torch.float32 and w.dtype == torch.float32:
        if out.dtype != torch.float32:
            raise KernelError("gemm: 32-bit operands need a 32-bit result")
        lib = _lib("gemm_f32")
        _launch(lib, lib.gb_gemm_f32, _p(a), lda, _p(w), ldw, _p(out), ldc, M, N, K, 1 if accumulate else 0, _stream())
    elif a.dtype == torch.bfloat16 and w.dtype == torch.bfloat16:
        if accumulate and out.dtype != torch.float32:
            raise KernelError("gemm: accumulation is into a 32-bit result")
        lib = _lib("gemm_bf16")
        if workspace is not None:
            _dev(workspace)
            if workspace.dtype != torch.float32 or not workspace.is_contiguous():
                raise KernelError("gemm: the workspace must be contiguous float32")
        e_gamma = e_h = e_ss = parts = None
        e_ldh = n_parts = 0
        eps = 0.0
        if emit is not None and not isinstance(emit[2], torch.Tensor):
            e_gamma, e_h, eps = emit
            _dev(e_gamma, e_h)
            if (not accumulate or workspace is None or gemm_emit_mode(M, N, K) != 2 or e_gamma.numel() != N
                    or not e_gamma.is_contiguous() or e_h.dtype != torch.bfloat16 or e_h.shape != (M, N)):
                raise KernelError("gemm: the whole norm can be emitted by an accumulating product that divides k "
                                  "(gemm_emit_mode 2, with its workspace), given gamma of N entries and a bfloat16 [M, N] buffer")
            e_ldh = _rows(e_h, "emit h")
        elif emit is not None:
            e_gamma, e_h, e_ss = emit
            _dev(e_gamma, e_h, e_ss)
            want = gemm_emit_parts(M, N)
            if (not accumulate or want == 0 or e_gamma.numel() != N or not e_gamma.is_contiguous()
                    or e_h.dtype != torch.bfloat16 or e_h.shape != (M, N) or e_ss.dtype != torch.float32
                    or not e_ss.is_contiguous() or e_ss.numel() < want * parts_stride(M)):
                raise KernelError("gemm: emit needs an accumulating product that gemm_emit_parts accepts, gamma of N "
                                  "entries, a bfloat16 [M, N] operand buffer and parts_stride(M) float32 per part")
            e_ldh = _rows(e_h, "emit h")
        if rms_parts is not None:
            parts, n_parts, eps = rms_parts
            _dev(parts)
            if (M > 64 or accumulate or parts.dtype != torch.float32 or not parts.is_contiguous()
                    or parts.numel() < n_parts * parts_stride(M) or n_parts <= 0):
                raise KernelError("gemm: partial sums of a norm go with at most 64 rows and a storing product")
        _launch(lib, lib.gb_gemm_bf16, _p(a), lda, _p(w), ldw, _p(out), ldc, dtype_code(out), M, N, K,
                                     2 if silu_mul else (1 if accumulate else 0), None, 0, float(eps),
                                     _p(e_gamma), dtype_code(e_gamma) if e_gamma is not None else 0, _p(e_h), e_ldh,
                                     _p(e_ss), _p(parts), int(n_parts), _p(workspace),
                                     workspace.numel() if workspace is not None else 0, _stream())
    else:
        raise KernelError(f"gemm: operand types {a.dtype} and {w.dtype} do not match a kernel")


def gemm_glu(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor, limit: float, alpha: float, plus: float = 1.0) -> None:
    """out = g' * sigmoid(alpha g') * (u' + plus) with g' = min(a . gate, limit) and u' = clamp(a . up, -limit, limit),
    formed where the product's tiles are finished: w stacks gate rows over up rows, all bfloat16, out [M, N / 2]."""
    _dev(a, w, out)
    M, K = a.shape
    N = w.shape[0]
    if (a.dtype != torch.bfloat16 or w.dtype != torch.bfloat16 or out.dtype != torch.bfloat16 or w.shape[1] != K
            or out.shape != (M, N // 2) or N % 2):
        raise KernelError(f"gemm_glu: bfloat16 a {tuple(a.shape)}, w {tuple(w.shape)}, out {tuple(out.shape)} do not match")
    lib = _lib("gemm_bf16")
    _launch(lib, lib.gb_gemm_bf16_glu, _p(a), _rows(a, "a"), _p(w), _rows(w, "w"), _p(out), _rows(out, "out"), M, N, K,
            float(limit), float(alpha), float(plus), _stream())


def gemm_takes(a: torch.Tensor, w: torch.Tensor) -> bool:
    """Whether ``gemm`` takes these operands: 32-bit ones always; bfloat16 ones whose inner size is a multiple of 8 and
    whose rows begin at 16-byte words."""
    if a.dtype != torch.bfloat16:
        return True
    return (a.shape[1] % 8 == 0 and a.stride(0) % 8 == 0 and w.stride(0) % 8 == 0 and a.data_ptr() % 16 == 0
            and w.data_ptr() % 16 == 0)


def gemm_plain(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor, accumulate: bool = False) -> None:
    """out (+)= a . w^T by the plain kernel (one thread a cell): operands of one type, bfloat16 or float32, of any size and
    alignment; out in the operands' type or float32.  What a model's odd sizes fall back to; ``gemm`` is the product."""
    _dev(a, w, out)
    M, K = a.shape
    N = w.shape[0]
    if w.shape[1] != K or out.shape != (M, N) or a.dtype != w.dtype:
        raise KernelError(f"gemm_plain: shapes or types do not match: a {tuple(a.shape)}, w {tuple(w.shape)}, out {tuple(out.shape)}")
    if accumulate and out.dtype != torch.float32:
        raise KernelError("gemm_plain: accumulation is into a 32-bit result")
    lib = _lib("elementwise")
    _launch(lib, lib.gb_gemm_plain, _p(a), _rows(a, "a"), _p(w), _rows(w, "w"), _p(out), _rows(out, "out"), dtype_code(a),
            dtype_code(out), M, N, K, 1 if accumulate else 0, _stream())


ROPE_PRODUCT_MAX_ROWS = 64


def gemm_rope(a: torch.Tensor, w: torch.Tensor, qkv: torch.Tensor, n_heads: int, n_kv_heads: int, head_dim: int,
              cos: Optional[torch.Tensor], sin: Optional[torch.Tensor], slots: Optional[torch.Tensor],
              k_pages: Optional[torch.Tensor], v_pages: Optional[torch.Tensor], rms: Optional[tuple] = None,
              rms_parts: Optional[tuple] = None) -> None:
    """The stacked query/key/value product of a step of at most 64 rows that rotates query and key heads
    (``cos``/``sin`` float32 ``[M, head_dim/2]``; None: no rotation) and writes key and value heads into
    the pages at ``slots`` (None: nothing stored) in its epilogue, besides writing ``qkv`` as ``gemm``
    does.  ``n_kv_heads`` 0: w holds query heads only.  ``rms`` / ``rms_parts`` as in ``gemm``."""
    _dev(a, w, qkv, cos, sin, slots, k_pages, v_pages)
    M, K = a.shape
    N = w.shape[0]
    if w.shape[1] != K or qkv.shape != (M, N) or N != (n_heads + 2 * n_kv_heads) * head_dim:
        raise KernelError(f"gemm_rope: shapes do not match: a {tuple(a.shape)}, w {tuple(w.shape)}, qkv {tuple(qkv.shape)}")
    if w.dtype != torch.bfloat16 or qkv.dtype != torch.bfloat16 or M > ROPE_PRODUCT_MAX_ROWS or head_dim % 16:
        raise KernelError("gemm_rope: bfloat16 weights and rows, at most 64 rows, head sizes in steps of 16")
    page_size = 0
    if slots is not None:
        _i32(slots, "slots", M)
        _, p_heads, page_size, p_hd = _check_pages(k_pages, v_pages, torch.bfloat16, "gemm_rope")
        if (p_heads, p_hd) != (n_kv_heads, head_dim):
            raise KernelError("gemm_rope: pages do not have this layer's kv heads and head size")
    if cos is not None:
        if sin is None or cos.shape[1] != head_dim // 2 or cos.shape[0] < M or cos.dtype != torch.float32 \
                or not cos.is_contiguous() or not sin.is_contiguous() or sin.shape != cos.shape:
            raise KernelError("gemm_rope: cos/sin must be contiguous float32 [M, head_dim/2]")
    gamma, eps, parts, n_parts = None, 0.0, None, 0
    if rms is not None:
        gamma, eps = rms
        if a.dtype != torch.float32 or gamma.numel() != K or not gamma.is_contiguous():
            raise KernelError("gemm_rope: the fused RMS norm takes float32 rows and a gamma of K entries")
    elif a.dtype != torch.bfloat16:
        raise KernelError("gemm_rope: rows must be bfloat16 (float32 only with rms=)")
    if rms_parts is not None:
        parts, n_parts, eps = rms_parts
        if rms is not None or parts.dtype != torch.float32 or not parts.is_contiguous() or parts.numel() < n_parts * parts_stride(M):
            raise KernelError("gemm_rope: partial sums of a norm go with no gamma and parts_stride(M) floats a part")
    lib = _lib("gemm_bf16")
    _launch(lib, lib.gb_gemm_bf16_rope, _p(a), _rows(a, "a"), _p(w), _rows(w, "w"), _p(qkv), _rows(qkv, "qkv"), M, N, K,
                                      _p(gamma), dtype_code(gamma) if gamma is not None else 0, float(eps), _p(parts),
                                      int(n_parts), _p(cos), _p(sin), _p(slots), _p(k_pages), _p(v_pages), n_heads,
                                      n_kv_heads, head_dim, page_size, _stream())


# ----------------------------------------------------------------------- attention
MAX_HEAD_DIM = 256        # attention_plain.hip: a head's dimensions are held by one block of threads
MAX_VOCAB = 1 << 20       # sampling.hip: a token id takes 20 bits of the (logit, token) key the sampler searches


PLAIN_SPLIT_MAX_PAIRS = 1024   # (token, head) pairs up to which a step of long contexts goes a workgroup a chunk


#: from so many rows of prompt portions on, ``attention_plain`` takes them eight rows a workgroup
PLAIN_GROUP_MIN_ROWS = 64


def attention_plain_split_floats(n: int, n_heads: int, head_dim: int, page_size: int, max_context: int,
                                 keep_first: int = 0) -> int:
    """Floats of workspace with which ``attention_plain`` spreads the chunks of long contexts over workgroups, or 0
    where it would not: many (token, head) pairs fill the chip by themselves, and a context of one chunk has
    nothing to spread.  The bits of the result are the same either way."""
    if n * n_heads > PLAIN_SPLIT_MAX_PAIRS or max_context <= 256:
        return 0
    f = _lib("attention_plain").gb_attention_plain_split_floats
    f.restype = C.c_longlong
    return int(f(n, n_heads, head_dim, page_size, max_context, int(keep_first)))


def attention_plain(q: torch.Tensor, out: torch.Tensor, positions: torch.Tensor, tok_seq: torch.Tensor,
                    tables: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor, n_heads: int,
                    scale: float, window: int = 0, workspace: Optional[torch.Tensor] = None, max_context: int = 0,
                    grouped: bool = False, keep_first: int = 0, chunk: int = 0, softcap: float = 0.0,
                    sinks: Optional[torch.Tensor] = None) -> None:
    """Paged attention, one block per (token, head); q may be a view into the stacked qkv rows.
    ``chunk`` > 0 (no window then): positions are cut into runs of ``chunk`` from 0 on and a token reads the keys of its
    own run up to itself; ``softcap`` > 0: scores pass softcap * tanh(score / softcap); ``sinks`` float32 [heads]:
    exp(sinks[h]) joins the softmax's denominator of head h and has no value.
    ``window`` > 0: a token at position p reads keys p - window + 1 .. p, and with ``keep_first`` also keys
    0 .. keep_first - 1 wherever the window has moved past them.
    ``workspace`` (float32, ``attention_plain_split_floats`` elements) with ``max_context`` (at least the most keys a
    token of the step reads): a workgroup a chunk of 256 keys and a second kernel that merges them, for steps of few
    tokens with long contexts; the same bits as without.  ``grouped`` (without a workspace): a workgroup takes eight
    rows and loads a key once where these are one request's consecutive tokens, for the rows of prompt portions; the
    same bits again."""
    _dev(q, out, positions, tok_seq, tables, k_pages, v_pages)
    n = q.shape[0]
    if q.dtype != out.dtype:
        raise KernelError("attention: q and out must share one element type")
    _, nkv, page_size, hd = _check_pages(k_pages, v_pages, q.dtype, "attention")
    if q.shape[1] != n_heads * hd or out.shape != (n, n_heads * hd):
        raise KernelError("attention: q and out must be [n, heads * head size]")
    _i32(positions, "positions", n)
    _i32(tok_seq, "tok_seq", n)
    if tables.dtype != torch.int32 or tables.dim() != 2 or tables.stride(1) != 1:
        raise KernelError("attention: block tables must be int32 [requests, pages]")
    if workspace is not None:
        _dev(workspace)
        if workspace.dtype != torch.float32 or not workspace.is_contiguous() or max_context <= 0:
            raise KernelError("attention: the workspace must be contiguous float32 and come with the longest context")
    lib = _lib("attention_plain")
    _launch(lib, lib.gb_attention_plain, _p(q), _rows(q, "q"), _p(out), _rows(out, "out"), dtype_code(q), _p(positions),
                                       _p(tok_seq), _p(tables), tables.stride(0), _p(k_pages), _p(v_pages), n,
                                       n_heads, nkv, hd, page_size, float(scale), int(window), int(keep_first),
                                       int(chunk), float(softcap), _p(_sinks(sinks, n_heads)),
                                       _p(workspace), workspace.numel() if workspace is not None else 0, int(max_context),
                                       1 if grouped else 0, _stream())


def _sinks(sinks: Optional[torch.Tensor], n_heads: int) -> Optional[torch.Tensor]:
    if sinks is not None and (not sinks.is_cuda or sinks.dtype != torch.float32 or not sinks.is_contiguous()
                              or sinks.numel() != n_heads):
        raise KernelError(f"attention: sinks must be contiguous float32 [{n_heads}] on the GPU")
    return sinks


def tuned_attention_supports(k_pages: torch.Tensor, n_heads: int, window: int, keep_first: int = 0) -> bool:
    """Whether the matrix-core attention kernels take this layer: bfloat16 pages, a head size that is
    a multiple of 16 up to 128, at most 16 query heads per kv head, pages of 16, 32, 64 ... keys."""
    _, nkv, n_pieces, page, piece = k_pages.shape
    hd = n_pieces * piece
    return (k_pages.dtype == torch.bfloat16 and hd % 16 == 0 and 16 <= hd <= 128 and n_heads % nkv == 0
            and n_heads // nkv <= 16 and page >= 16 and page & (page - 1) == 0)


@functools.lru_cache(maxsize=4096)   # a pure function of the sizes, asked for at every product
def decode_chunk(n_decode: int, n_kv_heads: int, max_context: int) -> int:
    """Keys per workgroup of the decode kernel: a multiple of 256.  With a workgroup for every compute
    unit from requests and kv heads alone (or for half of them, if the context is short), each takes a whole
    context (and sixteen waves: nothing is left to combine afterwards); otherwise small enough that the launch
    has about a thousand workgroups."""
    groups = max(1, n_decode * n_kv_heads)
    want_splits = 1 if groups >= 256 else min(256, max(1, 1024 // groups))   # the second pass combines up to 256
    if groups >= 128 and max_context <= 1024:
        # sixteen waves take a thousand keys in one round: the second pass would cost more than it saves (measured:
        # 32 requests of SmolLM2-360M -6 % a step, 4 of SmolLM2-1.7B -2 %; with 64 workgroups or 2,048 keys it is slower)
        want_splits = 1
    chunk = -(-max_context // want_splits)
    return max(256, -(-chunk // 256) * 256)


def attention_decode(q: torch.Tensor, out: torch.Tensor, ctx, cache, n_heads: int, scale: float, window: int,
                     keep_first: int = 0, chunk: int = 0, softcap: float = 0.0, sinks: Optional[torch.Tensor] = None) -> None:
    """Rows 0..n_decode-1 of the step (requests with a single token), split over their context."""
    n_dec = ctx.host["n_decode"]
    k_pages, v_pages = cache.k_pages, cache.v_pages
    _dev(q, out, k_pages, v_pages)
    _, nkv, page, hd = _check_pages(k_pages, v_pages, torch.bfloat16, "attention_decode")
    if q.dtype != torch.bfloat16 or out.dtype not in (torch.bfloat16, torch.float32) or q.shape[1] != n_heads * hd:
        raise KernelError("attention_decode: q must be bfloat16 [n, heads * head size], out bfloat16 or float32")
    tables = ctx.tables[cache.group]
    max_context = int(ctx.host["max_context"])
    mask_chunk = int(chunk)   # the runs of positions a token sees; ``chunk`` below is the keys a workgroup takes
    chunk = decode_chunk(n_dec, nkv, max_context)
    splits = -(-max_context // chunk)
    ws_acc = ctx.buffer("attn_ws_acc", (n_dec * n_heads * splits * hd,), torch.float32)
    ws_ml = ctx.buffer("attn_ws_ml", (n_dec * n_heads * splits * 2,), torch.float32)
    lib = _lib("attention_bf16")
    if mask_chunk or softcap or sinks is not None:
        _launch(lib, lib.gb_attention_decode_bf16_by, _p(q), _rows(q, "q"), _p(out), _rows(out, "out"),
                1 if out.dtype == torch.float32 else 0, _p(ws_acc), _p(ws_ml), _p(ctx.positions), _p(tables), tables.stride(0),
                _p(k_pages), _p(v_pages), n_dec, n_heads, nkv, hd, page, float(scale), int(window), int(keep_first), mask_chunk,
                float(softcap), _p(_sinks(sinks, n_heads)), chunk, max_context, _stream())
        return
    if keep_first or out.dtype == torch.float32:
        _launch(lib, lib.gb_attention_decode_bf16_out32 if out.dtype == torch.float32 else lib.gb_attention_decode_bf16_keep, _p(q), _rows(q, "q"), _p(out), _rows(out, "out"), _p(ws_acc), _p(ws_ml),
                _p(ctx.positions), _p(tables), tables.stride(0), _p(k_pages), _p(v_pages), n_dec, n_heads, nkv, hd, page,
                float(scale), int(window), int(keep_first), chunk, max_context, _stream())
        return
    _launch(lib, lib.gb_attention_decode_bf16, _p(q), _rows(q, "q"), _p(out), _rows(out, "out"), _p(ws_acc), _p(ws_ml),
                                             _p(ctx.positions), _p(tables), tables.stride(0), _p(k_pages), _p(v_pages),
                                             n_dec, n_heads, nkv, hd, page, float(scale), int(window), chunk,
                                             max_context, _stream())


@functools.lru_cache(maxsize=4096)
def _prefill_parts(max_q: int, max_ctx: int, n_heads: int, n_seqs: int, hd: int) -> int:
    return int(_lib("attention_bf16").gb_attention_prefill_parts(max_q, max_ctx, n_heads, n_seqs, hd))


def attention_prefill(q: torch.Tensor, out: torch.Tensor, ctx, cache, n_heads: int, scale: float, window: int,
                      keep_first: int = 0, chunk: int = 0, softcap: float = 0.0, sinks: Optional[torch.Tensor] = None) -> None:
    """The requests of the step that bring more than one token (they follow the single-token ones)."""
    n_dec, S = ctx.host["n_decode"], ctx.num_seqs
    k_pages, v_pages = cache.k_pages, cache.v_pages
    _dev(q, out, k_pages, v_pages)
    _, nkv, page, hd = _check_pages(k_pages, v_pages, torch.bfloat16, "attention_prefill")
    if q.dtype != torch.bfloat16 or out.dtype not in (torch.bfloat16, torch.float32) or q.shape[1] != n_heads * hd:
        raise KernelError("attention_prefill: q must be bfloat16 [n, heads * head size], out bfloat16 or float32")
    tables = ctx.tables[cache.group]
    lib = _lib("attention_bf16")
    max_q, max_ctx = int(ctx.host["max_q_len"]), int(ctx.host["max_context"])
    # the portions' rows follow the single-token requests' rows; few and short portions over long contexts share
    # their keys among workgroups, which need room for their sums
    first_row, n_rows = n_dec, q.shape[0] - n_dec
    parts = _prefill_parts(max_q, max_ctx, n_heads, S - n_dec, hd)
    ws = ctx.buffer("attn_parts", (parts * n_rows * n_heads * (hd + 2),), torch.float32) if parts > 1 else None
    if chunk or softcap or sinks is not None:
        _launch(lib, lib.gb_attention_prefill_bf16_by, _p(q), _rows(q, "q"), _p(out), _rows(out, "out"),
                1 if out.dtype == torch.float32 else 0, _p(ctx.q_start), _p(ctx.q_len), _p(ctx.pos0), n_dec, S - n_dec, max_q,
                max_ctx, _p(tables), tables.stride(0), _p(k_pages), _p(v_pages), n_heads, nkv, hd, page, float(scale),
                int(window), int(keep_first), int(chunk), float(softcap), _p(_sinks(sinks, n_heads)), first_row, n_rows, _p(ws),
                ws.numel() if ws is not None else 0, _stream())
        return
    if keep_first or out.dtype == torch.float32:
        _launch(lib, lib.gb_attention_prefill_bf16_out32 if out.dtype == torch.float32 else lib.gb_attention_prefill_bf16_keep, _p(q), _rows(q, "q"), _p(out), _rows(out, "out"), _p(ctx.q_start),
                _p(ctx.q_len), _p(ctx.pos0), n_dec, S - n_dec, max_q, max_ctx, _p(tables), tables.stride(0), _p(k_pages),
                _p(v_pages), n_heads, nkv, hd, page, float(scale), int(window), int(keep_first), first_row, n_rows, _p(ws),
                ws.numel() if ws is not None else 0, _stream())
        return
    _launch(lib, lib.gb_attention_prefill_bf16, _p(q), _rows(q, "q"), _p(out), _rows(out, "out"), _p(ctx.q_start),
                                              _p(ctx.q_len), _p(ctx.pos0), n_dec, S - n_dec, max_q, max_ctx, _p(tables),
                                              tables.stride(0), _p(k_pages), _p(v_pages), n_heads, nkv, hd, page,
                                              float(scale), int(window), first_row, n_rows, _p(ws),
                                              ws.numel() if ws is not None else 0, _stream())


# ------------------------------------------------------------------------ sampling
def _logit_rows(logits: torch.Tensor):
    if logits.dtype != torch.float32 or logits.dim() != 2 or not logits.is_contiguous() or not logits.is_cuda:
        raise KernelError("sampling works on contiguous float32 logits [rows, vocab] on the GPU")
    return logits.shape


def argmax(logits: torch.Tensor, out: torch.Tensor) -> None:
    """out[r] = index of the first maximum of row r."""
    rows, vocab = _logit_rows(logits)
    _i32(out, "out", rows)
    lib = _lib("sampling")
    _launch(lib, lib.gb_argmax, _p(logits), _p(out), rows, vocab, _stream())


def penalize(logits: torch.Tensor, rows: torch.Tensor, tokens: torch.Tensor, counts: torch.Tensor,
             penalties: torch.Tensor) -> None:
    """In place, for every (row, token, count, penalty): count times v = v / pen if v > 0 else v * pen."""
    _, vocab = _logit_rows(logits)
    pairs = rows.numel()
    for t, what in ((rows, "rows"), (tokens, "tokens"), (counts, "counts")):
        _i32(t, what, pairs)
    if penalties.dtype != torch.float32 or penalties.numel() < pairs:
        raise KernelError("penalize: penalties must be float32, one per pair")
    lib = _lib("sampling")
    _launch(lib, lib.gb_penalize, _p(logits), vocab, _p(rows), _p(tokens), _p(counts), _p(penalties), pairs, _stream())


def sample(logits: torch.Tensor, temperature: torch.Tensor, top_k: torch.Tensor, top_p: torch.Tensor,
           min_p: torch.Tensor, uniform: torch.Tensor, out_token: torch.Tensor, out_candidates: torch.Tensor) -> None:
    """The reference's sampler per row: temperature, top-k, min-p, top-p, then an inverse-CDF draw in
    descending order of probability with the given uniform number; temperature <= 0 is greedy.  A row that is not
    greedy is left divided by its temperature."""
    rows, vocab = _logit_rows(logits)
    for t, what in ((temperature, "temperature"), (top_p, "top_p"), (min_p, "min_p"), (uniform, "uniform")):
        if t.dtype != torch.float32 or t.numel() < rows or not t.is_cuda:
            raise KernelError(f"sample: {what} must be float32 on the GPU, one per row")
    _i32(top_k, "top_k", rows)
    _i32(out_token, "out_token", rows)
    _i32(out_candidates, "out_candidates", rows)
    lib = _lib("sampling")
    _launch(lib, lib.gb_sample, _p(logits), rows, vocab, _p(temperature), _p(top_k), _p(top_p), _p(min_p), _p(uniform),
                              _p(out_token), _p(out_candidates), _stream())


# ------------------------------------------------------------------------ bounded norms, prepared heads, gates
def _vec32(t: Optional[torch.Tensor], n: int, what: str) -> None:
    if t is not None and (not t.is_cuda or t.dtype != torch.float32 or not t.is_contiguous() or t.numel() != n):
        raise KernelError(f"{what} must be contiguous float32 [{n}] on the GPU")


def tanh_norm(x: torch.Tensor, alpha: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor, out: torch.Tensor,
              rows: Optional[torch.Tensor] = None) -> None:
    """out[r] = tanh(alpha * x[rows[r] or r]) * weight + bias; x float32 [n, d], ``alpha`` one number on the device;
    ``out`` may be x itself."""
    _dev(x, out, rows)
    m, d = out.shape
    if x.dtype != torch.float32 or x.dim() != 2 or x.shape[1] != d or (rows is None and x.shape[0] < m):
        raise KernelError("tanh_norm: x must be float32 [n, d] with a row for every row of out")
    _vec32(alpha, 1, "tanh_norm: alpha")
    _vec32(weight, d, "tanh_norm: weight")
    _vec32(bias, d, "tanh_norm: bias")
    _i32(rows, "rows", m)
    lib = _lib("tanhmix")
    _launch(lib, lib.gb_tanh_norm, _p(x), _rows(x, "x"), _p(rows), _p(alpha), _p(weight), _p(bias), _p(out), dtype_code(out),
            _rows(out, "out"), m, d, _stream())


def tanh_norm_add(x: torch.Tensor, y: torch.Tensor, norm: tuple, slices: int = 1, then: Optional[tuple] = None,
                  h: Optional[torch.Tensor] = None) -> None:
    """x += tanh(alpha * y) * weight + bias with ``norm = (alpha, weight, bias)``; x float32 [n, d]; y float32 [n, d] or, with
    ``slices`` > 1, that many such pieces one behind the other, added up in their order first.  ``then = (alpha, weight,
    bias)`` with ``h`` [n, d]: h = tanh(alpha * x) * weight + bias of the new x, in h's type, in the same pass."""
    _dev(x, y, h)
    n, d = x.shape
    if x.dtype != torch.float32 or not x.is_contiguous() or y.dtype != torch.float32 or not y.is_contiguous() \
            or y.numel() < slices * n * d:
        raise KernelError("tanh_norm_add: x and y must be contiguous float32, y with a piece of x's size for every slice")
    for a, w, b in (norm,) + ((then,) if then is not None else ()):
        _vec32(a, 1, "tanh_norm_add: alpha")
        _vec32(w, d, "tanh_norm_add: weight")
        _vec32(b, d, "tanh_norm_add: bias")
    if (then is None) != (h is None) or (h is not None and (tuple(h.shape) != (n, d) or not h.is_contiguous())):
        raise KernelError("tanh_norm_add: the next norm and the rows it writes come together, rows contiguous [n, d]")
    a2, w2, b2 = then if then is not None else (None, None, None)
    lib = _lib("tanhmix")
    _launch(lib, lib.gb_tanh_norm_add, _p(x), _p(y), int(slices), n * d, _p(norm[0]), _p(norm[1]), _p(norm[2]), _p(a2), _p(w2),
            _p(b2), _p(h), dtype_code(h) if h is not None else F32, n, d, _stream())


def qk_heads(proj: torch.Tensor, ctx, out: torch.Tensor, head_cols: int, n_heads: int, n_kv_heads: int, dim: int, vdim: int,
             eps: float, joint: bool, norm_q: Optional[torch.Tensor], norm_k: Optional[torch.Tensor],
             bias: Optional[torch.Tensor] = None, wconv: Optional[torch.Tensor] = None, state: Optional[torch.Tensor] = None,
             cos: Optional[torch.Tensor] = None, sin: Optional[torch.Tensor] = None, rot: int = 0, magnitude: float = 1.0,
             neighbours: bool = True, tied: bool = False, slots: Optional[torch.Tensor] = None,
             k_pages: Optional[torch.Tensor] = None, v_pages: Optional[torch.Tensor] = None) -> None:
    """The query, key and value heads of every row of the step as attention reads them, ``out`` [n, (heads + 2 kv heads) *
    head_cols], from the stacked projections ``proj`` ([n, query channels | key channels | value channels | ...]; with
    ``tied`` there are no value channels: the key channels, biased and convolved, are the values):
    ``bias`` (float32, one a channel) is added; ``wconv`` ([taps, query + key channels] float32, a row a tap) convolves every query and
    key channel over the request's earlier rows and its ``state`` slot ([slots, taps - 1, channels] float32, moved on here
    in a step of single tokens, else by ``qk_conv_state``); an RMS norm over all query (key) channels at once with a weight a
    channel (``joint``) or over each head with ``dim`` weights that the heads share; the first ``rot`` channels of each
    head turned by the rows' angles (``cos``, ``sin`` float32 [n, rot / 2], times ``magnitude``), channel 2i with 2i + 1
    (``neighbours``) or i with i + rot / 2.  With ``slots`` keys and values also go to their pages."""
    _dev(proj, out, bias, wconv, state, cos, sin, slots, k_pages, v_pages, norm_q, norm_k)
    n = proj.shape[0]
    channels = (n_heads + n_kv_heads) * dim
    taps = 0
    if wconv is not None:
        taps = wconv.shape[0]
        _f32_rows(wconv, (taps, channels), "qk_heads: wconv")
        if taps > 1 and (state is None or state.dtype != torch.float32 or not state.is_contiguous()
                         or tuple(state.shape[1:]) != (taps - 1, channels)):
            raise KernelError(f"qk_heads: state must be contiguous float32 [slots, {taps - 1}, {channels}]")
    if proj.dtype != out.dtype or out.shape[0] != n or out.shape[1] != (n_heads + 2 * n_kv_heads) * head_cols:
        raise KernelError("qk_heads: out must be [n, (heads + 2 kv heads) * head_cols] of the projections' type")
    _vec32(bias, channels + (0 if tied else n_kv_heads * vdim), "qk_heads: bias")
    for w, size, what in ((norm_q, n_heads * dim if joint else dim, "norm_q"), (norm_k, n_kv_heads * dim if joint else dim, "norm_k")):
        _vec32(w, size, f"qk_heads: {what}")
    if rot:
        _f32_rows(cos, (n, rot // 2), "qk_heads: cos")
        _f32_rows(sin, (n, rot // 2), "qk_heads: sin")
    page = 0
    if slots is not None:
        _i32(slots, "slots", n)
        _, nkv, page, hd = _check_pages(k_pages, v_pages, proj.dtype, "qk_heads")
        if nkv != n_kv_heads or hd != head_cols:
            raise KernelError("qk_heads: the pages hold other heads than these")
    single = 1 if ctx.host["n_decode"] == ctx.num_seqs else 0
    # one norm over a whole row: the rows' squares are added up in a pass of their own, which every (token, head) then reads
    sums = ctx.buffer("qk_heads_sums", (n, 2), torch.float32) if joint else None
    lib = _lib("tanhmix")
    _launch(lib, lib.gb_qk_heads, _p(proj), dtype_code(proj), _rows(proj, "proj"), _p(bias), _p(wconv), _p(sums), _p(state),
            _p(ctx.tok_seq), _p(ctx.q_start), _p(ctx.pos0), _p(ctx.state_slots),
            single | (2 if joint else 0) | (4 if neighbours else 0) | (8 if tied else 0) | (int(taps) << 8), _p(norm_q), _p(norm_k),
            float(eps),
            _p(cos), _p(sin), int(rot), float(magnitude), _p(out), _rows(out, "out"), int(head_cols), _p(slots), _p(k_pages),
            _p(v_pages), int(page), n, n_heads, n_kv_heads, dim, vdim, _stream())
    if taps > 1 and not single:
        _launch(lib, lib.gb_qk_conv_state, _p(proj), dtype_code(proj), _rows(proj, "proj"), _p(bias), _p(state), _p(ctx.q_start),
                _p(ctx.q_len), _p(ctx.state_slots), ctx.num_seqs, channels, int(taps), _stream())


def gate_rows(att: torch.Tensor, head_cols: int, gate: torch.Tensor, out: torch.Tensor, n_heads: int, vdim: int,
              per_head: bool) -> None:
    """out[:, h, c] = att[:, h, c] * sigmoid(g) for c < vdim, g = gate[:, h] (``per_head``) or gate[:, h, c]: ``att`` [n, heads *
    head_cols], ``out`` [n, heads * vdim]; ``gate`` may be columns of a wider tensor."""
    _dev(att, gate, out)
    n = att.shape[0]
    if att.dtype != gate.dtype or att.dtype != out.dtype or att.shape[1] != n_heads * head_cols or out.shape != (n, n_heads * vdim) \
            or gate.shape != (n, n_heads if per_head else n_heads * vdim):
        raise KernelError("gate_rows: att [n, heads * head_cols], gate [n, heads (* vdim)] and out [n, heads * vdim] of one type")
    lib = _lib("tanhmix")
    _launch(lib, lib.gb_gate_rows, _p(att), _rows(att, "att"), int(head_cols), _p(gate), _rows(gate, "gate"), 1 if per_head else 0,
            dtype_code(att), _p(out), _rows(out, "out"), n, n_heads, vdim, _stream())
