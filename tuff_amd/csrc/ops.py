"""Python face of the HIP kernels: loads the compiled libraries with ctypes, checks every
operand on the host (device, dtype, contiguity, shape) and launches on torch's current stream.

There is no other implementation behind these functions: a missing library is compiled, a
library that cannot be compiled or a tensor that is not on the GPU is an error.
"""
from __future__ import annotations

import ctypes
import math
import os
from typing import Optional

import torch

from . import build

DT_F32, DT_BF16 = 0, 1
OUT_BF16, OUT_F32, OUT_F32_ACCUM, OUT_SWIGLU = 0, 1, 2, 3

_c_int, _c_float, _c_void_p, _c_ll = ctypes.c_int, ctypes.c_float, ctypes.c_void_p, ctypes.c_longlong


class KernelError(RuntimeError):
    pass


_SIGNATURES = {
    "elementwise": {
        "tuff_embed_rows": [_c_void_p, _c_int, _c_void_p, _c_void_p, _c_int, _c_int, _c_float, _c_void_p],
        "tuff_add_bias": [_c_void_p, _c_int, _c_void_p, _c_ll, _c_int, _c_void_p],
        "tuff_scale_cap": [_c_void_p, _c_ll, _c_float, _c_float, _c_void_p],
        "tuff_rmsnorm": [_c_void_p, _c_void_p, _c_int, _c_void_p, _c_int, _c_void_p, _c_int, _c_int, _c_float, _c_void_p],
        "tuff_swiglu": [_c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_void_p],
        "tuff_cast": [_c_void_p, _c_int, _c_void_p, _c_int, _c_ll, _c_void_p],
        "tuff_cast_bias": [_c_void_p, _c_void_p, _c_void_p, _c_int, _c_ll, _c_int, _c_void_p],
        "tuff_fill_u32": [_c_void_p, ctypes.c_uint32, _c_ll, _c_void_p],
        "tuff_scatter_i32": [_c_void_p, _c_int, _c_void_p, _c_int, _c_void_p, _c_int, _c_void_p],
        "tuff_dyt": [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_void_p, _c_int, _c_int, _c_void_p],
        "tuff_glu": [_c_void_p, _c_int, _c_void_p, _c_int, _c_int, _c_int, _c_int, _c_void_p, _c_float, _c_float, _c_void_p],
        "tuff_act_rows": [_c_void_p, _c_int, _c_void_p, _c_int, _c_ll, _c_int, _c_int, _c_void_p, _c_int, _c_int, _c_void_p, _c_void_p],
        "tuff_pad_cols": [_c_void_p, _c_void_p, _c_int, _c_ll, _c_int, _c_int, _c_void_p],
    },
    "recurrent": {
        "tuff_shift_mix": [_c_void_p, _c_int, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p,
                           _c_int, _c_int, _c_int, _c_void_p],
        "tuff_shift_state": [_c_void_p, _c_int, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_int, _c_void_p],
        "tuff_conv_act": [_c_void_p, _c_int, _c_ll, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_void_p, _c_void_p, _c_void_p,
                          _c_void_p, _c_int, _c_int, _c_int, _c_int, _c_int, _c_void_p],
        "tuff_wkv_scan": [_c_void_p, _c_void_p, _c_void_p, _c_int, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p,
                          _c_void_p, _c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_int, _c_void_p],
        "tuff_delta_scan": [_c_void_p, _c_void_p, _c_void_p, _c_int, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_ll,
                            _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_int, _c_int,
                            _c_int, _c_int, _c_int, _c_ll, _c_ll, _c_void_p],
        "tuff_head_norm_gate": [_c_void_p, _c_void_p, _c_int, _c_void_p, _c_ll, _c_int, _c_int, _c_int, _c_int, _c_void_p, _c_int, _c_int,
                                _c_int, _c_float, _c_void_p],
        "tuff_ssd_scan": [_c_void_p, _c_int, _c_ll, _c_void_p, _c_ll, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p,
                          _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_int, _c_int,
                          _c_int, _c_void_p],
        "tuff_ssd_chunked": [_c_void_p, _c_ll, _c_void_p, _c_ll, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p,
                             _c_void_p, _c_int, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_int,
                             _c_int, _c_int, _c_void_p],
        "tuff_forget_scan": [_c_void_p, _c_int, _c_ll, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p,
                             _c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_int, _c_int, _c_void_p],
    },
    "moe": {
        "tuff_moe_route": [_c_void_p, _c_int, _c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_int, _c_void_p],
        "tuff_moe_router": [_c_void_p, _c_int, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_int, _c_int,
                            _c_int, _c_void_p, _c_void_p, _c_int, _c_int, _c_float, _c_void_p],
        "tuff_moe_grouped_tile_rows": [_c_ll, _c_int],
        "tuff_moe_grouped_wide_from": [_c_int],
        "tuff_moe_grouped_tiled_from": [_c_int],
        "tuff_moe_experts_grouped": [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_void_p,
                                     _c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_float, _c_float, _c_void_p],
        "tuff_moe_experts": [_c_void_p, _c_void_p, _c_void_p, _c_int, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p,
                             _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_float, _c_float, _c_void_p],
    },
    "gemm_f32": {
        "tuff_gemm_f32": [_c_void_p, _c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_int, _c_void_p],
    },
    "gemm_bf16": {
        "tuff_gemm_bf16": [_c_void_p, _c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_int, _c_void_p, _c_void_p],
        "tuff_gemm_bf16_workspace": [_c_int, _c_int, _c_int, _c_int, ctypes.POINTER(_c_ll)],
        "tuff_gemm_bf16_emit_layout": [_c_int, _c_int, _c_int, ctypes.POINTER(_c_int), ctypes.POINTER(_c_int)],
        "tuff_gemm_bf16_scaled_supported": [_c_int, _c_int, _c_int],
        "tuff_gemm_bf16_accum_emit": [_c_void_p, _c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_void_p, _c_void_p,
                                      _c_void_p, _c_void_p, _c_void_p],
        "tuff_gemm_bf16_scaled": [_c_void_p, _c_void_p, _c_int, _c_float, _c_void_p, _c_void_p, _c_int, _c_int, _c_int,
                                  _c_int, _c_void_p, _c_void_p],
        "tuff_gemm_bf16_conv": [_c_void_p, _c_int, _c_void_p, _c_float, _c_void_p, _c_int, _c_void_p, _c_void_p, _c_int, _c_int,
                                _c_int, _c_void_p, _c_int, _c_int, _c_void_p, _c_void_p, _c_void_p],
        "tuff_gemm_bf16_conv64": [_c_void_p, _c_void_p, _c_int, _c_float, _c_void_p, _c_void_p, _c_int, _c_int, _c_int,
                                  _c_void_p, _c_int, _c_int, _c_void_p, _c_void_p, _c_void_p, _c_void_p],
        "tuff_gemm_bf16_normed": [_c_void_p, _c_void_p, _c_void_p, _c_float, _c_void_p, _c_void_p, _c_int, _c_int, _c_int,
                                  _c_int, _c_void_p],
    },
    "rope_kv": {
        "tuff_qkv_post": [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_int,
                          _c_void_p, _c_void_p, _c_int, _c_float,
                          _c_void_p, _c_int, _c_int, _c_void_p, _c_void_p,
                          _c_int, _c_int, _c_int, _c_int, _c_int, _c_void_p, _c_int, _c_int, _c_void_p],
        "tuff_rope_table": [_c_void_p, _c_int, _c_int, _c_void_p, _c_void_p],
        "tuff_kv_write": [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_void_p,
                          _c_int, _c_int, _c_int, _c_int, _c_int, _c_void_p],
    },
    "attention": {
        "tuff_attention_general": [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_void_p, _c_int,
                                   _c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int,
                                   _c_float, _c_void_p, _c_void_p, _c_int, _c_void_p, _c_void_p, _c_int, _c_void_p],
        "tuff_attention_decode_exact": [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_void_p, _c_void_p, _c_void_p,
                                        _c_void_p, _c_int, _c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int,
                                        _c_int, _c_float, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p,
                                        _c_int, _c_int, _c_void_p],
        "tuff_head_mix_gate": [_c_void_p, _c_int, _c_void_p, _c_void_p, _c_int, _c_void_p, _c_int, _c_int, _c_int, _c_int, _c_int,
                               _c_void_p],
    },
    "postnorm": {
        "tuff_post_norm_add": [_c_void_p, _c_void_p, _c_void_p, _c_float, _c_float, _c_void_p, _c_void_p, _c_float, _c_void_p,
                               _c_int, _c_int, _c_int, _c_int, _c_void_p, _c_void_p],
        "tuff_normed_mean2": [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_float, _c_float, _c_void_p, _c_int, _c_int, _c_void_p],
        "tuff_scale_add_layer_norm": [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_float, _c_void_p, _c_int, _c_void_p, _c_int, _c_int,
                                      _c_int, _c_void_p],
    },
    "hyper": {
        "tuff_hc_step": [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_void_p,
                         _c_int, _c_int, _c_int, _c_float, _c_int, _c_void_p],
    },
    "latent": {
        "tuff_latent_post": [_c_void_p, _c_int, _c_int, _c_int, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_int, _c_void_p, _c_int, _c_float,
                             _c_void_p, _c_int, _c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_int, _c_int, _c_void_p],
        "tuff_head_matmul": [_c_void_p, _c_ll, _c_ll, _c_void_p, _c_void_p, _c_ll, _c_ll, _c_void_p, _c_ll, _c_int,
                             _c_int, _c_int, _c_int, _c_int, _c_void_p],
        "tuff_head_matmul_mfma": [_c_void_p, _c_ll, _c_ll, _c_void_p, _c_void_p, _c_ll, _c_ll, _c_void_p, _c_ll,
                                  _c_int, _c_int, _c_int, _c_int, _c_void_p],
    },
    "attention_mfma": {
        "tuff_attention_mfma": [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_int,
                                _c_void_p, _c_int, _c_int, _c_void_p, _c_void_p,
                                _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_float, _c_int, _c_void_p],
        "tuff_attention_mfma_sinks": [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_int,
                                      _c_void_p, _c_int, _c_int, _c_void_p, _c_void_p,
                                      _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_float, _c_int, _c_void_p, _c_void_p],
        "tuff_attention_mfma_biased": [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_int,
                                       _c_void_p, _c_int, _c_int, _c_void_p, _c_void_p,
                                       _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_float, _c_int, _c_void_p, _c_void_p, _c_void_p],
        "tuff_attention_merge_sinks": [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int,
                                       _c_void_p, _c_void_p],
        "tuff_attention_merge": [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int,
                                 _c_void_p],
        "tuff_attention_decode_fused": [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_int,
                                        _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_float,
                                        _c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_float, _c_int,
                                        _c_void_p],
        "tuff_attention_mfma_static": [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_int,
                                       _c_void_p, _c_int, _c_int, _c_void_p, _c_void_p,
                                       _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_float, _c_int, _c_void_p],
    },
    "attention_prefill": {
        "tuff_attention_prefill": [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_void_p, _c_int,
                                   _c_void_p, _c_int, _c_int, _c_int, _c_int, _c_int, _c_float, _c_int, _c_int,
                                   _c_void_p, _c_void_p, _c_void_p],
        "tuff_attention_prefill_sinks": [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_void_p, _c_int,
                                         _c_void_p, _c_int, _c_int, _c_int, _c_int, _c_int, _c_float, _c_int, _c_int,
                                         _c_void_p, _c_void_p, _c_void_p, _c_void_p],
        "tuff_attention_prefill_biased": [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_void_p, _c_int,
                                          _c_void_p, _c_int, _c_int, _c_int, _c_int, _c_int, _c_float, _c_int, _c_int,
                                          _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p],
        "tuff_attention_prefill_wide": [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_void_p, _c_int,
                                        _c_void_p, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_float,
                                        _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_void_p],
        "tuff_attention_prefill_block_columns": [_c_int],
    },
    "shortconv": {
        "tuff_shortconv_fwd": [_c_void_p, _c_void_p, _c_int, _c_void_p, _c_void_p, _c_int, _c_void_p, _c_void_p,
                               _c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_void_p],
        "tuff_shortconv_decode": [_c_void_p, _c_void_p, _c_int, _c_void_p, _c_void_p, _c_int, _c_void_p,
                                  _c_int, _c_int, _c_int, _c_void_p],
        "tuff_shortconv_state": [_c_void_p, _c_int, _c_void_p, _c_void_p, _c_void_p, _c_void_p,
                                 _c_int, _c_int, _c_int, _c_void_p],
    },
    "sampling": {
        "tuff_argmax": [_c_void_p, _c_void_p, _c_int, _c_int, _c_void_p],
        "tuff_sample": [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p,
                        _c_int, _c_int, _c_void_p],
        "tuff_repeat_penalty": [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_void_p],
    },
}

_libs: dict[str, ctypes.CDLL] = {}

# TUFF_TRACE=1: GPU time by kernel class.  Every entry point of the kernel libraries is timed with a pair of
# events around its launches (an entry point is a class of kernels: the attention of single tokens is its
# partition kernel and its merge), and trace_report() prints calls, total, mean, least and most per class, in the
# manner of the reference's TUFF_TRACE report (src/cupti_profiler.cu:115-181, switched on at src/main.c:1787-1789).
# Events cannot be recorded into a graph, so an engine records no steps while this is on, and the step's time is
# that of its launches one by one.
TRACE = os.environ.get("TUFF_TRACE", "")[:1] == "1"
_trace_open: list = []                   # (class, start event, end event) not yet read
_trace_stats: dict = {}                  # class -> [calls, total ms, least ms, most ms]


def _trace_fold(everything: bool) -> None:
    """Reads the events that have completed (all of them after a synchronisation) into the statistics."""
    if everything:
        torch.cuda.synchronize()
    keep = []
    for name, a, b in _trace_open:
        if not everything and not b.query():
            keep.append((name, a, b))
            continue
        ms = a.elapsed_time(b)
        st = _trace_stats.setdefault(name, [0, 0.0, float("inf"), 0.0])
        st[0] += 1
        st[1] += ms
        st[2] = min(st[2], ms)
        st[3] = max(st[3], ms)
    _trace_open[:] = keep


def _traced(name: str, fn):
    def call(*args):
        if torch.cuda.is_current_stream_capturing():
            return fn(*args)
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        rc = fn(*args)
        b.record()
        _trace_open.append((name, a, b))
        if len(_trace_open) >= 4096:
            _trace_fold(False)
        return rc
    return call


def trace_reset() -> None:
    _trace_fold(True)
    _trace_stats.clear()


def trace_stats() -> dict:
    """{kernel class: (calls, total ms, least ms, most ms)} since the last trace_reset()."""
    _trace_fold(True)
    return {k: tuple(v) for k, v in _trace_stats.items()}


def trace_report(out) -> None:
    stats = sorted(trace_stats().items(), key=lambda kv: -kv[1][1])
    total = sum(v[1] for _, v in stats)
    line = "=" * 104
    print(f"\n{line}\n{'GPU TIME BY KERNEL CLASS (TUFF_TRACE)':^104}\n{line}", file=out)
    print(f"Total GPU time in kernel classes: {total:.3f} ms\n", file=out)
    print(f"{'Kernel class (entry point)':<44} | {'Calls':>7} | {'Total(ms)':>10} | {'Avg(us)':>9} | {'Min(us)':>9} | "
          f"{'Max(us)':>9} | {'GPU Time%':>9}", file=out)
    print("-" * 104, file=out)
    for name, (calls, ms, lo, hi) in stats:
        print(f"{name:<44} | {calls:>7} | {ms:>10.3f} | {1e3 * ms / calls:>9.2f} | {1e3 * lo:>9.2f} | {1e3 * hi:>9.2f} | "
              f"{100 * ms / total if total else 0:>8.1f}%", file=out)
    print(line, file=out)


def load(module: str) -> ctypes.CDLL:
    """The loaded library of a kernel module; compiled at first use if it is not built yet."""
    lib = _libs.get(module)
    if lib is None:
        path = build.ensure_built(module)
        lib = ctypes.CDLL(path)
        for name, argtypes in _SIGNATURES.get(module, {}).items():
            fn = getattr(lib, name)
            fn.argtypes = argtypes
            fn.restype = _c_int
            if TRACE and argtypes and argtypes[-1] is _c_void_p:        # (the last argument is the stream: it launches)
                setattr(lib, name, _traced(name, fn))
        _libs[module] = lib
    return lib


def loaded_modules() -> list[str]:
    return sorted(_libs)


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)
_get_device = getattr(torch._C, "_cuda_getDevice", None) or torch.cuda.current_device


def _stream() -> int:
    """Handle of torch's current stream on the current device (the stream a graph is being
    recorded on, inside a recording).  Called once a launch, so through the cheapest way there is."""
    if _raw_stream is not None:
        return _raw_stream(_get_device())
    return torch.cuda.current_stream().cuda_stream


def _dt(t: torch.Tensor) -> int:
    if t.dtype == torch.float32:
        return DT_F32
    if t.dtype == torch.bfloat16:
        return DT_BF16
    raise KernelError(f"unsupported element type {t.dtype}; kernels take float32 and bfloat16")


def _gpu(name: str, t: torch.Tensor, dtype=None, shape=None) -> int:
    if not isinstance(t, torch.Tensor):
        raise KernelError(f"{name}: expected a tensor, got {type(t).__name__}")
    if not t.is_cuda:
        raise KernelError(f"{name}: tensor is on '{t.device}'; the kernels run on the GPU only "
                          f"and there is no CPU fallback")
    if not t.is_contiguous():
        raise KernelError(f"{name}: tensor must be contiguous (shape {tuple(t.shape)}, stride {t.stride()})")
    if dtype is not None and t.dtype != dtype:
        raise KernelError(f"{name}: expected {dtype}, got {t.dtype}")
    if shape is not None and tuple(shape) != t.shape:        # torch.Size compares equal to a tuple
        if len(shape) != t.dim() or any(s is not None and s != g for s, g in zip(shape, t.shape)):
            raise KernelError(f"{name}: expected shape {tuple(shape)}, got {tuple(t.shape)}")
    return t.data_ptr()


def _opt(name, t, dtype=None, shape=None) -> Optional[int]:
    return None if t is None else _gpu(name, t, dtype, shape)


def _check(code: int, what: str) -> None:
    if code != 0:
        if code == -2:
            raise KernelError(f"{what}: the kernel refuses these sizes")
        if code == -7:
            raise KernelError(f"{what}: the step needs more work space than the library's static array holds")
        raise KernelError(f"{what}: launch failed with HIP error {code}")


# ------------------------------------------------------------------------ row kernels
def embed_rows(table: torch.Tensor, tokens: torch.Tensor, out: torch.Tensor, scale: float = 1.0) -> None:
    """out[t] = table[tokens[t]] * scale, float32."""
    n, d = out.shape
    _check(load("elementwise").tuff_embed_rows(
        _gpu("table", table, shape=(None, d)), _dt(table), _gpu("tokens", tokens, torch.int32, (n,)),
        _gpu("out", out, torch.float32), n, d, float(scale), _stream()), "embed_rows")


def add_bias(y: torch.Tensor, bias: torch.Tensor) -> None:
    """y[r, c] += bias[c] in place (y float32 or bfloat16 [rows, N], bias float32 [N])."""
    rows, N = y.shape
    _gpu("y", y)
    _gpu("bias", bias, torch.float32, (N,))
    _check(load("elementwise").tuff_add_bias(y.data_ptr(), _dt(y), bias.data_ptr(), rows, N, _stream()), "add_bias")


def scale_cap(x: torch.Tensor, scale: float = 1.0, cap: float = 0.0) -> None:
    """x <- x * scale, then, with cap > 0, x <- cap * tanh(x / cap); float32, in place."""
    _gpu("x", x, torch.float32)
    _check(load("elementwise").tuff_scale_cap(x.data_ptr(), x.numel(), float(scale), float(cap), _stream()), "scale_cap")


def rmsnorm(x: torch.Tensor, w: torch.Tensor, out: torch.Tensor, eps: float,
            rows: Optional[torch.Tensor] = None) -> None:
    n, d = out.shape
    if rows is None:
        _gpu("x", x, torch.float32, (n, d))
    else:
        _gpu("x", x, torch.float32, (None, d))
    _check(load("elementwise").tuff_rmsnorm(
        x.data_ptr(), _gpu("w", w, shape=(d,)), _dt(w), _gpu("out", out), _dt(out),
        _opt("rows", rows, torch.int32, (n,)), n, d, float(eps), _stream()), "rmsnorm")


def swiglu(gu: torch.Tensor, act: torch.Tensor) -> None:
    n, F = act.shape
    _check(load("elementwise").tuff_swiglu(
        _gpu("gu", gu, act.dtype, (n, 2 * F)), _gpu("act", act), _dt(act), n, F, _stream()), "swiglu")


def cast(inp: torch.Tensor, out: torch.Tensor, bias: Optional[torch.Tensor] = None) -> None:
    """out = inp in out's type.  bias (float32 [N], inp float32 [rows, N]): out = inp + bias, rounded once."""
    if inp.numel() != out.numel():
        raise KernelError(f"cast: {inp.numel()} elements in, {out.numel()} out")
    if bias is not None:
        N = inp.shape[-1]
        _check(load("elementwise").tuff_cast_bias(_gpu("inp", inp, torch.float32), _gpu("bias", bias, torch.float32, (N,)),
                                                  _gpu("out", out), _dt(out), inp.numel(), N, _stream()), "cast_bias")
        return
    _check(load("elementwise").tuff_cast(_gpu("inp", inp), _dt(inp), _gpu("out", out), _dt(out),
                                         inp.numel(), _stream()), "cast")


def fill_u32(t: torch.Tensor, value: int = 0) -> None:
    """Sets every 32-bit word of `t` to `value` (t must be a 4-byte type)."""
    if t.element_size() != 4:
        raise KernelError("fill_u32: tensor elements must be 4 bytes wide")
    if not t.is_cuda or not t.is_contiguous():
        raise KernelError("fill_u32: contiguous GPU tensor required")
    _check(load("elementwise").tuff_fill_u32(t.data_ptr(), value, t.numel(), _stream()), "fill_u32")


def scatter_i32(dst: torch.Tensor, src: torch.Tensor, idx: torch.Tensor) -> None:
    """dst[idx[i]] = src[idx[n + i]] for i < n = len(idx) / 2; all int32 on the GPU."""
    n = idx.shape[0] // 2
    _check(load("elementwise").tuff_scatter_i32(_gpu("dst", dst, torch.int32), dst.numel(), _gpu("src", src, torch.int32),
                                                src.numel(), _gpu("idx", idx, torch.int32, (2 * n,)), n, _stream()),
           "scatter_i32")


def dyt(x: torch.Tensor, w: torch.Tensor, b: torch.Tensor, alpha: torch.Tensor, out: torch.Tensor,
        rows: Optional[torch.Tensor] = None) -> None:
    """out = tanh(alpha * x[rows]) * w + b; x float32 [*, d], w and b float32 [d], alpha float32 [1]."""
    n, d = out.shape
    _gpu("x", x, torch.float32, (n if rows is None else None, d))
    _check(load("elementwise").tuff_dyt(
        x.data_ptr(), _gpu("w", w, torch.float32, (d,)), _gpu("b", b, torch.float32, (d,)),
        _gpu("alpha", alpha, torch.float32, (1,)), _gpu("out", out), _dt(out),
        _opt("rows", rows, torch.int32, (n,)), n, d, _stream()), "dyt")


ACTIVATIONS = {"silu": 0, "gelu_tanh": 1, "relu2": 2, "tanh": 3, "sigmoid": 4}
GLU_ACTIVATIONS = dict(ACTIVATIONS, swish_clamp=5)


def glu(gu: torch.Tensor, act: torch.Tensor, activation: str, bias: Optional[torch.Tensor] = None, *,
        limit: float = 0.0, alpha: float = 1.0) -> None:
    """act[t, f] = activation(gu[t, f] + bias[f]) * (gu[t, F + f] + bias[F + f]); gu of act's type or float32, bias
    float32 [2 F] or None.  activation "swish_clamp": g' sigmoid(alpha g') (u' + 1) with g' = min(g, limit),
    u' = clamp(u, -limit, limit)."""
    n, F = act.shape
    if activation == "swish_clamp" and not limit > 0:
        raise KernelError("glu: the clamped form needs a positive limit")
    _check(load("elementwise").tuff_glu(
        _gpu("gu", gu, shape=(n, 2 * F)), _dt(gu), _gpu("act", act), _dt(act), n, F, GLU_ACTIVATIONS[activation],
        _opt("bias", bias, torch.float32, (2 * F,)), float(limit), float(alpha), _stream()), "glu")


def act_rows(inp: torch.Tensor, out: torch.Tensor, activation: str, row_gate: Optional[torch.Tensor] = None,
             gate_col: int = 0, gate_activation: Optional[str] = None, bias: Optional[torch.Tensor] = None) -> None:
    """out = activation(inp [+ bias]), each row times gate_activation(row_gate[row, gate_col]) where row_gate
    (float32 [rows, *]) is given (gate_activation None: the number as it is).  bias: float32 [N], a number a column,
    added before the activation.  inp may be out."""
    rows, N = out.shape
    _gpu("inp", inp, shape=(rows, N))
    _gpu("out", out)
    gp, stride = None, 0
    if row_gate is not None:
        _gpu("row_gate", row_gate, torch.float32, (rows, None))
        if not 0 <= gate_col < row_gate.shape[1]:
            raise KernelError("act_rows: gate_col outside row_gate")
        gp, stride = row_gate.data_ptr() + 4 * gate_col, row_gate.shape[1]
    _check(load("elementwise").tuff_act_rows(
        inp.data_ptr(), _dt(inp), out.data_ptr(), _dt(out), rows, N, ACTIVATIONS[activation], gp, stride,
        -1 if gate_activation is None else ACTIVATIONS[gate_activation], _opt("bias", bias, torch.float32, (N,)), _stream()), "act_rows")


def pad_cols(inp: torch.Tensor, width: int) -> torch.Tensor:
    """inp [rows, N] widened to [rows, width] with zeros."""
    rows, N = inp.shape
    if width < N:
        raise KernelError("pad_cols: narrower than the input")
    out = torch.empty(rows, width, dtype=inp.dtype, device=inp.device)
    _check(load("elementwise").tuff_pad_cols(_gpu("inp", inp), out.data_ptr(), _dt(inp), rows, N, width, _stream()), "pad_cols")
    return out


# ------------------------------------------------------------------------------ GEMM
class TiledWeight:
    """A bfloat16 weight [N, K] in the order the matrix kernels stream it: blocks of 16 rows x 32 k,
    [ceil(N/16)][ceil(K/32)] of them, each 1 KB with piece l of 16 bytes = row l % 16,
    k 8 (l // 16) .. 8 (l // 16) + 7; rows and k beyond the matrix are zero."""

    def __init__(self, blocks: torch.Tensor, N: int, K: int):
        self.blocks, self.shape = blocks, (int(N), int(K))
        self.dtype, self.device = blocks.dtype, blocks.device

    def data_ptr(self) -> int:
        return self.blocks.data_ptr()

    def rows(self) -> torch.Tensor:
        """The weight back in row-major order [N, K] (a copy)."""
        N, K = self.shape
        t = self.blocks.view(-1, self.blocks.shape[1], 4, 16, 8).permute(0, 3, 1, 2, 4)
        return t.reshape(t.shape[0] * 16, -1)[:N, :K].contiguous()


def tile_weight(w: torch.Tensor) -> TiledWeight:
    """The tile-major copy of a row-major bfloat16 weight [N, K].  Made once when a weight is bound."""
    if w.dim() != 2 or w.dtype != torch.bfloat16:
        raise KernelError(f"tile_weight: a bfloat16 matrix is needed, got {w.dtype} {tuple(w.shape)}")
    N, K = w.shape
    Np, Kp = -(-N // 16) * 16, -(-K // 32) * 32
    if (Np, Kp) != (N, K):
        padded = torch.zeros(Np, Kp, dtype=w.dtype, device=w.device)
        padded[:N, :K] = w
        w = padded
    blocks = w.view(Np // 16, 16, Kp // 32, 4, 8).permute(0, 2, 3, 1, 4).contiguous()
    return TiledWeight(blocks.view(Np // 16, Kp // 32, 64, 8), N, K)


def _tiled(w, N: int, K: int) -> TiledWeight:
    """w as the bfloat16 kernels take it.  A plain tensor is converted on the spot (tests and single
    calls; the parts bind tiled weights)."""
    if not isinstance(w, TiledWeight):
        _gpu("w", w, torch.bfloat16, (N, K))
        w = tile_weight(w)
    if not w.blocks.is_cuda or not w.blocks.is_contiguous() or w.shape != (N, K):
        raise KernelError(f"w: a tiled weight {(N, K)} on the GPU is needed, got {w.shape} on {w.device}")
    return w


def _bf16_mode(out: torch.Tensor, accumulate: bool, swiglu: bool, M: int, N: int) -> int:
    if swiglu:
        if accumulate or out.dtype != torch.bfloat16 or N % 2:
            raise KernelError("gemm: the SwiGLU epilogue writes bfloat16 [M, N/2] and cannot accumulate")
        _gpu("out", out, shape=(M, N // 2))
        return OUT_SWIGLU
    _gpu("out", out, shape=(M, N))
    if out.dtype == torch.float32:
        return OUT_F32_ACCUM if accumulate else OUT_F32
    if out.dtype == torch.bfloat16:
        if accumulate:
            raise KernelError("gemm: accumulation needs a float32 output")
        return OUT_BF16
    raise KernelError(f"gemm: unsupported output type {out.dtype}")


def gemm(x: torch.Tensor, w: torch.Tensor, out: torch.Tensor, accumulate: bool = False,
         swiglu: bool = False) -> None:
    """out (=|+=) x @ w.T.  x [M, K], w [N, K] of one dtype; float32 operands give the true
    float32 product, bfloat16 operands the matrix-core product with float32 accumulation.
    `out` is float32 (stored or accumulated into) or, for bfloat16 operands, bfloat16.
    swiglu (bfloat16 only): the rows of w are gate and up rows interleaved and out [M, N/2] is
    silu(gate) * up."""
    M, K = x.shape
    N = w.shape[0]
    _gpu("x", x)
    if x.dtype == torch.float32:
        if isinstance(w, TiledWeight):
            raise KernelError("gemm: float32 activations with a tiled bfloat16 weight")
        _gpu("w", w, x.dtype, (N, K))
        if out.dtype != torch.float32 or swiglu:
            raise KernelError("gemm: float32 operands need a float32 output and have no fused epilogue")
        _gpu("out", out, shape=(M, N))
        _check(load("gemm_f32").tuff_gemm_f32(x.data_ptr(), w.data_ptr(), out.data_ptr(), M, N, K,
                                              int(accumulate), _stream()), "gemm_f32")
        return
    if x.dtype != torch.bfloat16:
        raise KernelError(f"gemm: unsupported operand type {x.dtype}")
    if K % 8 != 0:
        raise KernelError(f"gemm: the bfloat16 kernels need an inner size that is a multiple of 8, got {K}")
    w = _tiled(w, N, K)
    mode = _bf16_mode(out, accumulate, swiglu, M, N)
    ws = _gemm_workspace(M, N, K, x.device)
    _check(load("gemm_bf16").tuff_gemm_bf16(x.data_ptr(), w.data_ptr(), out.data_ptr(), M, N, K, mode,
                                            None if ws is None else ws.data_ptr(), _stream()), "gemm_bf16")


NORMED_MAX_ROWS, NORMED_MAX_K = 16, 8192      # gemm_normed: the norm inside the product's kernel
EMIT_MAX_ROWS = 64                            # gemm_accum_emit / gemm_scaled: the skinny products; beyond, the tiled one


def gemm_normed(x: torch.Tensor, norm_w: torch.Tensor, eps: float, w: torch.Tensor, out: torch.Tensor, *,
                rows: Optional[torch.Tensor] = None, accumulate: bool = False, swiglu: bool = False) -> None:
    """out (=|+=) rmsnorm(x[rows]) @ w.T in one kernel, for at most 16 rows: x float32 [*, K],
    norm_w float32 [K], w bfloat16 [N, K].  The row's 1/rms scales the result, the norm weight
    the operand."""
    K = x.shape[1]
    M = x.shape[0] if rows is None else rows.shape[0]
    N = w.shape[0]
    _gpu("x", x, torch.float32)
    _gpu("norm_w", norm_w, torch.float32, (K,))
    w = _tiled(w, N, K)
    _opt("rows", rows, torch.int32, (M,))
    if M > NORMED_MAX_ROWS or K > NORMED_MAX_K or K % 8:
        raise KernelError(f"gemm_normed: at most {NORMED_MAX_ROWS} rows and an inner size that is a multiple of 8 "
                          f"up to {NORMED_MAX_K}; got {M} rows, inner size {K}")
    mode = _bf16_mode(out, accumulate, swiglu, M, N)
    _check(load("gemm_bf16").tuff_gemm_bf16_normed(
        x.data_ptr(), None if rows is None else rows.data_ptr(), norm_w.data_ptr(), float(eps), w.data_ptr(),
        out.data_ptr(), M, N, K, mode, _stream()), "gemm_bf16_normed")


_emit_layouts: dict = {}


def gemm_emit_layout(M: int, N: int, K: int) -> Optional[tuple]:
    """(tiles, rows): shape of the sums of squares gemm_accum_emit leaves for a product of M rows
    with N outputs and inner size K, or None where such a product cannot leave them (more than 64 rows
    and an inner size that is no multiple of 64, a product cut along K, a last block of columns that is
    not whole)."""
    key = (M if M > 16 else 0, N, K)                   # (which kernel takes 17 to 64 rows depends on all three)
    if key not in _emit_layouts:
        t, r = _c_int(0), _c_int(0)
        _check(load("gemm_bf16").tuff_gemm_bf16_emit_layout(M, N, K, ctypes.byref(t), ctypes.byref(r)), "gemm_emit_layout")
        _emit_layouts[key] = (int(t.value), int(r.value)) if t.value > 0 else None
    return _emit_layouts[key]


def gemm_accum_emit(x: torch.Tensor, w, residual: torch.Tensor, next_norm_w: torch.Tensor,
                    xw: torch.Tensor, ss: torch.Tensor) -> None:
    """residual += x @ w.T, and for the RMSNorm that follows: xw = the new residual times next_norm_w as
    bfloat16, ss [gemm_emit_layout(M, N, K)] = per-tile sums of squares of each row."""
    M, K = x.shape
    N = w.shape[0]
    _gpu("x", x, torch.bfloat16)
    w = _tiled(w, N, K)
    _gpu("residual", residual, torch.float32, (M, N))
    _gpu("next_norm_w", next_norm_w, torch.float32, (N,))
    _gpu("xw", xw, torch.bfloat16, (M, N))
    layout = gemm_emit_layout(M, N, K) if K % 8 == 0 else None
    if layout is None:
        raise KernelError(f"gemm_accum_emit: a product of {M} rows, {N} outputs and inner size {K} cannot leave the next "
                          f"norm's operand (ask gemm_emit_layout first)")
    _gpu("ss", ss, torch.float32, layout)
    ws = _gemm_workspace(M, N, K, x.device, emit=True)
    _check(load("gemm_bf16").tuff_gemm_bf16_accum_emit(x.data_ptr(), w.data_ptr(), residual.data_ptr(), M, N, K,
                                                       next_norm_w.data_ptr(), xw.data_ptr(), ss.data_ptr(),
                                                       None if ws is None else ws.data_ptr(), _stream()),
           "gemm_bf16_accum_emit")


_scaled_ok: dict = {}


def gemm_scaled_supported(M: int, N: int, K: int, out_dtype=torch.bfloat16, accumulate: bool = False) -> bool:
    """Whether gemm_scaled takes this product: any with at most 64 rows; with more, bfloat16 (or SwiGLU)
    outputs of products that run in one piece."""
    if K % 8:
        return False
    if M <= EMIT_MAX_ROWS:
        return True
    if accumulate or out_dtype != torch.bfloat16:
        return False
    key = (M, N, K)
    if key not in _scaled_ok:
        _scaled_ok[key] = bool(load("gemm_bf16").tuff_gemm_bf16_scaled_supported(M, N, K))
    return _scaled_ok[key]


def gemm_scaled(xw: torch.Tensor, ss: torch.Tensor, eps: float, w, out: torch.Tensor, *,
                accumulate: bool = False, swiglu: bool = False) -> None:
    """out (=|+=) rmsnorm(x) @ w.T from what gemm_accum_emit left for the same number of rows:
    xw = bf16(x * norm weight) and the per-tile sums of squares ss; each row of the product is
    scaled by 1 / sqrt(sum(ss) / K + eps)."""
    M, K = xw.shape
    N = w.shape[0]
    _gpu("xw", xw, torch.bfloat16)
    if not gemm_scaled_supported(M, N, K, out.dtype, accumulate):
        raise KernelError(f"gemm_scaled: a product of {M} rows, {N} outputs, inner size {K} into {out.dtype} is not "
                          f"supported (ask gemm_scaled_supported first)")
    _gpu("ss", ss, torch.float32, (None, 16 if M <= 16 else 64 if M <= EMIT_MAX_ROWS else M))
    w = _tiled(w, N, K)
    mode = _bf16_mode(out, accumulate, swiglu, M, N)
    ws = _gemm_workspace(M, N, K, xw.device)
    _check(load("gemm_bf16").tuff_gemm_bf16_scaled(xw.data_ptr(), ss.data_ptr(), ss.shape[0], float(eps), w.data_ptr(),
                                                   out.data_ptr(), M, N, K, mode,
                                                   None if ws is None else ws.data_ptr(), _stream()), "gemm_bf16_scaled")


CONV_MAX_ROWS = 32                            # gemm_conv: one token a row (the norm inside: at most NORMED_MAX_ROWS)


def conv_group_rows(w_in: torch.Tensor) -> torch.Tensor:
    """The input projection [3 d, K] of a gated short convolution (rows: B, then C, then X) with its
    rows regrouped for gemm_conv: sixteen channels a group, each group as [its B rows | its C rows |
    its X rows].  d must be a multiple of 16."""
    three_d, K = w_in.shape
    d = three_d // 3
    if three_d != 3 * d or d % 16:
        raise KernelError(f"conv_group_rows: [3 d, K] with d a multiple of 16 is needed, got {tuple(w_in.shape)}")
    return w_in.view(3, d // 16, 16, K).permute(1, 0, 2, 3).reshape(three_d, K).contiguous()


def gemm_conv(x: torch.Tensor, w, out: torch.Tensor, *, conv_w: torch.Tensor, state: torch.Tensor, state_slot: torch.Tensor,
              norm_w: Optional[torch.Tensor] = None, eps: float = 0.0, ss: Optional[torch.Tensor] = None) -> None:
    """Input projection and gated short convolution of single tokens (row r is request r's token, at
    most 32 rows) in one kernel: out [M, d] bfloat16 = C * conv(B * X) with (B, C, X) = x @ w.T, and
    the rows' states shifted.  w: conv_group_rows() of the projection, tiled.  x: bfloat16 [M, K]; or
    the float32 residual stream with norm_w and eps (the RMSNorm runs inside); or bf16(x * norm weight)
    with ss and eps as gemm_accum_emit leaves them."""
    M, K = x.shape
    d = out.shape[1]
    taps = conv_w.shape[1]
    _gpu("out", out, torch.bfloat16, (M, d))
    w = _tiled(w, 3 * d, K)
    _gpu("conv_w", conv_w, shape=(d, taps))
    _gpu("state", state, torch.float32, (None, taps - 1, d))
    _gpu("state_slot", state_slot, torch.int32, (M,))
    if M > CONV_MAX_ROWS or K % 8 or d % 16 or not 2 <= taps <= 17:
        raise KernelError(f"gemm_conv: at most {CONV_MAX_ROWS} rows, an inner size that is a multiple of 8, a width that is a "
                          f"multiple of 16 and 2 to 17 taps; got {M} rows, inner size {K}, width {d}, {taps} taps")
    kind, nw_ptr, ss_ptr, n_ss = 0, None, None, 0
    if ss is not None:
        _gpu("x", x, torch.bfloat16)
        _gpu("ss", ss, torch.float32, (None, 16 if M <= 16 else 64))
        kind, ss_ptr, n_ss = 2, ss.data_ptr(), ss.shape[0]
    elif norm_w is not None:
        _gpu("x", x, torch.float32)
        _gpu("norm_w", norm_w, torch.float32, (K,))
        if K > NORMED_MAX_K or M > NORMED_MAX_ROWS:
            raise KernelError(f"gemm_conv: the norm inside needs an inner size up to {NORMED_MAX_K} and at most "
                              f"{NORMED_MAX_ROWS} rows, got {K} and {M}")
        kind, nw_ptr = 1, norm_w.data_ptr()
    else:
        _gpu("x", x, torch.bfloat16)
    _check(load("gemm_bf16").tuff_gemm_bf16_conv(
        x.data_ptr(), kind, nw_ptr, float(eps), ss_ptr, n_ss, w.data_ptr(), out.data_ptr(), M, d, K,
        conv_w.data_ptr(), _dt(conv_w), taps, state.data_ptr(), state_slot.data_ptr(), _stream()), "gemm_bf16_conv")


CONV64_MAX_ROWS = 64                          # gemm_conv64: one token a row


def gemm_conv64(x: torch.Tensor, w, out: torch.Tensor, *, conv_w: torch.Tensor, state: torch.Tensor, state_slot: torch.Tensor,
                eps: float = 0.0, ss: Optional[torch.Tensor] = None) -> None:
    """gemm_conv for 33 to 64 rows, in two kernels (the projection's partial tiles; the kernel that adds
    them and runs the convolution), without the projected rows ever being written.  w: the projection
    [3 d, K] as the checkpoint has it (B | C | X), tiled.  x: bfloat16 [M, K], or bf16(x * norm weight)
    with ss [tiles][64] and eps as gemm_accum_emit leaves them for these rows."""
    M, K = x.shape
    d = out.shape[1]
    taps = conv_w.shape[1]
    _gpu("x", x, torch.bfloat16)
    _gpu("out", out, torch.bfloat16, (M, d))
    w = _tiled(w, 3 * d, K)
    _gpu("conv_w", conv_w, shape=(d, taps))
    _gpu("state", state, torch.float32, (None, taps - 1, d))
    _gpu("state_slot", state_slot, torch.int32, (M,))
    if not CONV_MAX_ROWS < M <= CONV64_MAX_ROWS or K % 8 or d % 16 or not 2 <= taps <= 17:
        raise KernelError(f"gemm_conv64: {CONV_MAX_ROWS + 1} to {CONV64_MAX_ROWS} rows, an inner size that is a multiple of 8, a width that is "
                          f"a multiple of 16 and 2 to 17 taps; got {M} rows, inner size {K}, width {d}, {taps} taps")
    ss_ptr, n_ss = None, 0
    if ss is not None:
        _gpu("ss", ss, torch.float32, (None, 64))
        ss_ptr, n_ss = ss.data_ptr(), ss.shape[0]
    ws = _gemm_workspace(M, 3 * d, K, x.device, emit=True)
    _check(load("gemm_bf16").tuff_gemm_bf16_conv64(
        x.data_ptr(), ss_ptr, n_ss, float(eps), w.data_ptr(), out.data_ptr(), M, d, K,
        conv_w.data_ptr(), _dt(conv_w), taps, state.data_ptr(), state_slot.data_ptr(), ws.data_ptr(), _stream()), "gemm_bf16_conv64")


_plans: dict = {}


def _gemm_workspace(M: int, N: int, K: int, device, emit: bool = False) -> Optional[torch.Tensor]:
    """The float32 work space a bfloat16 product of this shape needs, or None.  Taken anew for every
    call: the allocator hands the same block out again."""
    if M <= 16:
        return None
    key = (M, N, K, emit)
    n = _plans.get(key)
    if n is None:
        a = _c_ll(0)
        load("gemm_bf16").tuff_gemm_bf16_workspace(M, N, K, int(emit), ctypes.byref(a))
        n = _plans[key] = int(a.value)
    return torch.empty(n, dtype=torch.float32, device=device) if n else None


# ----------------------------------------------------------------- q/k/v post-processing
def qkv_post(qkv, q_out, *, H, Hkv, hd, positions, eps=0.0, q_norm_w=None, k_norm_w=None,
             inv_freq=None, rotary_dim=0, interleaved=False, k_out=None,
             k_cache=None, v_cache=None, slot_mapping=None, page_size=1, angles=None, wide_rows: bool = False) -> None:
    """wide_rows: a row of qkv holds more than (H + 2 Hkv) hd elements or fewer (values of another width behind the
    keys); then only q_out and k_out are written (no cache)."""
    T = qkv.shape[0]
    dt = qkv.dtype
    if wide_rows:
        _gpu("qkv", qkv, shape=(T, None))
        if qkv.shape[1] < (H + Hkv) * hd or k_cache is not None:
            raise KernelError("qkv_post: wide rows hold at least the q and k heads and go with no cache write")
    else:
        _gpu("qkv", qkv, shape=(T, (H + 2 * Hkv) * hd))
    _gpu("q_out", q_out, dt, (T, H * hd))
    _opt("k_out", k_out, dt, (T, Hkv * hd))
    if (k_cache is None) != (v_cache is None):
        raise KernelError("qkv_post: k_cache and v_cache go together")
    if k_cache is not None:
        if slot_mapping is None:
            raise KernelError("qkv_post: a cache write needs slot_mapping")
        P = k_cache.shape[0]
        _gpu("k_cache", k_cache, dt, (P, Hkv, page_size, hd))
        _gpu("v_cache", v_cache, dt, (P, Hkv, hd, page_size))
        _gpu("slot_mapping", slot_mapping, torch.int32, (T,))
    norm_dt = DT_F32
    if q_norm_w is not None or k_norm_w is not None:
        if q_norm_w is None or k_norm_w is None or q_norm_w.dtype != k_norm_w.dtype:
            raise KernelError("qkv_post: q and k norm weights go together and share a dtype")
        _gpu("q_norm_w", q_norm_w, shape=(hd,))
        _gpu("k_norm_w", k_norm_w, shape=(hd,))
        norm_dt = _dt(q_norm_w)
    if inv_freq is not None:
        if rotary_dim <= 0 or rotary_dim > hd or rotary_dim % 2:
            raise KernelError(f"qkv_post: rotary_dim {rotary_dim} must be even and within the head size {hd}")
        _gpu("inv_freq", inv_freq, torch.float32, (rotary_dim // 2,))
        _opt("angles", angles, torch.float32, (None, 2, rotary_dim // 2))      # rope_table(inv_freq, n)
    _gpu("positions", positions, torch.int32, (T,))
    if hd > 256:
        raise KernelError(f"qkv_post: head size {hd} above 256 is not supported")
    p = lambda t: None if t is None else t.data_ptr()
    _check(load("rope_kv").tuff_qkv_post(
        qkv.data_ptr(), q_out.data_ptr(), p(k_out), p(k_cache), p(v_cache), _dt(qkv),
        p(q_norm_w), p(k_norm_w), norm_dt, float(eps), p(inv_freq), int(rotary_dim), int(interleaved),
        positions.data_ptr(), p(slot_mapping), T, H, Hkv, hd, page_size,
        p(angles) if inv_freq is not None else None, 0 if angles is None else angles.shape[0],
        qkv.shape[1] if wide_rows else 0, _stream()), "qkv_post")


def rope_table(inv_freq: torch.Tensor, n_pos: int) -> torch.Tensor:
    """float32 [n_pos, 2, len(inv_freq)]: cosines and sines of pos * inv_freq, bit for bit what the
    rotation kernels compute for themselves."""
    n_freq = inv_freq.shape[0]
    _gpu("inv_freq", inv_freq, torch.float32, (n_freq,))
    out = torch.empty(int(n_pos), 2, n_freq, dtype=torch.float32, device=inv_freq.device)
    _check(load("rope_kv").tuff_rope_table(inv_freq.data_ptr(), n_freq, int(n_pos), out.data_ptr(), _stream()), "rope_table")
    return out


def kv_write(k, v, k_cache, v_cache, slot_mapping, *, Hkv, hd, page_size, vd=None) -> None:
    """Rows of keys [T, Hkv * hd] and values [T, Hkv * vd] (vd: hd unless given) into the paged cache."""
    T = k.shape[0]
    dt = k.dtype
    vd = hd if vd is None else int(vd)
    _gpu("k", k, shape=(T, Hkv * hd))
    _gpu("v", v, dt, (T, Hkv * vd))
    P = k_cache.shape[0]
    _gpu("k_cache", k_cache, dt, (P, Hkv, page_size, hd))
    _gpu("v_cache", v_cache, dt, (P, Hkv, vd, page_size))
    _gpu("slot_mapping", slot_mapping, torch.int32, (T,))
    _check(load("rope_kv").tuff_kv_write(k.data_ptr(), v.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(),
                                         _dt(k), slot_mapping.data_ptr(), T, Hkv, hd, vd, page_size, _stream()),
           "kv_write")


# -------------------------------------------------------------------------- attention
def attention_general(q, k_cache, v_cache, out, *, block_table, req_of_token, positions,
                      H, Hkv, hd, page_size, window=0, scale=None, vd=None, sinks=None, slopes=None,
                      log_distance=None, all_values: bool = False) -> None:
    """vd: width of a value where it is not the keys'.  sinks: float32 [H], a logit per head that counts
    once in the softmax's denominator and has no value.  slopes: float32 [H]; slopes[h] * (position - key) is
    taken off head h's scaled scores.  v_cache None: the values are the first vd channels of the key rows.
    log_distance: (r1, r2), float32 [H] each; r1[h] * ln(1 + r2[h] * (position - key)) is taken off head h's scaled
    scores.  all_values: every query head's weights are applied to the values of every kv head; out is then float32
    [T, H * Hkv * vd] (head, kv head, channel), for head_mix_gate."""
    T = q.shape[0]
    dt = q.dtype
    vd = hd if vd is None else int(vd)
    _gpu("q", q, shape=(T, H * hd))
    if all_values:
        if v_cache is None:
            raise KernelError("attention: all_values needs a value cache")
        _gpu("out", out, torch.float32, (T, H * Hkv * vd))
    else:
        _gpu("out", out, dt, (T, H * vd))
    r1 = r2 = None
    if log_distance is not None:
        r1, r2 = log_distance
        _gpu("log_distance r1", r1, torch.float32, (H,))
        _gpu("log_distance r2", r2, torch.float32, (H,))
    P = k_cache.shape[0]
    _gpu("k_cache", k_cache, dt, (P, Hkv, page_size, hd))
    if v_cache is None:
        if vd > hd:
            raise KernelError("attention: values inside the key rows cannot be wider than the keys")
    else:
        _gpu("v_cache", v_cache, dt, (P, Hkv, vd, page_size))
    _opt("sinks", sinks, torch.float32, (H,))
    _opt("slopes", slopes, torch.float32, (H,))
    _gpu("block_table", block_table, torch.int32)
    if block_table.dim() != 2:
        raise KernelError("attention: block_table must be [requests, blocks]")
    _gpu("req_of_token", req_of_token, torch.int32, (T,))
    _gpu("positions", positions, torch.int32, (T,))
    if hd > ATTN_GENERAL_MAX_DIM or vd > ATTN_GENERAL_MAX_DIM or H % Hkv:
        raise KernelError(f"attention: head size {hd} (values {vd}) / heads {H}:{Hkv} not supported")
    if scale is None:
        scale = 1.0 / math.sqrt(hd)
    _check(load("attention").tuff_attention_general(
        q.data_ptr(), k_cache.data_ptr(), None if v_cache is None else v_cache.data_ptr(), out.data_ptr(), _dt(q),
        block_table.data_ptr(), block_table.shape[1], req_of_token.data_ptr(), positions.data_ptr(),
        T, H, Hkv, hd, vd, page_size, int(window or 0), float(scale), None if sinks is None else sinks.data_ptr(),
        None if slopes is None else slopes.data_ptr(), int(v_cache is None),
        None if r1 is None else r1.data_ptr(), None if r2 is None else r2.data_ptr(), int(all_values), _stream()), "attention_general")


def head_mix_gate(o, out, *, H, Hkv, vd, talk=None, gates=None) -> None:
    """After attention: out[t, h] = sigmoid(gates[t, h]) * o[t, h] (o [T, H * vd]), or, with talk float32 [H, H] and
    o float32 [T, H * Hkv * vd] as attention_general(all_values=True) leaves it,
    out[t, h] = sigmoid(gates[t, h]) * sum_g talk[h, g] o[t, g, kv head of h].  gates float32 [T, >= H] (rows of one
    stride; the first H columns count) or None for no gate; out [T, H * vd] of the compute type."""
    T = out.shape[0]
    _gpu("out", out, shape=(T, H * vd))
    if talk is not None:
        _gpu("talk", talk, torch.float32, (H, H))
        _gpu("o", o, torch.float32, (T, H * Hkv * vd))
    else:
        _gpu("o", o, shape=(T, H * vd))
    stride = 0
    if gates is not None:
        if not gates.is_cuda or gates.dtype != torch.float32 or gates.dim() != 2 or gates.shape[0] != T or gates.shape[1] < H \
                or gates.stride(1) != 1:
            raise KernelError(f"head_mix_gate: gates must be float32 [{T}, >= {H}] on the GPU, got {tuple(gates.shape)} {gates.dtype}")
        stride = gates.stride(0)
    _check(load("attention").tuff_head_mix_gate(
        o.data_ptr(), _dt(o), None if talk is None else talk.data_ptr(), None if gates is None else gates.data_ptr(), stride,
        out.data_ptr(), _dt(out), T, H, Hkv, vd, _stream()), "head_mix_gate")


# ------------------------------------------------- sublayers normed before they join the stream
def post_norm_add(x, *, y=None, w=None, eps: float = 0.0, mult: float = 1.0, extra=None, next_w=None, next_eps: float = 0.0,
                  h_out=None, clear_y: bool = False, y_next=None) -> None:
    """One kernel over the residual stream x (float32 [T, d], in place).  With y float32 [T, d] and w float32 [d]:
    x <- x + mult * y / sqrt(mean(y^2) + eps) * w (y is then cleared, if asked).  With extra float32 [T, d]:
    x <- x + extra.  With next_w float32 [d] and h_out [T, d]: h_out = x / sqrt(mean(x^2) + next_eps) * next_w,
    from the new x.  y_next float32 [d] (with clear_y): every row of y is left holding y_next instead of zeros, the bias of
    the product that adds into y next."""
    T, d = x.shape
    _opt("y_next", y_next, torch.float32, (d,))
    _gpu("x", x, torch.float32, (T, d))
    _opt("y", y, torch.float32, (T, d))
    if y is not None:
        _gpu("w", w, torch.float32, (d,))
    _opt("extra", extra, torch.float32, (T, d))
    if (next_w is None) != (h_out is None):
        raise KernelError("post_norm_add: next_w and h_out go together")
    if next_w is not None:
        _gpu("next_w", next_w, torch.float32, (d,))
        _gpu("h_out", h_out, shape=(T, d))
    _check(load("postnorm").tuff_post_norm_add(
        x.data_ptr(), None if y is None else y.data_ptr(), None if y is None else w.data_ptr(), float(eps), float(mult),
        None if extra is None else extra.data_ptr(), None if next_w is None else next_w.data_ptr(), float(next_eps),
        None if h_out is None else h_out.data_ptr(), DT_F32 if h_out is None else _dt(h_out), T, d, int(clear_y),
        None if y_next is None else y_next.data_ptr(), _stream()),
        "post_norm_add")


def scale_add_layer_norm(x, *, y=None, ls=None, next_w=None, eps: float = 0.0, h_out=None, rows=None, clear_y: bool = False) -> None:
    """One kernel over the residual stream x (float32 [T, d], in place).  With y float32 [T, d] and ls float32 [d]:
    x <- x + ls * y (y is then cleared, if asked).  With next_w float32 [d] and h_out: h_out = (x - mean) /
    sqrt(mean((x - mean)^2) + eps) * next_w from the new x, a layer norm with a weight and no bias.  rows (int32 [n],
    only without y): h_out [n, d] holds the norm of those rows of x, in that order."""
    T, d = x.shape
    _gpu("x", x, torch.float32, (T, d))
    if (y is None) != (ls is None):
        raise KernelError("scale_add_layer_norm: y and ls go together")
    if (next_w is None) != (h_out is None):
        raise KernelError("scale_add_layer_norm: next_w and h_out go together")
    if rows is not None and y is not None:
        raise KernelError("scale_add_layer_norm: chosen rows go with the norm alone")
    _opt("y", y, torch.float32, (T, d))
    _opt("ls", ls, torch.float32, (d,))
    n = T if rows is None else rows.shape[0]
    _opt("rows", rows, torch.int32, (n,))
    if next_w is not None:
        _gpu("next_w", next_w, torch.float32, (d,))
        _gpu("h_out", h_out, shape=(n, d))
    p = lambda t: None if t is None else t.data_ptr()
    _check(load("postnorm").tuff_scale_add_layer_norm(
        x.data_ptr(), p(y), p(ls), p(next_w), float(eps), p(h_out), DT_F32 if h_out is None else _dt(h_out), p(rows), n, d,
        int(bool(clear_y)), _stream()), "scale_add_layer_norm")


def normed_mean2(a, wa, b, wb, out, *, eps: float, coef: float = 0.5) -> None:
    """out <- out + coef * (a / sqrt(mean(a^2) + eps) * wa + b / sqrt(mean(b^2) + eps) * wb); a, b, out float32
    [T, d]; wa, wb float32 [d]."""
    T, d = a.shape
    _check(load("postnorm").tuff_normed_mean2(
        _gpu("a", a, torch.float32, (T, d)), _gpu("wa", wa, torch.float32, (d,)), _gpu("b", b, torch.float32, (T, d)),
        _gpu("wb", wb, torch.float32, (d,)), float(eps), float(coef), _gpu("out", out, torch.float32, (T, d)), T, d, _stream()),
        "normed_mean2")


ATTN_GENERAL_MAX_DIM = 640   # widest key or value row of the general attention kernel


# ------------------------------------------------------------- several residual streams
HC_MAX_STREAMS, HC_MAX_DIM = 8, 15360


def hc_step(xs, *, y=None, mix=None, out_w=None, in_w=None, norm_w=None, eps: float = 0.0, h_out=None, u_out=None,
            clear_y: bool = False) -> None:
    """One kernel over the residual streams xs (float32 [S, T, d], in place).  With y [T, d], mix [S, S] (indexed
    [from, to]) and out_w [S]: xs[r] <- sum_s mix[s, r] xs[s] + out_w[r] y.  Then, with in_w [S]: u = sum_s in_w[s]
    xs[s] (of the new values); with norm_w (float32 [d]) h_out [T, d] = u / sqrt(mean(u^2) + eps) * norm_w in h_out's
    type, without it u_out [T, d] = u in float32.  clear_y: y is zero afterwards (ready for the next sublayer to add into)."""
    S, T, d = xs.shape
    _gpu("xs", xs, torch.float32)
    if S > HC_MAX_STREAMS or d > HC_MAX_DIM:
        raise KernelError(f"hc_step: at most {HC_MAX_STREAMS} streams of at most {HC_MAX_DIM} channels")
    if (y is None) != (mix is None) or (y is None) != (out_w is None):
        raise KernelError("hc_step: y, mix and out_w go together")
    _opt("y", y, torch.float32, (T, d))
    _opt("mix", mix, torch.float32, (S, S))
    _opt("out_w", out_w, torch.float32, (S,))
    _opt("in_w", in_w, torch.float32, (S,))
    _opt("norm_w", norm_w, torch.float32, (d,))
    if in_w is not None:
        if norm_w is not None:
            _gpu("h_out", h_out, shape=(T, d))
        else:
            _gpu("u_out", u_out, torch.float32, (T, d))
    p = lambda t: None if t is None else t.data_ptr()
    _check(load("hyper").tuff_hc_step(xs.data_ptr(), p(y), p(mix), p(out_w), p(in_w), p(norm_w), p(h_out),
                                      DT_F32 if h_out is None else _dt(h_out), p(u_out), S, T, d, float(eps), int(bool(clear_y)), _stream()), "hc_step")


# ------------------------------------------------------------------- latent attention
def latent_post(proj, q_lat, cache, *, q_off: int, ckr_off: int, norm_w, eps: float, inv_freq, rot_dims: int, positions,
                slot_mapping, H: int, dim: int, rot: int, rank: int, cache_t=None) -> None:
    """From a token's projected row proj[t] (queries [H, dim + rot] from column q_off; the latent's raw channels
    [rank] and the shared key part [rot] from column ckr_off): the cache row [norm(c) * norm_w | rotate(k)] at
    slot_mapping[t] (cache [pages, 1, page size, rank + rot]; slot_mapping None: no write) and the rotated query
    parts into q_lat[t, h, rank:] (q_lat [T, H * (rank + rot)]).  Rotation of neighbouring pairs of the first rot_dims
    channels by position * inv_freq (float32 [rot_dims / 2]).  cache_t ([pages, 1, rank + rot, page size], optional):
    the same rows once more with a channel's positions contiguous within the page."""
    T = proj.shape[0]
    dt = proj.dtype
    lat = rank + rot
    _gpu("proj", proj, shape=(T, None))
    if q_off + H * (dim + rot) > proj.shape[1] or ckr_off + lat > proj.shape[1] or min(q_off, ckr_off) < 0:
        raise KernelError("latent_post: the columns lie outside the projected row")
    _gpu("q_lat", q_lat, dt, (T, H * lat))
    if cache.dim() != 4 or cache.shape[1] != 1 or cache.shape[3] != lat:
        raise KernelError(f"latent_post: the cache must be [pages, 1, page size, {lat}], got {tuple(cache.shape)}")
    _gpu("cache", cache, dt)
    _opt("cache_t", cache_t, dt, (cache.shape[0], 1, lat, cache.shape[2]))
    _gpu("norm_w", norm_w, shape=(rank,))
    if rot_dims % 2 or not 0 <= rot_dims <= rot:
        raise KernelError(f"latent_post: {rot_dims} rotated channels of {rot}")
    if rot_dims:
        _gpu("inv_freq", inv_freq, torch.float32, (rot_dims // 2,))
    _gpu("positions", positions, torch.int32, (T,))
    _opt("slot_mapping", slot_mapping, torch.int32, (T,))
    _check(load("latent").tuff_latent_post(
        proj.data_ptr(), proj.shape[1], int(q_off), int(ckr_off), q_lat.data_ptr(), cache.data_ptr(),
        None if cache_t is None else cache_t.data_ptr(), cache.shape[2], _dt(proj),
        norm_w.data_ptr(), _dt(norm_w), float(eps), inv_freq.data_ptr() if rot_dims else None, int(rot_dims),
        positions.data_ptr(), None if slot_mapping is None else slot_mapping.data_ptr(), T, H, dim, rot, rank, _stream()),
        "latent_post")


HEAD_MATMUL_MAX_K = 2048


HEAD_MATMUL_MFMA_MAX_K = 512


def head_matmul_mfma_supported(dtype, K: int, x_width: int, x_col: int, x_head: int) -> bool:
    """Whether the matrix-core form takes these operands: bfloat16, an inner size that is a multiple of 8 up to 512,
    every head's row of x on a 16-byte border."""
    return (dtype == torch.bfloat16 and K % 8 == 0 and 8 <= K <= HEAD_MATMUL_MFMA_MAX_K
            and x_width % 8 == 0 and x_col % 8 == 0 and x_head % 8 == 0)


def head_matmul(x, w, y, *, H: int, x_col: int = 0, x_head: int, y_col: int = 0, y_head: int, gate=None, gate_col: int = 0,
                w_nk=None) -> None:
    """y[t, y_col + h * y_head + n] = sum_k x[t, x_col + h * x_head + k] * w[h, k, n], n < N, k < K, for w [H, K, N];
    with gate ([T, *], its column gate_col + h the head's) times sigmoid(gate).  x, w, y, gate of one type; rows of x, y
    and gate may be wider than what is read or written.  w_nk: the same weights as [H, N, K]; where it is given and
    head_matmul_mfma_supported() holds the product runs on the matrix cores (w may then be None)."""
    if w_nk is not None and head_matmul_mfma_supported(x.dtype, w_nk.shape[2], x.shape[1], x_col, x_head):
        T = x.shape[0]
        Hw, N, K = w_nk.shape
        _gpu("x", x, torch.bfloat16, (T, None))
        _gpu("w_nk", w_nk, torch.bfloat16)
        _gpu("y", y, torch.bfloat16, (T, None))
        if Hw != H:
            raise KernelError(f"head_matmul: w_nk is {tuple(w_nk.shape)} for {H} heads")
        if x_col + (H - 1) * x_head + K > x.shape[1] or y_col + (H - 1) * y_head + N > y.shape[1] or min(x_col, y_col) < 0:
            raise KernelError("head_matmul: the heads' columns lie outside a row")
        if x_head < 0 or (y_head < N and H > 1):
            raise KernelError("head_matmul: the heads' outputs overlap")
        gp = None
        if gate is not None:
            _gpu("gate", gate, torch.bfloat16, (T, None))
            if gate_col < 0 or gate_col + H > gate.shape[1]:
                raise KernelError("head_matmul: the gates' columns lie outside a row")
            gp = gate.data_ptr() + gate_col * 2
        _check(load("latent").tuff_head_matmul_mfma(
            x.data_ptr() + x_col * 2, x.shape[1], int(x_head), w_nk.data_ptr(), y.data_ptr() + y_col * 2, y.shape[1], int(y_head),
            gp, 0 if gate is None else gate.shape[1], T, H, K, N, _stream()), "head_matmul_mfma")
        return
    if w is None:
        raise KernelError("head_matmul: these operands need the weights as [H, K, N]")
    T = x.shape[0]
    dt = x.dtype
    Hw, K, N = w.shape
    _gpu("x", x, shape=(T, None))
    _gpu("w", w, dt)
    _gpu("y", y, dt, (T, None))
    if Hw != H or K > HEAD_MATMUL_MAX_K:
        raise KernelError(f"head_matmul: w is {tuple(w.shape)} for {H} heads (inner size at most {HEAD_MATMUL_MAX_K})")
    if x_col + (H - 1) * x_head + K > x.shape[1] or y_col + (H - 1) * y_head + N > y.shape[1] or min(x_col, y_col) < 0:
        raise KernelError("head_matmul: the heads' columns lie outside a row")
    if x_head < 0 or (y_head < N and H > 1):
        raise KernelError("head_matmul: the heads' outputs overlap")
    gp = None
    if gate is not None:
        _gpu("gate", gate, dt, (T, None))
        if gate_col < 0 or gate_col + H > gate.shape[1]:
            raise KernelError("head_matmul: the gates' columns lie outside a row")
        gp = gate.data_ptr() + gate_col * gate.element_size()
    es = x.element_size()
    _check(load("latent").tuff_head_matmul(
        x.data_ptr() + x_col * es, x.shape[1], int(x_head), w.data_ptr(), y.data_ptr() + y_col * es, y.shape[1], int(y_head),
        gp, 0 if gate is None else gate.shape[1], _dt(x), T, H, K, N, _stream()), "head_matmul")


ATTN_PARTITION = 256        # keys a partition of the matrix-core attention kernel covers


def attention_mfma_supported(dtype, hd: int, page_size: int) -> bool:
    return dtype == torch.bfloat16 and hd % 8 == 0 and hd <= 256 and page_size % 16 == 0


def attention_mfma(q, k_cache, v_cache, out, *, block_table, blocks, nb, req_info, positions,
                   H, Hkv, hd, page_size, max_ctx_len, window=0, scale=None, sinks=None, slopes=None) -> None:
    """Matrix-core attention over the paged bfloat16 cache.  blocks: int32 [n_blocks, 2] from
    query_blocks(), or None when every request's columns fit one block (block b = request b).
    req_info: int32 [R, 4] = (first token in the step, tokens, first position, -) per request.
    max_ctx_len bounds every position + 1 of the step.  sinks: float32 [H] or None, a logit per head that
    counts once in the softmax's denominator and has no value.  slopes: float32 [H] or None; slopes[h] * (position - key)
    is taken off head h's scaled scores."""
    T = q.shape[0]
    _opt("sinks", sinks, torch.float32, (H,))
    _opt("slopes", slopes, torch.float32, (H,))
    if not attention_mfma_supported(q.dtype, hd, page_size):
        raise KernelError(f"attention_mfma: needs bfloat16, a head size that is a multiple of 8 (got {hd}) "
                          f"and a page size that is a multiple of 16 (got {page_size})")
    _gpu("q", q, torch.bfloat16, (T, H * hd))
    _gpu("out", out, torch.bfloat16, (T, H * hd))
    P = k_cache.shape[0]
    _gpu("k_cache", k_cache, torch.bfloat16, (P, Hkv, page_size, hd))
    _gpu("v_cache", v_cache, torch.bfloat16, (P, Hkv, hd, page_size))
    _gpu("block_table", block_table, torch.int32)
    R = req_info.shape[0]
    _gpu("req_info", req_info, torch.int32, (R, 4))
    if block_table.dim() != 2 or block_table.shape[0] != R:
        raise KernelError("attention_mfma: block_table must be [requests, blocks]")
    n_parts = max(1, -(-int(max_ctx_len) // ATTN_PARTITION))
    if block_table.shape[1] * page_size < int(max_ctx_len):
        raise KernelError("attention_mfma: block_table is narrower than the longest context")
    G = H // Hkv
    if blocks is None:
        if G > 16 * nb:
            raise KernelError("attention_mfma: without a block list a request's columns must fit one block")
        nblk = R
    else:
        nblk = blocks.shape[0]
        _gpu("blocks", blocks, torch.int32, (nblk, 2))
    _gpu("positions", positions, torch.int32, (T,))
    if nb not in (1, 2, 4) or (hd > 128 and nb == 4) or H % Hkv:
        raise KernelError(f"attention_mfma: unsupported column blocking nb={nb} for head size {hd}")
    if scale is None:
        scale = 1.0 / math.sqrt(hd)
    ws_o = torch.empty(T * H * n_parts * hd, dtype=torch.float32, device=q.device)
    ws_ml = torch.empty(T * H * n_parts * 2, dtype=torch.float32, device=q.device)
    args = (q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), out.data_ptr(), ws_o.data_ptr(), ws_ml.data_ptr(),
            block_table.data_ptr(), block_table.shape[1], None if blocks is None else blocks.data_ptr(), nblk, nb,
            req_info.data_ptr(), positions.data_ptr(), T, H, Hkv, hd, page_size, int(window or 0), float(scale), n_parts)
    if slopes is not None:
        _check(load("attention_mfma").tuff_attention_mfma_biased(*args, None if sinks is None else sinks.data_ptr(), slopes.data_ptr(),
                                                                 _stream()), "attention_mfma")
    elif sinks is None:
        _check(load("attention_mfma").tuff_attention_mfma(*args, _stream()), "attention_mfma")
    else:
        _check(load("attention_mfma").tuff_attention_mfma_sinks(*args, sinks.data_ptr(), _stream()), "attention_mfma")


def attention_decode_fused_supported(dtype, H: int, Hkv: int, hd: int, page_size: int, rotary_dim: int, interleaved: bool) -> bool:
    """A step of single tokens can go from the projected q/k/v rows to the attention output in one
    kernel and its merge: bfloat16, heads of 64 rotated whole in half-split pairs, at most sixteen
    query heads a kv head."""
    return (dtype == torch.bfloat16 and hd == 64 and rotary_dim == 64 and not interleaved and page_size % 16 == 0
            and H % Hkv == 0 and H // Hkv <= 16)


def attention_decode_fused(qkv, k_cache, v_cache, out, *, block_table, req_info, positions, inv_freq, H, Hkv, page_size,
                           max_ctx_len, slot_mapping=None, q_norm_w=None, k_norm_w=None, eps=0.0, window=0, scale=None,
                           angles=None) -> None:
    """Attention of a step in which every request has one token (row r of qkv is request r's), from the
    projected rows qkv [R, (H + 2 Hkv) * 64]: QK-norm, rotation, the write of the new key and value
    into the cache (slot_mapping; None: the cache is only read), attention over the cache, merge.
    angles: rope_table(inv_freq, n) or None; positions below n take their cosines and sines from it
    (computing them costs the kernel more than everything else it does for a short context)."""
    R = qkv.shape[0]
    hd = 64
    _gpu("qkv", qkv, torch.bfloat16, (R, (H + 2 * Hkv) * hd))
    _gpu("out", out, torch.bfloat16, (R, H * hd))
    P = k_cache.shape[0]
    _gpu("k_cache", k_cache, torch.bfloat16, (P, Hkv, page_size, hd))
    _gpu("v_cache", v_cache, torch.bfloat16, (P, Hkv, hd, page_size))
    _gpu("block_table", block_table, torch.int32)
    _gpu("req_info", req_info, torch.int32, (R, 4))
    _gpu("positions", positions, torch.int32, (R,))
    _opt("slot_mapping", slot_mapping, torch.int32, (R,))
    _gpu("inv_freq", inv_freq, torch.float32, (hd // 2,))
    _opt("angles", angles, torch.float32, (None, 2, hd // 2))
    if block_table.dim() != 2 or block_table.shape[0] != R:
        raise KernelError("attention_decode_fused: block_table must be [requests, blocks]")
    if block_table.shape[1] * page_size < int(max_ctx_len):
        raise KernelError("attention_decode_fused: block_table is narrower than the longest context")
    if not attention_decode_fused_supported(qkv.dtype, H, Hkv, hd, page_size, hd, False):
        raise KernelError(f"attention_decode_fused: heads {H}:{Hkv} / page size {page_size} not supported")
    norm_dt = DT_F32
    if q_norm_w is not None or k_norm_w is not None:
        if q_norm_w is None or k_norm_w is None or q_norm_w.dtype != k_norm_w.dtype:
            raise KernelError("attention_decode_fused: q and k norm weights go together and share a dtype")
        _gpu("q_norm_w", q_norm_w, shape=(hd,))
        _gpu("k_norm_w", k_norm_w, shape=(hd,))
        norm_dt = _dt(q_norm_w)
    n_parts = max(1, -(-int(max_ctx_len) // ATTN_PARTITION))
    if scale is None:
        scale = 1.0 / math.sqrt(hd)
    ws_o = torch.empty(R * H * n_parts * hd, dtype=torch.float32, device=qkv.device)
    ws_ml = torch.empty(R * H * n_parts * 2, dtype=torch.float32, device=qkv.device)
    p = lambda t: None if t is None else t.data_ptr()
    _check(load("attention_mfma").tuff_attention_decode_fused(
        qkv.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), out.data_ptr(), ws_o.data_ptr(), ws_ml.data_ptr(),
        block_table.data_ptr(), block_table.shape[1], req_info.data_ptr(), positions.data_ptr(), p(slot_mapping),
        p(q_norm_w), p(k_norm_w), norm_dt, float(eps), inv_freq.data_ptr(), p(angles),
        0 if angles is None else angles.shape[0], R, H, Hkv, page_size,
        int(window or 0), float(scale), n_parts, _stream()), "attention_decode_fused")


def attention_prefill_block_columns(hd: int) -> int:
    """Columns (token, head in the kv group) a query block of attention_prefill holds."""
    return 128


PREFILL_WORKGROUP_SLOTS = 512    # workgroups of attention_prefill the part runs side by side (two a CU); with at most
                                 # half as many blocks the keys are cut into segments, a workgroup a segment
PREFILL_MIN_SEGMENT = 1024       # keys; shorter segments are not worth their merge


def attention_prefill(q, k_cache, v_cache, out, *, block_table, blocks, req_info,
                      H, Hkv, hd, page_size, max_ctx_len, window=0, scale=None, positions=None, sinks=None, slopes=None) -> None:
    """Matrix-core attention for steps with prompt portions: a workgroup walks over all keys of a
    block of query columns, keys and values staged through LDS; writes `out` directly.
    blocks: int32 [n_blocks, 2] from query_blocks(q_len, G, attention_prefill_block_columns(hd) // 16),
    or None when every request's columns fit one block (block b = request b).
    positions (int32 [T], optional): with them, a step with few blocks and long contexts (a short
    portion far into a long prompt) cuts the keys into segments, a workgroup a segment, and merges the
    segments' results as a step of single tokens merges its partitions.  Then every row of `out` is
    written, also those of tokens no block covers (with meaningless values)."""
    T = q.shape[0]
    _opt("sinks", sinks, torch.float32, (H,))      # a logit per head that counts once in the denominator and has no value
    _opt("slopes", slopes, torch.float32, (H,))    # slopes[h] * (position - key) is taken off head h's scaled scores
    if not attention_mfma_supported(q.dtype, hd, page_size):
        raise KernelError(f"attention_prefill: needs bfloat16, a head size that is a multiple of 8 (got {hd}) "
                          f"and a page size that is a multiple of 16 (got {page_size})")
    _gpu("q", q, torch.bfloat16, (T, H * hd))
    _gpu("out", out, torch.bfloat16, (T, H * hd))
    P = k_cache.shape[0]
    _gpu("k_cache", k_cache, torch.bfloat16, (P, Hkv, page_size, hd))
    _gpu("v_cache", v_cache, torch.bfloat16, (P, Hkv, hd, page_size))
    _gpu("block_table", block_table, torch.int32)
    R = req_info.shape[0]
    _gpu("req_info", req_info, torch.int32, (R, 4))
    if block_table.dim() != 2 or block_table.shape[0] != R:
        raise KernelError("attention_prefill: block_table must be [requests, blocks]")
    if block_table.shape[1] * page_size < int(max_ctx_len):
        raise KernelError("attention_prefill: block_table is narrower than the longest context")
    if H % Hkv:
        raise KernelError("attention_prefill: the query heads must be a multiple of the kv heads")
    G = H // Hkv
    if blocks is None:
        if G > attention_prefill_block_columns(hd):
            raise KernelError("attention_prefill: without a block list a request's columns must fit one block")
        nblk = R
    else:
        nblk = blocks.shape[0]
        _gpu("blocks", blocks, torch.int32, (nblk, 2))
    if scale is None:
        scale = 1.0 / math.sqrt(hd)
    n_segs, seg_keys, ws_o, ws_ml = 1, 0, None, None
    workgroups = nblk * Hkv
    if positions is not None and 0 < 2 * workgroups <= PREFILL_WORKGROUP_SLOTS and int(max_ctx_len) >= 2 * PREFILL_MIN_SEGMENT:
        # as many segments as fill the slots once, not more: what does not fit waits for a second round
        want = min(PREFILL_WORKGROUP_SLOTS // workgroups, int(max_ctx_len) // PREFILL_MIN_SEGMENT, 64)
        seg_keys = -(-(-(-int(max_ctx_len) // want)) // 64) * 64
        n_segs = -(-int(max_ctx_len) // seg_keys)
    if n_segs > 1:
        _gpu("positions", positions, torch.int32, (T,))
        ws_o = torch.empty(T * H * n_segs * hd, dtype=torch.float32, device=q.device)
        ws_ml = torch.empty(T * H * n_segs * 2, dtype=torch.float32, device=q.device)
    else:
        n_segs, seg_keys = 1, 0
    args = (q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), out.data_ptr(),
            block_table.data_ptr(), block_table.shape[1], None if blocks is None else blocks.data_ptr(), nblk,
            req_info.data_ptr(), H, Hkv, hd, page_size, int(window or 0), float(scale), n_segs, seg_keys,
            None if ws_o is None else ws_o.data_ptr(), None if ws_ml is None else ws_ml.data_ptr())
    merge = (ws_o.data_ptr(), ws_ml.data_ptr(), out.data_ptr(), positions.data_ptr(), T, H, hd, int(window or 0), n_segs,
             seg_keys) if n_segs > 1 else None
    if slopes is not None:
        _check(load("attention_prefill").tuff_attention_prefill_biased(*args, None if sinks is None else sinks.data_ptr(),
                                                                       slopes.data_ptr(), _stream()), "attention_prefill")
        if merge is not None and sinks is None:
            _check(load("attention_mfma").tuff_attention_merge(*merge, _stream()), "attention_merge")
        elif merge is not None:
            _check(load("attention_mfma").tuff_attention_merge_sinks(*merge, sinks.data_ptr(), _stream()), "attention_merge")
    elif sinks is None:
        _check(load("attention_prefill").tuff_attention_prefill(*args, _stream()), "attention_prefill")
        if merge is not None:
            _check(load("attention_mfma").tuff_attention_merge(*merge, _stream()), "attention_merge")
    else:
        _check(load("attention_prefill").tuff_attention_prefill_sinks(*args, sinks.data_ptr(), _stream()), "attention_prefill")
        if merge is not None:
            _check(load("attention_mfma").tuff_attention_merge_sinks(*merge, sinks.data_ptr(), _stream()), "attention_merge")


DECODE_EXACT_KEYS = 256          # keys a part of attention_decode_exact


def attention_decode_exact_supported(dtype, H: int, hd: int, vd: int, page_size: int) -> bool:
    return (dtype == torch.bfloat16 and H <= 256 and hd % 8 == 0 and hd <= 256 and 1 <= vd <= DECODE_EXACT_KEYS
            and page_size % 8 == 0 and DECODE_EXACT_KEYS % page_size == 0)


def attention_decode_exact(q, k_cache, v_cache, out, *, block_table, req_of_token, positions, H, Hkv, hd, vd, page_size,
                           max_ctx_len, window=0, scale=None, sinks=None, slopes=None, log_distance=None, talk=None,
                           gates=None) -> None:
    """Single tokens over the bfloat16 cache with float32 softmax weights: the scores of parts of 256 keys (a key's row
    read once for all heads of its kv group), then the normalised weights on the values (read once too), then the sum over
    the parts.  log_distance = (r1, r2): r1[h] * ln(1 + r2[h] * (position - key)) is taken off the scaled scores.
    talk float32 [H, H]: head h's weights are sum_g talk[h, g] weights_g, on the values of h's own kv head.
    gates float32 [T, >= H] (a row may be wider): out[t, h] is multiplied by sigmoid(gates[t, h]).
    out [T, H * vd], bfloat16 or float32."""
    T = q.shape[0]
    if not attention_decode_exact_supported(q.dtype, H, hd, vd, page_size):
        raise KernelError(f"attention_decode_exact: bfloat16, heads {H} <= 256, key size {hd} a multiple of 8, "
                          f"value size {vd} <= 256, page size {page_size} a divisor of 256")
    _gpu("q", q, torch.bfloat16, (T, H * hd))
    _gpu("out", out, shape=(T, H * vd))
    P = k_cache.shape[0]
    _gpu("k_cache", k_cache, torch.bfloat16, (P, Hkv, page_size, hd))
    _gpu("v_cache", v_cache, torch.bfloat16, (P, Hkv, vd, page_size))
    _opt("sinks", sinks, torch.float32, (H,))
    _opt("slopes", slopes, torch.float32, (H,))
    _opt("talk", talk, torch.float32, (H, H))
    r1 = r2 = None
    if log_distance is not None:
        r1, r2 = log_distance
        _gpu("log_distance r1", r1, torch.float32, (H,))
        _gpu("log_distance r2", r2, torch.float32, (H,))
    gate_stride = 0
    if gates is not None:
        _gpu("gates", gates, torch.float32)
        if gates.dim() != 2 or gates.shape[0] != T or gates.shape[1] < H or gates.stride(1) != 1:
            raise KernelError("attention_decode_exact: gates must be float32 [tokens, >= heads]")
        gate_stride = gates.stride(0)
    _gpu("block_table", block_table, torch.int32)
    if block_table.dim() != 2 or block_table.shape[1] * page_size < int(max_ctx_len):
        raise KernelError("attention_decode_exact: block_table must be [requests, blocks] and cover the longest context")
    _gpu("req_of_token", req_of_token, torch.int32, (T,))
    _gpu("positions", positions, torch.int32, (T,))
    if H % Hkv:
        raise KernelError("attention_decode_exact: the query heads must be a multiple of the kv heads")
    if scale is None:
        scale = 1.0 / math.sqrt(hd)
    n_parts = max(1, -(-int(max_ctx_len) // DECODE_EXACT_KEYS))
    S = torch.empty(T * H * n_parts * DECODE_EXACT_KEYS, dtype=torch.float32, device=q.device)
    ml = torch.empty(T * H * n_parts * 2, dtype=torch.float32, device=q.device)
    po = torch.empty(T * H * n_parts * vd, dtype=torch.float32, device=q.device)
    ptr = lambda x: None if x is None else x.data_ptr()
    _check(load("attention").tuff_attention_decode_exact(
        q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), out.data_ptr(), _dt(out), S.data_ptr(), ml.data_ptr(), po.data_ptr(),
        block_table.data_ptr(), block_table.shape[1], req_of_token.data_ptr(), positions.data_ptr(), T, H, Hkv, hd, vd, page_size,
        int(window or 0), float(scale), ptr(sinks), ptr(slopes), ptr(r1), ptr(r2), ptr(talk), ptr(gates), gate_stride, n_parts,
        _stream()), "attention_decode_exact")


def attention_prefill_wide_supported(dtype, hd: int, vd: int, page_size: int) -> bool:
    return dtype == torch.bfloat16 and hd % 8 == 0 and vd % 8 == 0 and max(hd, vd) <= 256 and page_size % 16 == 0


def attention_prefill_wide(q, k_cache, v_cache, out, *, block_table, blocks, req_info, H, Hkv, hd, vd, page_size, max_ctx_len,
                           window=0, scale=None, sinks=None, slopes=None, log_distance=None, all_values: bool = False) -> None:
    """attention_prefill's kernel in its wide form: values of vd channels (v_cache [P, Hkv, vd, page_size]), softmax
    weights that keep float32's precision through the matrix cores, and optionally log_distance = (r1, r2), float32 [H]
    each: r1[h] * ln(1 + r2[h] * (position - key)) is taken off head h's scaled scores.  all_values: every query head's
    weights are applied to the values of every kv head and out is float32 [T, H * Hkv * vd] (head, kv head, channel), for
    head_mix_gate; otherwise out is bfloat16 [T, H * vd].  The keys are not cut into segments."""
    T = q.shape[0]
    if not attention_prefill_wide_supported(q.dtype, hd, vd, page_size):
        raise KernelError(f"attention_prefill_wide: needs bfloat16, head sizes that are multiples of 8 (got {hd}, {vd}) "
                          f"and a page size that is a multiple of 16 (got {page_size})")
    _opt("sinks", sinks, torch.float32, (H,))
    _opt("slopes", slopes, torch.float32, (H,))
    r1 = r2 = None
    if log_distance is not None:
        r1, r2 = log_distance
        _gpu("log_distance r1", r1, torch.float32, (H,))
        _gpu("log_distance r2", r2, torch.float32, (H,))
    _gpu("q", q, torch.bfloat16, (T, H * hd))
    if all_values:
        _gpu("out", out, torch.float32, (T, H * Hkv * vd))
    else:
        _gpu("out", out, torch.bfloat16, (T, H * vd))
    P = k_cache.shape[0]
    _gpu("k_cache", k_cache, torch.bfloat16, (P, Hkv, page_size, hd))
    _gpu("v_cache", v_cache, torch.bfloat16, (P, Hkv, vd, page_size))
    _gpu("block_table", block_table, torch.int32)
    R = req_info.shape[0]
    _gpu("req_info", req_info, torch.int32, (R, 4))
    if block_table.dim() != 2 or block_table.shape[0] != R:
        raise KernelError("attention_prefill_wide: block_table must be [requests, blocks]")
    if block_table.shape[1] * page_size < int(max_ctx_len):
        raise KernelError("attention_prefill_wide: block_table is narrower than the longest context")
    if H % Hkv:
        raise KernelError("attention_prefill_wide: the query heads must be a multiple of the kv heads")
    if blocks is None:
        if H // Hkv > attention_prefill_block_columns(max(hd, vd)):
            raise KernelError("attention_prefill_wide: without a block list a request's columns must fit one block")
        nblk = R
    else:
        nblk = blocks.shape[0]
        _gpu("blocks", blocks, torch.int32, (nblk, 2))
    if scale is None:
        scale = 1.0 / math.sqrt(hd)
    _check(load("attention_prefill").tuff_attention_prefill_wide(
        q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), out.data_ptr(), block_table.data_ptr(), block_table.shape[1],
        None if blocks is None else blocks.data_ptr(), nblk, req_info.data_ptr(), H, Hkv, hd, vd, page_size, int(window or 0),
        float(scale), None if sinks is None else sinks.data_ptr(), None if slopes is None else slopes.data_ptr(),
        None if r1 is None else r1.data_ptr(), None if r2 is None else r2.data_ptr(), int(bool(all_values)), _stream()),
        "attention_prefill_wide")


def query_blocks(q_len, G: int, nb: int, ctx_len=None):
    """Host list of query blocks for attention_mfma and attention_prefill: for request r with q_len[r]
    tokens the columns (token, head in group) are cut into blocks of 16 * nb.  Returns int32
    [n_blocks, 2] = (request, first column).  With ctx_len (tokens of each request in the cache after
    the step) the blocks whose last column sees the most keys come first (attention_prefill starts
    its workgroups in the list's order, and the longest should not start last); the order has no
    influence on any result."""
    import numpy as np
    q_len = np.asarray(q_len, dtype=np.int64)
    per = -(-(q_len * G) // (16 * nb))
    blk_req = np.repeat(np.arange(len(q_len)), per)
    starts = np.concatenate([[0], np.cumsum(per)])[:-1]
    blk_col0 = (np.arange(int(per.sum())) - np.repeat(starts, per)) * 16 * nb
    if ctx_len is not None and len(blk_req):
        ctx_len = np.asarray(ctx_len, dtype=np.int64)
        last_tok = np.minimum(q_len[blk_req] - 1, (blk_col0 + 16 * nb - 1) // G)
        keys = ctx_len[blk_req] - q_len[blk_req] + last_tok + 1
        order = np.argsort(-keys, kind="stable")
        blk_req, blk_col0 = blk_req[order], blk_col0[order]
    return np.stack([blk_req, blk_col0], axis=1).astype(np.int32)


# ------------------------------------------------------------------------- short conv
def shortconv_fwd(bcx, conv_w, state, out, *, req_of_token, q_start, state_slot, K, q_len=None) -> None:
    """The gated short convolution of a step's tokens, each request's earlier values from its state slot.
    With q_len (int32 [requests]) the state of every request with tokens in the step is rewritten too,
    as shortconv_state would afterwards; without, the state is only read."""
    T, d = out.shape
    dt = out.dtype
    _gpu("bcx", bcx, dt, (T, 3 * d))
    _gpu("out", out)
    _gpu("conv_w", conv_w, shape=(d, K))
    _gpu("state", state, torch.float32, (None, K - 1, d))
    R = q_start.shape[0]
    _gpu("req_of_token", req_of_token, torch.int32, (T,))
    _gpu("q_start", q_start, torch.int32, (R,))
    _gpu("state_slot", state_slot, torch.int32, (R,))
    if q_len is not None:
        _gpu("q_len", q_len, torch.int32, (R,))
    _check(load("shortconv").tuff_shortconv_fwd(
        bcx.data_ptr(), conv_w.data_ptr(), _dt(conv_w), state.data_ptr(), out.data_ptr(), _dt(out),
        req_of_token.data_ptr(), q_start.data_ptr(), None if q_len is None else q_len.data_ptr(), state_slot.data_ptr(),
        T, d, K, _stream()), "shortconv_fwd")


def shortconv_decode(bcx, conv_w, state, out, *, state_slot, K) -> None:
    """Output and state update in one kernel for a step in which every request has one token
    (row r of bcx is request r's token)."""
    R, d = out.shape
    dt = out.dtype
    _gpu("bcx", bcx, dt, (R, 3 * d))
    _gpu("out", out)
    _gpu("conv_w", conv_w, shape=(d, K))
    _gpu("state", state, torch.float32, (None, K - 1, d))
    _gpu("state_slot", state_slot, torch.int32, (R,))
    _check(load("shortconv").tuff_shortconv_decode(
        bcx.data_ptr(), conv_w.data_ptr(), _dt(conv_w), state.data_ptr(), out.data_ptr(), _dt(out),
        state_slot.data_ptr(), R, d, K, _stream()), "shortconv_decode")


def shortconv_state(bcx, state, *, q_start, q_len, state_slot, K) -> None:
    d = state.shape[2]
    R = q_start.shape[0]
    _gpu("bcx", bcx, shape=(None, 3 * d))
    _gpu("state", state, torch.float32, (None, K - 1, d))
    _gpu("q_start", q_start, torch.int32, (R,))
    _gpu("q_len", q_len, torch.int32, (R,))
    _gpu("state_slot", state_slot, torch.int32, (R,))
    _check(load("shortconv").tuff_shortconv_state(
        bcx.data_ptr(), _dt(bcx), state.data_ptr(), q_start.data_ptr(), q_len.data_ptr(),
        state_slot.data_ptr(), R, d, K, _stream()), "shortconv_state")


# -------------------------------------------------------------------- recurrent mixers
def shift_mix(h, prev_state, mu, out, *, req_of_token, q_start, state_slot, q_len=None) -> None:
    """out[s, t] = h[t] + (h[t - 1] - h[t]) * mu[s]; the row before a request's first token of the step is
    prev_state[slot] (float32 [slots, d]).  h [T, d]; mu float32 [n, d]; out [n, T, d] of h's type.  With q_len
    the state is then rewritten with each request's last row of the step (as shift_state does); without, it is
    only read."""
    T, d = h.shape
    n = mu.shape[0]
    R = q_start.shape[0]
    _check(load("recurrent").tuff_shift_mix(
        _gpu("h", h), _dt(h), _gpu("prev_state", prev_state, torch.float32, (None, d)), _gpu("mu", mu, torch.float32, (n, d)),
        _gpu("out", out, h.dtype, (n, T, d)), _gpu("req_of_token", req_of_token, torch.int32, (T,)),
        _gpu("q_start", q_start, torch.int32, (R,)), _opt("q_len", q_len, torch.int32, (R,)),
        _gpu("state_slot", state_slot, torch.int32, (R,)), T, d, n, _stream()), "shift_mix")


def shift_state(h, prev_state, *, q_start, q_len, state_slot) -> None:
    """prev_state[slot] = the last row each request has in the step."""
    T, d = h.shape
    R = q_start.shape[0]
    _check(load("recurrent").tuff_shift_state(
        _gpu("h", h), _dt(h), _gpu("prev_state", prev_state, torch.float32, (None, d)),
        _gpu("q_start", q_start, torch.int32, (R,)), _gpu("q_len", q_len, torch.int32, (R,)),
        _gpu("state_slot", state_slot, torch.int32, (R,)), R, d, _stream()), "shift_state")


CONV_ACT_MAX_TAPS = 17


def _rows_view(name: str, t: torch.Tensor, width: Optional[int] = None) -> int:
    """Checks a [T, width] tensor on the GPU whose rows may be a column range of a wider tensor (unit column
    stride, any row stride of at least the width); returns the row stride in elements."""
    if not isinstance(t, torch.Tensor) or not t.is_cuda:
        raise KernelError(f"{name}: expected a tensor on the GPU")
    if t.dim() != 2 or (width is not None and t.shape[1] != width) or (t.shape[1] > 1 and t.stride(1) != 1):
        raise KernelError(f"{name}: expected [tokens, {width}] with unit column stride, got {tuple(t.shape)} stride {t.stride()}")
    ld = t.stride(0) if t.shape[0] > 1 else max(t.stride(0), t.shape[1])
    if ld < t.shape[1]:
        raise KernelError(f"{name}: rows overlap (stride {t.stride()})")
    return ld


def conv_act(x, taps, state, out, *, req_of_token, q_start, state_slot, q_len=None, activation: Optional[str] = "silu",
             bias=None) -> None:
    """out[t, c] = activation(sum_j taps[c, j] x[t - (K - 1) + j, c] + bias[c]) along each request; rows before the
    step's first come from state[slot] (float32 [slots, K - 1, C]; None with one tap).  With q_len the state
    is then rewritten with the last K - 1 inputs; without, it is only read.  x may be a column range of a wider
    tensor, and float32 where out is bfloat16 (a product's sums as they are); bias float32 [C] or None."""
    T, C = x.shape
    K = taps.shape[1]
    R = q_start.shape[0]
    if activation not in (None, "silu"):
        raise KernelError("conv_act: activation is 'silu' or None")
    if not 1 <= K <= CONV_ACT_MAX_TAPS:
        raise KernelError(f"conv_act: 1 to {CONV_ACT_MAX_TAPS} taps, got {K}")
    if K > 1:
        _gpu("state", state, torch.float32, (None, K - 1, C))
    ldx = _rows_view("x", x)
    if x.dtype != out.dtype and x.dtype != torch.float32:
        raise KernelError(f"conv_act: input {x.dtype} with output {out.dtype}")
    _check(load("recurrent").tuff_conv_act(
        x.data_ptr(), _dt(x), ldx, _gpu("taps", taps, torch.float32, (C, K)), _opt("bias", bias, torch.float32, (C,)),
        None if K == 1 else state.data_ptr(),
        _gpu("out", out, shape=(T, C)), _dt(out), _gpu("req_of_token", req_of_token, torch.int32, (T,)),
        _gpu("q_start", q_start, torch.int32, (R,)), _opt("q_len", q_len, torch.int32, (R,)),
        _gpu("state_slot", state_slot, torch.int32, (R,)), T, R, C, K, 1 if activation == "silu" else 0, _stream()), "conv_act")


SCAN_MAX_DIM = 256


def wkv_scan(r, k, v, lw, w0, u, state, out, *, q_start, q_len, state_slot, H, D) -> None:
    """The decaying outer-product recurrence over each request's tokens of the step, from and to
    state[slot] (float32 [slots, H, D, D]): o = (S + diag(u) k v^T)^T r, then S = diag(w) S + k v^T with
    w = exp(-exp(lw + w0)).  r, k, v [T, H * D]; lw float32 [T, H * D] (overwritten with the decays); w0 float32
    [H * D]; u float32 [H, D]; out float32 [T, H * D]."""
    T = r.shape[0]
    R = q_start.shape[0]
    dt = r.dtype
    if D > SCAN_MAX_DIM:
        raise KernelError(f"wkv_scan: head size {D} above {SCAN_MAX_DIM}")
    _check(load("recurrent").tuff_wkv_scan(
        _gpu("r", r, shape=(T, H * D)), _gpu("k", k, dt, (T, H * D)), _gpu("v", v, dt, (T, H * D)), _dt(r),
        _gpu("lw", lw, torch.float32, (T, H * D)), _gpu("w0", w0, torch.float32, (H * D,)), _gpu("u", u, torch.float32, (H, D)),
        torch.empty(T, H, dtype=torch.float32, device=r.device).data_ptr(),
        _gpu("state", state, torch.float32, (None, H, D, D)), _gpu("out", out, torch.float32, (T, H * D)),
        _gpu("q_start", q_start, torch.int32, (R,)), _gpu("q_len", q_len, torch.int32, (R,)),
        _gpu("state_slot", state_slot, torch.int32, (R,)), T, R, H, D, _stream()), "wkv_scan")


def delta_scan(q, k, v, a, dt_bias, A_log, b, state, out, *, q_start, q_len, state_slot, H, Hk, D, Dv, per_head: bool = False) -> None:
    """The gated delta rule over each request's tokens of the step, from and to state[slot] (float32
    [slots, H, D, Dv]): S = g S; e = beta (v - S^T k); S = S + k e^T; o = S^T q, with q and k made unit
    vectors per head (q also times D^-1/2), g = exp(-exp(A_log) softplus(a + dt_bias)), beta = sigmoid(b).
    q, k [T, Hk * D]; v [T, H * Dv]; a float32 [T, H * D] (overwritten with the decays) and dt_bias [H * D]; b float32
    [T, H]; out float32 [T, H * Dv].  per_head: one decay per head, a float32 [T, H] and dt_bias [H] (a and b may then
    be column ranges of one wider tensor, with one row stride)."""
    T = q.shape[0]
    R = q_start.shape[0]
    dt = q.dtype
    # q, k and v may be column ranges of one wider tensor (the convolution's output): rows of one stride
    ld, ldv = q.stride(0), v.stride(0)
    for name, t, width, want in (("q", q, Hk * D, ld), ("k", k, Hk * D, ld), ("v", v, H * Dv, ldv)):
        if (not t.is_cuda or t.dtype != dt or t.dim() != 2 or t.shape != (T, width) or t.stride(1) != 1 or t.stride(0) != want
                or want < width):
            raise KernelError(f"delta_scan: {name} must be [{T}, {width}] of {dt} on the GPU with unit column stride (q and k "
                              f"with one row stride); got {tuple(t.shape)} {t.dtype} stride {t.stride()}")
    if D > SCAN_MAX_DIM or Hk < 1 or H % Hk:
        raise KernelError(f"delta_scan: key size {D} (at most {SCAN_MAX_DIM}) / heads {H}:{Hk} not supported")
    work = torch.empty(2, T, H * D, dtype=torch.float32, device=q.device)       # q and k as unit vectors
    if per_head:
        ld_small = _rows_view("b", b, H)
        if a.dtype != torch.float32 or b.dtype != torch.float32 or _rows_view("a", a, H) != ld_small:
            raise KernelError("delta_scan: a and b must be float32 [tokens, heads] with one row stride")
        decays = torch.empty(T, H * D, dtype=torch.float32, device=q.device)
        a_head, a_ptr = a.data_ptr(), decays.data_ptr()
        _gpu("dt_bias", dt_bias, torch.float32, (H,))
    else:
        ld_small, a_head = H, None
        a_ptr = _gpu("a", a, torch.float32, (T, H * D))
        _gpu("dt_bias", dt_bias, torch.float32, (H * D,))
        _gpu("b", b, torch.float32, (T, H))
    _check(load("recurrent").tuff_delta_scan(
        q.data_ptr(), k.data_ptr(), v.data_ptr(), _dt(q),
        a_ptr, dt_bias.data_ptr(), _gpu("A_log", A_log, torch.float32, (H,)), b.data_ptr(), a_head, ld_small,
        work[0].data_ptr(), work[1].data_ptr(), torch.empty(T, H, dtype=torch.float32, device=q.device).data_ptr(),
        _gpu("state", state, torch.float32, (None, H, D, Dv)), _gpu("out", out, torch.float32, (T, H * Dv)),
        _gpu("q_start", q_start, torch.int32, (R,)), _gpu("q_len", q_len, torch.int32, (R,)),
        _gpu("state_slot", state_slot, torch.int32, (R,)), T, R, H, Hk, D, Dv, ld, ldv, _stream()), "delta_scan")


def ssd_scan(xbc, dt_raw, dt_bias, A_log, D_skip, state, out, *, q_start, q_len, state_slot, H, G, N, P) -> None:
    """The state-space recurrence with a scalar decay per head over each request's tokens of the step, from and to
    state[slot] (float32 [slots, H, N, P]): with dt = softplus(dt_raw + dt_bias) per head,
    S = exp(-exp(A_log) dt) S + dt B x^T;  y = S^T C + D_skip x  (the read sees the token's own write).
    xbc [T, H P + 2 G N]: a token's x, B and C side by side (after their convolution), head h reading B and C of
    group h // (H / G); dt_raw float32 [T, H] (it may be a column range of a wider tensor); dt_bias, A_log, D_skip
    float32 [H]; out float32 [T, H * P]."""
    T = xbc.shape[0]
    R = q_start.shape[0]
    if N > SCAN_MAX_DIM:
        raise KernelError(f"ssd_scan: state size {N} above {SCAN_MAX_DIM}")
    if G < 1 or H % G:
        raise KernelError(f"ssd_scan: {H} heads in {G} groups")
    ld = _rows_view("xbc", xbc, H * P + 2 * G * N)
    ld_dt = _rows_view("dt_raw", dt_raw, H)
    if dt_raw.dtype != torch.float32:
        raise KernelError("ssd_scan: dt_raw must be float32")
    work = torch.empty(2, T, H, dtype=torch.float32, device=xbc.device)     # step sizes and decays
    _check(load("recurrent").tuff_ssd_scan(
        xbc.data_ptr(), _dt(xbc), ld, dt_raw.data_ptr(), ld_dt, _gpu("dt_bias", dt_bias, torch.float32, (H,)),
        _gpu("A_log", A_log, torch.float32, (H,)), _gpu("D_skip", D_skip, torch.float32, (H,)),
        work[0].data_ptr(), work[1].data_ptr(),
        _gpu("state", state, torch.float32, (None, H, N, P)), _gpu("out", out, torch.float32, (T, H * P)),
        _gpu("q_start", q_start, torch.int32, (R,)), _gpu("q_len", q_len, torch.int32, (R,)),
        _gpu("state_slot", state_slot, torch.int32, (R,)), T, R, H, G, N, P, _stream()), "ssd_scan")


SSD_CHUNK = 64                   # tokens a chunk of ssd_chunked


def ssd_chunked_supported(dtype, N: int, P: int) -> bool:
    """Whether the chunked form takes these sizes: bfloat16 rows, state and head sizes that are multiples of 16, a state of
    at most 128 and heads of at most 64 channels (what a workgroup's 64 KB of LDS hold)."""
    return dtype == torch.bfloat16 and N % 16 == 0 and P % 16 == 0 and 0 < N <= 128 and 0 < P <= 64


def ssd_chunked(xbc, dt_raw, dt_bias, A_log, D_skip, state, out, *, q_start, q_len, state_slot, H, G, N, P) -> None:
    """ssd_scan's recurrence for prompt portions in chunks of 64 tokens on the matrix cores (float32 matrix instructions;
    all factors, sums and the state float32): the same function, its sums in another order.  xbc bfloat16; the other
    arguments as for ssd_scan."""
    T = xbc.shape[0]
    R = q_start.shape[0]
    if not ssd_chunked_supported(xbc.dtype, N, P):
        raise KernelError(f"ssd_chunked: bfloat16 rows, a state of {N} (a multiple of 16 up to 128) and heads of {P} (up to 64) channels")
    if G < 1 or H % G:
        raise KernelError(f"ssd_chunked: {H} heads in {G} groups")
    ld = _rows_view("xbc", xbc, H * P + 2 * G * N)
    ld_dt = _rows_view("dt_raw", dt_raw, H)
    if dt_raw.dtype != torch.float32:
        raise KernelError("ssd_chunked: dt_raw must be float32")
    chunks = -(-T // SSD_CHUNK) + R
    small = torch.empty(3 * T * H + chunks * H, dtype=torch.float32, device=xbc.device)      # step sizes, decays, their logarithms; chunk decays
    U = torch.empty(chunks, H, N, P, dtype=torch.float32, device=xbc.device)
    at = lambda i: small.data_ptr() + 4 * i * T * H
    _check(load("recurrent").tuff_ssd_chunked(
        xbc.data_ptr(), ld, dt_raw.data_ptr(), ld_dt, _gpu("dt_bias", dt_bias, torch.float32, (H,)),
        _gpu("A_log", A_log, torch.float32, (H,)), _gpu("D_skip", D_skip, torch.float32, (H,)),
        at(0), at(1), at(2), U.data_ptr(), at(3), chunks,
        _gpu("state", state, torch.float32, (None, H, N, P)), _gpu("out", out, torch.float32, (T, H * P)),
        _gpu("q_start", q_start, torch.int32, (R,)), _gpu("q_len", q_len, torch.int32, (R,)),
        _gpu("state_slot", state_slot, torch.int32, (R,)), T, R, H, G, N, P, _stream()), "ssd_chunked")


def forget_scan(x, bias, lower, state, out, *, q_start, q_len, state_slot, H, D, Dv) -> None:
    """The forget-gate recurrence over each request's tokens of the step, from and to state[slot] (float32
    [slots, H, D, Dv]): f = lower + (1 - lower) sigmoid(z + bias); S = diag(f) S + (1 - f) v^T; o = S^T silu(q).
    x [T, 2 H D + H Dv]: a token's projected rows q, z, v side by side; bias (or None) and lower float32 [H * D];
    out float32 [T, H * Dv]."""
    T = x.shape[0]
    R = q_start.shape[0]
    if D > SCAN_MAX_DIM:
        raise KernelError(f"forget_scan: key size {D} above {SCAN_MAX_DIM}")
    work = torch.empty(2, T, H * D, dtype=torch.float32, device=x.device)       # silu(q) and the gates
    _check(load("recurrent").tuff_forget_scan(
        _gpu("x", x, shape=(T, 2 * H * D + H * Dv)), _dt(x), x.shape[1], _opt("bias", bias, torch.float32, (H * D,)),
        _gpu("lower", lower, torch.float32, (H * D,)), work[0].data_ptr(), work[1].data_ptr(),
        _gpu("state", state, torch.float32, (None, H, D, Dv)), _gpu("out", out, torch.float32, (T, H * Dv)),
        _gpu("q_start", q_start, torch.int32, (R,)), _gpu("q_len", q_len, torch.int32, (R,)),
        _gpu("state_slot", state_slot, torch.int32, (R,)), T, R, H, D, Dv, _stream()), "forget_scan")


def head_norm_gate(o, w, gate, out, *, H, Dv, eps, per_head_weight: bool, gate_activation: Optional[str],
                   gate_first: bool = False) -> None:
    """out[t, h] = o[t, h] / sqrt(mean(o[t, h]^2) + eps) * w * f(gate[t, h]); o float32 [T, H * Dv]; w float32
    [H * Dv] (per_head_weight) or [Dv] (shared by the heads); out [T, H * Dv] of the compute type, gate of that
    type or float32 (it may be a column range of a wider tensor), or None for no gate.  gate_first: the gate comes
    before the norm, out = u / sqrt(mean(u^2) + eps) * w with u = o f(gate)."""
    T = o.shape[0]
    gate_ld = 0 if gate is None else _rows_view("gate", gate, H * Dv)
    _check(load("recurrent").tuff_head_norm_gate(
        _gpu("o", o, torch.float32, (T, H * Dv)), _gpu("w", w, torch.float32, (H * Dv if per_head_weight else Dv,)),
        Dv if per_head_weight else 0, None if gate is None else gate.data_ptr(), gate_ld, _dt(out if gate is None else gate), _dt(out),
        {None: 0, "silu": 1, "sigmoid": 2}[gate_activation], int(bool(gate_first)), _gpu("out", out, shape=(T, H * Dv)), T, H, Dv,
        float(eps), _stream()), "head_norm_gate")


# ------------------------------------------------------------------ mixture of experts
def moe_route(z, ids, wts, *, E, top, weights: str = "sigmoid") -> None:
    """ids, wts [T, top]: the `top` largest of z[t, :E] (float32 [T, >= E]; the lower index wins a tie) and
    their weights, sigmoid(z) each on its own or a softmax over the chosen."""
    T = z.shape[0]
    _gpu("z", z, torch.float32)
    if z.dim() != 2 or z.shape[1] < E:
        raise KernelError("moe_route: z must be [tokens, >= experts]")
    _check(load("moe").tuff_moe_route(z.data_ptr(), z.shape[1], _gpu("ids", ids, torch.int32, (T, top)),
                                      _gpu("wts", wts, torch.float32, (T, top)), T, E, top,
                                      {"sigmoid": 0, "softmax": 1}[weights], _stream()), "moe_route")


ROUTER_MAX_FLOATS = 16380          # hidden size + logits a token: what the router kernel keeps in LDS


def moe_router(h, w, z, ids, wts, *, E, top, weights: str = "sigmoid", bias=None, correction=None, groups: int = 0,
               keep: int = 0, scale: float = 1.0) -> None:
    """z = h @ w.T in float32 (h [T, d] of the compute type, w float32 [N, d], z float32 [T, N]) and, of its first
    E columns, the choice as moe_route makes it, in one kernel.  bias: float32 [E], added to the experts' logits.
    groups > 0 (sigmoid weights): a limited choice.  It runs on sigmoid(z) + correction (float32 [E] or None) and only
    inside the `keep` groups, of `groups` equal groups of neighbouring experts, whose two largest such scores have the
    largest sum; the weights are sigmoid(z) of the chosen, without the correction, times `scale`."""
    T, d = h.shape
    N = w.shape[0]
    if d + N + (E if groups else 0) > ROUTER_MAX_FLOATS:
        raise KernelError(f"moe_router: hidden size {d} + {N} logits above {ROUTER_MAX_FLOATS}")
    if groups and (weights != "sigmoid" or groups > 64 or E % groups or not 1 <= keep <= groups or top > keep * (E // groups)):
        raise KernelError(f"moe_router: a limited choice of {top} among {keep} of {groups} groups of {E} experts is not possible")
    _check(load("moe").tuff_moe_router(_gpu("h", h), _dt(h), _gpu("w", w, torch.float32, (N, d)), _gpu("z", z, torch.float32, (T, N)),
                                       _gpu("ids", ids, torch.int32, (T, top)), _gpu("wts", wts, torch.float32, (T, top)),
                                       T, d, N, E, top, {"sigmoid": 0, "softmax": 1}[weights],
                                       _opt("bias", bias, torch.float32, (E,)), _opt("correction", correction, torch.float32, (E,)),
                                       int(groups), int(keep), float(scale), _stream()), "moe_router")


def tile_experts(ws) -> torch.Tensor:
    """Every expert's bfloat16 matrix [N, K] in the order tile_weight gives one, stacked: [E, ceil(N/16), ceil(K/32), 64, 8]."""
    return torch.stack([tile_weight(w).blocks for w in ws]).contiguous()


def moe_grouped_supported(dtype, d: int, F: int, E: int) -> bool:
    return dtype == torch.bfloat16 and d % 8 == 0 and F % 8 == 0 and 1 <= E <= 1024


EXPERT_ACTIVATIONS = {"relu2": 0, "silu": 1, "gelu_tanh": 2, "swish_clamp": 3}


def _expert_activation(activation: str, gated: bool, limit: float) -> int:
    if activation == "swish_clamp" and (not gated or not limit > 0):
        raise KernelError("experts: the clamped form needs gated experts and a positive limit")
    return EXPERT_ACTIVATIONS[activation]


def interleave_gate_up(gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
    """[2 F, d] with row 2 f = gate[f] and row 2 f + 1 = up[f]: the first matrix of a gated expert as
    moe_experts_grouped takes it (before tile_experts)."""
    return torch.stack([gate, up], dim=1).reshape(2 * gate.shape[0], gate.shape[1]).contiguous()


def moe_experts_grouped(h, up_tiles, down_tiles, ids, wts, residual, *, F: int, activation: str = "relu2",
                        scale_input: bool = True, gated: bool = False, limit: float = 0.0, alpha: float = 1.0) -> None:
    """moe_experts on the matrix cores, bfloat16: the rows (token, choice) are sorted by expert and every expert's
    rows go through its two matrices in tiles.  up_tiles, down_tiles: tile_experts() of the [F, d] and [d, F] matrices;
    gated: of interleave_gate_up(gate, up) [2 F, d] and [d, F]."""
    T, d = h.shape
    E, top = up_tiles.shape[0], ids.shape[1]
    if not moe_grouped_supported(h.dtype, d, F, E):
        raise KernelError(f"moe_experts_grouped: bfloat16, sizes that are multiples of 8 and at most 1024 experts; got {h.dtype}, {d}, {F}, {E}")
    _gpu("h", h, torch.bfloat16)
    _gpu("up_tiles", up_tiles, torch.bfloat16, (E, -(-(2 * F if gated else F) // 16), -(-d // 32), 64, 8))
    _gpu("down_tiles", down_tiles, torch.bfloat16, (E, -(-d // 16), -(-F // 32), 64, 8))
    _gpu("ids", ids, torch.int32, (T, top))
    _gpu("wts", wts, torch.float32, (T, top))
    _gpu("residual", residual, torch.float32, (T, d))
    R = T * top
    lib = load("moe")
    max_tiles = -(-R // int(lib.tuff_moe_grouped_tile_rows(R, E))) + E
    dev = h.device
    srt = torch.empty(R, dtype=torch.int32, device=dev)
    tiles = torch.empty(3 * max_tiles, dtype=torch.int32, device=dev)
    a = torch.empty(R, F, dtype=torch.bfloat16, device=dev)
    y = torch.empty(R, d, dtype=torch.float32, device=dev)
    _check(lib.tuff_moe_experts_grouped(h.data_ptr(), up_tiles.data_ptr(), down_tiles.data_ptr(), ids.data_ptr(), wts.data_ptr(),
                                        srt.data_ptr(), tiles.data_ptr(), max_tiles, a.data_ptr(), y.data_ptr(),
                                        residual.data_ptr(), T, d, F, E, top,
                                        _expert_activation(activation, gated, limit), int(scale_input), int(gated),
                                        float(limit), float(alpha), _stream()),
           "moe_experts_grouped")


def moe_experts(h, w_up, w_down, ids, wts, residual, *, activation: str = "relu2", scale_input: bool = True,
                gated: bool = False, limit: float = 0.0, alpha: float = 1.0) -> None:
    """residual[t] += sum over the token's choices of W_down[e] act(W_up[e] x), x = h[t] times the choice's
    weight (scale_input) or the product times it.  h [T, d]; w_up [E, F, d]; w_down [E, d, F], all of one type.
    gated: w_up is [E, 2 F, d], an expert's gate rows then its up rows, and the activation joins the two."""
    T, d = h.shape
    E, F, _ = w_up.shape
    if gated:
        if F % 2:
            raise KernelError("moe_experts: a gated expert's first matrix holds gate and up rows, an even number")
        F //= 2
    top = ids.shape[1]
    dt = h.dtype
    _gpu("h", h)
    _gpu("w_up", w_up, dt, (E, 2 * F if gated else F, d))
    _gpu("w_down", w_down, dt, (E, d, F))
    _gpu("ids", ids, torch.int32, (T, top))
    _gpu("wts", wts, torch.float32, (T, top))
    _gpu("residual", residual, torch.float32, (T, d))
    a = torch.empty(T * top, F, dtype=dt, device=h.device)
    y = torch.empty(T * top, d, dtype=torch.float32, device=h.device)
    _check(load("moe").tuff_moe_experts(h.data_ptr(), w_up.data_ptr(), w_down.data_ptr(), _dt(h), ids.data_ptr(),
                                        wts.data_ptr(), a.data_ptr(), y.data_ptr(), residual.data_ptr(), T, d, F, top,
                                        _expert_activation(activation, gated, limit), int(scale_input), int(gated),
                                        float(limit), float(alpha), _stream()),
           "moe_experts")


# --------------------------------------------------------------------------- sampling
def argmax(logits: torch.Tensor, out: torch.Tensor) -> None:
    R, V = logits.shape
    _check(load("sampling").tuff_argmax(_gpu("logits", logits, torch.float32), _gpu("out", out, torch.int32, (R,)),
                                        R, V, _stream()), "argmax")


def sample(logits, out, *, temps=None, top_ks=None, top_ps=None, min_ps=None, uniforms=None) -> None:
    """One token per row: greedy where temps[r] <= 0 (or temps is None), else the reference's
    chain min-p -> top-k -> top-p -> draw with the host-supplied uniform of that row."""
    R, V = logits.shape
    _gpu("logits", logits, torch.float32)
    _gpu("out", out, torch.int32, (R,))
    if temps is not None and uniforms is None:
        raise KernelError("sample: stochastic rows need uniforms")
    p = lambda n, t, dt: None if t is None else _gpu(n, t, dt, (R,))
    _check(load("sampling").tuff_sample(
        logits.data_ptr(), p("temps", temps, torch.float32), p("top_ks", top_ks, torch.int32),
        p("top_ps", top_ps, torch.float32), p("min_ps", min_ps, torch.float32),
        p("uniforms", uniforms, torch.float32), out.data_ptr(), R, V, _stream()), "sample")


def repeat_penalty(logits, recent, counts, penalties) -> None:
    """In place: each row's logits penalised once per entry of its ring of recent tokens."""
    R, V = logits.shape
    cap = recent.shape[1]
    _gpu("logits", logits, torch.float32)
    _gpu("recent", recent, torch.int32, (R, cap))
    _gpu("counts", counts, torch.int32, (R,))
    _gpu("penalties", penalties, torch.float32, (R,))
    _check(load("sampling").tuff_repeat_penalty(logits.data_ptr(), recent.data_ptr(), counts.data_ptr(),
                                                penalties.data_ptr(), R, cap, V, _stream()), "repeat_penalty")
