"""Python faces of the HIP kernels: each checks its operands on the host (device, dtype, shape,
contiguity) and launches on torch's current stream.  Tensors are torch tensors used as plain
device memory; no torch arithmetic happens here.
"""
from __future__ import annotations

import ctypes
from ctypes import c_float, c_int, c_long, c_void_p

from functools import lru_cache
from typing import Optional

import torch

from . import library

F32, BF16 = 0, 1
_CODE = {torch.float32: F32, torch.bfloat16: BF16}


class KernelError(RuntimeError):
    pass


_SIGNATURES = {
    "gi_embed": [c_void_p, c_int, c_void_p, c_void_p, c_int, c_int, c_void_p],
    "gi_embed_handing": [c_void_p, c_int, c_void_p, c_void_p, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p],
    "gi_rmsnorm": [c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_int, c_int, c_int, c_float, c_long, c_long, c_void_p],
    "gi_rope_cos_sin": [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_float, c_void_p],
    "gi_rope_store": [c_void_p, c_void_p, c_void_p, c_long, c_long, c_long, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                      c_int, c_void_p, c_int, c_void_p, c_int, c_long, c_int, c_int, c_int, c_int, c_int, c_void_p],
    "gi_silu_mul": [c_void_p, c_void_p, c_int, c_int, c_int, c_void_p],
    "gi_gather_rows": [c_void_p, c_void_p, c_void_p, c_int, c_int, c_void_p],
    "gi_scale_rows": [c_void_p, c_int, c_int, c_long, c_float, c_void_p],
    "gi_softcap_rows": [c_void_p, c_int, c_int, c_long, c_float, c_void_p],
    "gi_gemm_exact": [c_void_p, c_int, c_void_p, c_int, c_void_p, c_int, c_int, c_int, c_int, c_int, c_long, c_long, c_long, c_void_p],
    "gi_attention_exact": [c_void_p, c_int, c_void_p, c_int, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int, c_long, c_int,
                           c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_float, c_float, c_void_p, c_void_p, c_long, c_void_p],
    "gi_rmsnorm_add": [c_void_p, c_void_p, c_int, c_void_p, c_int, c_int, c_float, c_long, c_long, c_void_p],
    "gi_rmsnorm_add_norm": [c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_int, c_int, c_int, c_float, c_float, c_long, c_long, c_long, c_void_p],
    "gi_norm_rope_store": [c_void_p, c_void_p, c_void_p, c_long, c_long, c_long, c_void_p, c_void_p, c_int, c_float, c_void_p, c_void_p, c_int,
                           c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_int, c_void_p, c_int, c_long, c_int, c_int, c_int, c_int, c_int, c_int,
                           c_void_p, c_void_p, c_void_p, c_void_p, c_long, c_void_p, c_void_p, c_long, c_int, c_float, c_void_p, c_void_p],
    "gi_concat_rows": [c_void_p, c_long, c_int, c_void_p, c_long, c_int, c_void_p, c_int, c_long, c_int, c_void_p],
    "gi_add_weighted": [c_void_p, c_long, c_void_p, c_long, c_float, c_void_p, c_long, c_float, c_int, c_int, c_void_p],
    "gi_add_vector": [c_void_p, c_long, c_void_p, c_int, c_int, c_int, c_void_p],
    "gi_gate_token_columns": [c_void_p, c_long, c_void_p, c_int, c_long, c_int, c_void_p, c_void_p, c_int, c_long, c_int, c_int, c_int, c_void_p],
    "gi_gate_token_columns_rows": [c_void_p, c_long, c_void_p, c_int, c_long, c_int, c_void_p, c_int, c_long, c_int, c_void_p, c_void_p, c_int, c_long, c_int, c_int, c_int, c_int,
                                   c_void_p],
    "gi_ssm_conv": [c_void_p, c_long, c_void_p, c_int, c_void_p, c_void_p, c_long, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_void_p],
    "gi_ssm_tail": [c_void_p, c_long, c_int, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_long, c_int, c_int, c_void_p],
    "gi_ssm_scan": [c_void_p, c_void_p, c_long, c_void_p, c_void_p, c_long, c_int, c_int, c_void_p, c_long, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p,
                    c_void_p, c_long, c_void_p, c_int, c_long, c_int, c_int, c_int, c_int, c_void_p, c_void_p, c_float, c_void_p, c_long, c_int, c_int, c_int, c_void_p],
    "gi_route_top": [c_void_p, c_long, c_int, c_int, c_int, c_int, c_int, c_float, c_int, c_int, c_void_p, c_void_p, c_void_p],
    "gi_experts_gate_up": [c_void_p, c_int, c_long, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_int, c_void_p, c_int, c_long, c_int, c_int, c_int, c_int, c_int, c_float, c_int, c_void_p],
    "gi_route_rows": [c_void_p, c_int, c_long, c_void_p, c_int, c_long, c_int, c_int, c_int, c_int, c_int, c_int, c_float, c_int, c_int, c_void_p, c_void_p, c_void_p, c_long, c_int, c_void_p, c_long,
                      c_void_p],
    "gi_experts_place": [c_void_p, c_int, c_int, c_void_p, c_void_p, c_void_p, c_int, c_void_p],
    "gi_experts_gather": [c_void_p, c_long, c_void_p, c_void_p, c_int, c_int, c_int, c_void_p, c_long, c_int, c_void_p],
    "gi_experts_combine": [c_void_p, c_long, c_void_p, c_void_p, c_int, c_int, c_int, c_void_p, c_long, c_int, c_int, c_void_p],
    "gi_gemm_bf16_grouped": [c_void_p, c_void_p, c_void_p, c_int, c_int, c_float, c_int, c_int, c_int, c_long, c_long, c_long, c_void_p, c_long, c_void_p],
    "gi_experts_down": [c_void_p, c_int, c_long, c_void_p, c_int, c_void_p, c_void_p, c_int, c_void_p, c_long, c_int, c_int, c_int, c_int, c_int, c_void_p],
    "gi_xielu": [c_void_p, c_long, c_void_p, c_int, c_long, c_int, c_int, c_void_p, c_void_p],
    "gi_delta_prepare": [c_void_p, c_long, c_int, c_int, c_int, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_long, c_void_p, c_void_p,
                         c_int, c_int, c_int, c_int, c_int, c_float, c_int, c_void_p],
    "gi_delta_tail": [c_void_p, c_long, c_int, c_int, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_long, c_int, c_int, c_int, c_int, c_void_p],
    "gi_delta_scan": [c_void_p, c_long, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_long, c_void_p, c_long, c_int, c_int, c_int, c_int, c_void_p],
    "gi_latent_prepare": [c_void_p, c_long, c_int, c_int, c_int, c_void_p, c_void_p, c_int, c_float, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int,
                          c_void_p, c_int, c_long, c_void_p, c_int, c_long, c_int, c_int, c_void_p],
    "gi_heads_product": [c_void_p, c_long, c_void_p, c_void_p, c_int, c_long, c_long, c_int, c_int, c_int, c_int, c_void_p],
    "gi_latent_attention_bf16": [c_void_p, c_void_p, c_void_p, c_void_p, c_long, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_long, c_int, c_int, c_int, c_int, c_int, c_int,
                                 c_float, c_int, c_void_p],
    "gi_latent_attention_tiles_bf16": [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_void_p, c_int, c_long, c_int, c_int, c_int, c_int, c_int, c_float, c_void_p],
    "gi_latent_queries": [c_void_p, c_long, c_void_p, c_void_p, c_void_p, c_int, c_long, c_void_p, c_int, c_long, c_int, c_int, c_int, c_int, c_int, c_void_p],
    "gi_act_mul": [c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_float, c_void_p],
    "gi_streams_spread": [c_void_p, c_long, c_void_p, c_long, c_int, c_int, c_int, c_void_p],
    "gi_streams_norm_shift": [c_void_p, c_long, c_int, c_int, c_void_p, c_void_p, c_int, c_float, c_void_p, c_void_p, c_long, c_void_p, c_void_p, c_void_p, c_int, c_long,
                              c_int, c_int, c_void_p],
    "gi_streams_write": [c_void_p, c_long, c_int, c_int, c_void_p, c_long, c_void_p, c_void_p, c_float, c_int, c_void_p],
    "gi_streams_write_norm": [c_void_p, c_long, c_int, c_int, c_void_p, c_long, c_void_p, c_void_p, c_float, c_void_p, c_void_p, c_int, c_float, c_void_p, c_int, c_long, c_int,
                              c_void_p],
    "gi_head_gate": [c_void_p, c_int, c_long, c_void_p, c_long, c_int, c_int, c_int, c_void_p],
    "gi_add_rows_gated": [c_void_p, c_long, c_void_p, c_long, c_void_p, c_long, c_int, c_int, c_void_p],
    "gi_segments": [c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_int, c_void_p],
    "gi_mlstm_scan": [c_void_p, c_long, c_int, c_int, c_int, c_int, c_int, c_void_p, c_void_p, c_float, c_float, c_void_p, c_void_p, c_int, c_void_p,
                      c_void_p, c_long, c_void_p, c_long, c_void_p, c_int, c_int, c_int, c_void_p],
    "gi_head_norm_gate": [c_void_p, c_long, c_void_p, c_void_p, c_long, c_void_p, c_int, c_void_p, c_int, c_long, c_int, c_int, c_int, c_float, c_int, c_int, c_void_p],
    "gi_gemm_bf16": [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_float, c_int, c_int, c_int, c_long, c_long, c_long, c_void_p, c_long, c_void_p],
    "gi_attention_prompt_bf16": [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_void_p, c_int, c_long, c_int, c_int, c_int, c_int, c_int,
                                 c_float, c_int, c_void_p, c_void_p, c_int, c_void_p, c_long, c_int, c_void_p, c_void_p, c_long, c_float, c_void_p],
    "gi_attention_decode_bf16": [c_void_p, c_void_p, c_void_p, c_void_p, c_long, c_long, c_long, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                 c_long, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int, c_long, c_int, c_int, c_int, c_int, c_int,
                                 c_float, c_int, c_int, c_int, c_void_p, c_void_p, c_long, c_float, c_void_p],
    "gi_random_normal": [c_void_p, c_int, c_long, ctypes.c_ulonglong, ctypes.c_double, ctypes.c_double, c_void_p],
    "gi_probe_stream": [c_void_p, c_void_p, c_long, c_void_p, c_int, c_int, c_void_p],
    "gi_probe_mfma": [c_int, c_void_p, c_int, c_void_p],
    "gi_gemm_bf16_handing": [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_float, c_int, c_int, c_int, c_long, c_long, c_long, c_void_p, c_long,
                             c_void_p, c_int, c_float, c_void_p, c_void_p, c_long, c_void_p, c_void_p],
    "gi_gemm_bf16_qkv_rope_store": [c_void_p, c_void_p, c_int, c_int, c_int, c_long, c_long, c_void_p, c_long, c_void_p, c_int, c_float, c_void_p, c_void_p,
                                    c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_long, c_int, c_int, c_int, c_int, c_void_p],
    "gi_argmax": [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_long, c_void_p],
    "gi_sample_temperature": [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_long, c_void_p],
    "gi_sample_filtered": [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_long, c_void_p],
}

_lib = None


def lib():
    global _lib
    if _lib is None:
        l = library.load()
        for name, sig in _SIGNATURES.items():
            fn = getattr(l, name)
            fn.argtypes = sig
            fn.restype = c_int
        l.gi_argmax_chunks.argtypes = [c_int]
        l.gi_argmax_chunks.restype = c_int
        l.gi_sample_filtered_histogram_bytes.argtypes = []
        l.gi_sample_filtered_histogram_bytes.restype = c_int
        l.gi_attention_exact_max_head_size.argtypes = []
        l.gi_attention_exact_max_head_size.restype = c_int
        l.gi_attention_decode_workgroups_per_unit.argtypes = [c_int, c_int, c_int, c_int]
        l.gi_attention_decode_workgroups_per_unit.restype = c_int
        l.gi_attention_bf16_supports.argtypes = [c_int, c_int, c_int]
        l.gi_attention_bf16_supports.restype = c_int
        l.gi_gemm_bf16_scratch_floats.argtypes = [c_int, c_int, c_int]
        l.gi_gemm_bf16_scratch_floats.restype = c_long
        l.gi_gemm_bf16_norm_parts.argtypes = [c_int, c_int, c_int]
        l.gi_gemm_bf16_norm_parts.restype = c_int
        l.gi_gemm_bf16_takes_norm.argtypes = [c_int, c_int, c_int, c_int]
        l.gi_gemm_bf16_takes_norm.restype = c_int
        l.gi_gemm_bf16_qkv_rope_store_takes.argtypes = [c_int, c_int, c_int, c_int]
        l.gi_gemm_bf16_qkv_rope_store_takes.restype = c_int
        l.gi_compute_units.argtypes = []
        l.gi_compute_units.restype = c_int
        l.gi_gemm_bf16_qkv_rope_store_max_parts.argtypes = [c_int, c_int, c_int]
        l.gi_gemm_bf16_qkv_rope_store_max_parts.restype = c_int
        l.gi_mlstm_state_floats.argtypes = [c_int, c_int, c_int]
        l.gi_mlstm_state_floats.restype = c_long
        l.gi_mlstm_max_key_dim.argtypes = []
        l.gi_mlstm_max_key_dim.restype = c_int
        l.gi_latent_attention_supports.argtypes = [c_int, c_int, c_int]
        l.gi_latent_attention_supports.restype = c_int
        l.gi_latent_attention_tiles_supports.argtypes = [c_int, c_int, c_int, c_int]
        l.gi_latent_attention_tiles_supports.restype = c_int
        l.gi_latent_attention_tiles_prepare.argtypes = []
        l.gi_latent_attention_tiles_prepare.restype = c_int
        l.gi_streams_write_norm_takes.argtypes = [c_int, c_int]
        l.gi_streams_write_norm_takes.restype = c_int
        l.gi_streams_max.argtypes = []
        l.gi_streams_max.restype = c_int
        l.gi_probe_mfma_flops.argtypes = [c_int, c_int]
        l.gi_probe_mfma_flops.restype = c_long
        _lib = l
    return _lib


_FUNCTIONS = {}


def _call(name, *args):
    fn = _FUNCTIONS.get(name)
    if fn is None:
        fn = _FUNCTIONS[name] = getattr(lib(), name)
    if _profile is not None:
        return _profile.timed(name, fn, args)
    if fn(*args) != 0:
        raise KernelError(lib().gi_last_error().decode())


_PROFILE_LABEL = {"gi_gemm_bf16_handing": "gemm_bf16", "gi_gemm_bf16_qkv_rope_store": "gemm_bf16"}        # the same products, with a norm's share on top


class KernelProfile:
    """Time per kernel entry point, with the device waited for before and after every call (so the times add up, and
    a step takes longer than it does unobserved).  What the reference's device model reports with --profile
    (src/gpu/gpu_transformer.cpp:178-224), by entry point and weight shape instead of a fixed list of sections.
    Matrix products are kept apart by the weight's shape, which tells the projections from one another, and count the
    weight bytes they read."""

    def __init__(self):
        self.seconds, self.calls, self.weight_bytes = {}, {}, {}
        self.note = None                        # (label suffix, weight bytes) of the product about to be launched

    def timed(self, name, fn, args):
        import time
        label, nbytes = _PROFILE_LABEL.get(name, name[3:]), 0
        if self.note is not None:
            label, nbytes = f"{label} {self.note[0]}", self.note[1]
            self.note = None
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        rc = fn(*args)
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        if rc != 0:
            raise KernelError(lib().gi_last_error().decode())
        self.seconds[label] = self.seconds.get(label, 0.0) + dt
        self.calls[label] = self.calls.get(label, 0) + 1
        self.weight_bytes[label] = self.weight_bytes.get(label, 0) + nbytes

    def report(self, positions: int, steps: int, wall_seconds: float) -> str:
        if not self.seconds or positions <= 0:
            return ""
        inside = sum(self.seconds.values())
        lines = [f"device profile: {positions} positions in {steps} steps, {wall_seconds * 1e3 / positions:.3f} ms per position "
                 "(the device waits before and after every kernel)",
                 f"  {'kernel':<34} {'calls':>8} {'ms/position':>12} {'share':>7} {'weights GB/s':>13}"]
        for label in sorted(self.seconds, key=self.seconds.get, reverse=True):
            sec, nbytes = self.seconds[label], self.weight_bytes[label]
            rate = f"{nbytes / sec / 1e9:.1f}" if nbytes and sec > 0 else ""
            lines.append(f"  {label:<34} {self.calls[label]:>8} {sec * 1e3 / positions:>12.4f} {100 * sec / wall_seconds:>6.1f}% {rate:>13}")
        rest = max(wall_seconds - inside, 0.0)
        lines.append(f"  {'host work, uploads, downloads':<34} {'':>8} {rest * 1e3 / positions:>12.4f} {100 * rest / wall_seconds:>6.1f}%")
        return "\n".join(lines) + "\n"


_profile: Optional[KernelProfile] = None


def set_profiling(on: bool) -> Optional[KernelProfile]:
    """Switches the per-kernel timing on (a fresh KernelProfile, which is returned) or off.  While it is on, steps are
    not replayed from captured graphs: a replay has no kernel boundaries to wait at."""
    global _profile
    _profile = KernelProfile() if on else None
    return _profile


def profiling() -> bool:
    return _profile is not None


# The current stream's handle, asked for at every launch (it changes under graph capture).  torch's
# public way costs several microseconds a call, and a step makes over a hundred launches.
_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)
_raw_device = getattr(torch._C, "_cuda_getDevice", None)


def _stream():
    if _raw_stream is not None and _raw_device is not None:
        return _raw_stream(_raw_device())
    return torch.cuda.current_stream().cuda_stream


def _code(t: torch.Tensor, what: str) -> int:
    try:
        return _CODE[t.dtype]
    except KeyError:
        raise KernelError(f"{what} has dtype {t.dtype}; float32 or bfloat16 is needed") from None


def _dev(*tensors):
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise KernelError("kernel operands must lie in device memory")


def _i32(t, what, n=None):
    if not (t.dtype == torch.int32 and t.is_contiguous()):
        raise KernelError(f"{what} must be a contiguous int32 tensor")
    if n is not None:
        if not (t.numel() >= n):
            raise KernelError(f"{what} holds {t.numel()} entries, {n} are needed")


def _ptr(t):
    return None if t is None else t.data_ptr()


def device_arch() -> str:
    buf = ctypes.create_string_buffer(64)
    l = lib()
    if l.gi_device_arch(buf, 64) != 0:
        raise KernelError(l.gi_last_error().decode())
    return buf.value.decode()


# ------------------------------------------------------------------------------------------------
def embed(table, tokens, out):
    """out[t, :] = table[tokens[t], :] widened to float32."""
    _dev(table, tokens, out)
    n, dim = out.shape
    if not (table.dim() == 2 and table.shape[1] == dim and table.is_contiguous()):
        raise KernelError("embed: table must be [vocab, dim], contiguous")
    if not (out.dtype == torch.float32 and out.is_contiguous()):
        raise KernelError("embed: out must be contiguous float32")
    _i32(tokens, "embed: tokens", n)
    _call("gi_embed", table.data_ptr(), _code(table, "embed: table"), tokens.data_ptr(), out.data_ptr(), n, dim, _stream())
    return out


def embed_handing(table, tokens, out, g, scaled, squares):
    """`embed`, and on the way the first half of an RMS norm of the rows for a product that finishes it (`gemm_bf16(..., norm_in=...)`):
    scaled = bfloat16(g * out) and squares [n, 1] = the rows' sums of out^2."""
    _dev(table, tokens, out, g, scaled, squares)
    n, dim = out.shape
    if not (table.dim() == 2 and table.shape[1] == dim and table.is_contiguous() and out.dtype == torch.float32 and out.is_contiguous()):
        raise KernelError("embed: table must be [vocab, dim], contiguous, and out contiguous float32")
    if not (g.dtype == torch.float32 and g.is_contiguous() and g.numel() == dim and scaled.dtype == torch.bfloat16 and scaled.shape == (n, dim)
            and scaled.is_contiguous() and squares.dtype == torch.float32 and squares.is_contiguous() and squares.shape == (n, 1)):
        raise KernelError("embed: handing a norm on needs float32 weights [dim], bfloat16 [n, dim] for the scaled rows and float32 [n, 1] for the sums of squares")
    _i32(tokens, "embed: tokens", n)
    _call("gi_embed_handing", table.data_ptr(), _code(table, "embed: table"), tokens.data_ptr(), out.data_ptr(), n, dim, g.data_ptr(), scaled.data_ptr(),
          squares.data_ptr(), _stream())
    return out


def rmsnorm_can_gather(x, weight, out) -> bool:
    dim = x.shape[1]
    return (dim % 4 == 0 and dim <= 4096 and x.stride(0) % 4 == 0 and out.stride(0) % 4 == 0 and x.data_ptr() % 16 == 0
            and weight.data_ptr() % 16 == 0 and out.data_ptr() % 16 == 0)


def rmsnorm(x, weight, eps, out, rows=None):
    """out = weight * (x * rsqrt(mean(x^2) + eps)) per row; x float32 [n, dim].  rows: int32 indices, out[i] = norm(x[rows[i]])."""
    _dev(x, weight, out, rows)
    dim = x.shape[1]
    n = x.shape[0] if rows is None else rows.numel()
    if not (x.dtype == torch.float32 and x.stride(1) == 1):
        raise KernelError("rmsnorm: x must be float32 with unit inner stride")
    if not (out.shape == (n, dim) and out.stride(1) == 1):
        raise KernelError("rmsnorm: out must be [rows, dim] with unit inner stride")
    if not (weight.shape == (dim,) and weight.is_contiguous()):
        raise KernelError("rmsnorm: weight must be [dim]")
    if rows is not None:
        _i32(rows, "rmsnorm: rows", n)
        if not (rmsnorm_can_gather(x, weight, out)):
            raise KernelError("rmsnorm: these operands cannot be gathered in the kernel")
    _call("gi_rmsnorm", x.data_ptr(), _ptr(rows), weight.data_ptr(), _code(weight, "rmsnorm: weight"), out.data_ptr(), _code(out, "rmsnorm: out"),
          n, dim, float(eps), x.stride(0), out.stride(0), _stream())
    return out


def rope_cos_sin(positions, inv_freq, cos_out, sin_out, magnitude: float = 1.0):
    """magnitude * cos/sin of positions[t] * inv_freq[k] with 64-bit angles; outputs float32 [n, half]."""
    _dev(positions, inv_freq, cos_out, sin_out)
    n, half = cos_out.shape
    _i32(positions, "rope_cos_sin: positions", n)
    if not (inv_freq.dtype == torch.float64 and inv_freq.shape == (half,) and inv_freq.is_contiguous()):
        raise KernelError("rope_cos_sin: inv_freq must be float64 [half]")
    for t in (cos_out, sin_out):
        if not (t.dtype == torch.float32 and t.is_contiguous() and t.shape == (n, half)):
            raise KernelError("rope_cos_sin: outputs must be float32 [n, half]")
    _call("gi_rope_cos_sin", positions.data_ptr(), inv_freq.data_ptr(), cos_out.data_ptr(), sin_out.data_ptr(), n, half, float(magnitude), _stream())


def _check_cache(cache, table, page_size, n_kv, hd, what):
    # the last two axes of the value half hold [hd][place]: values are stored transposed
    if not (cache.dim() == 5 and tuple(cache.shape[1:]) == (2, n_kv, page_size, hd) and cache.is_contiguous()):
        raise KernelError( f"{what}: the cache must be [pages, 2, {n_kv}, {page_size}, {hd}], contiguous; it is {tuple(cache.shape)}")
    if not (table.dim() == 2 and table.dtype == torch.int32 and table.stride(1) == 1):
        raise KernelError(f"{what}: the page table must be int32 [slots, pages]")


def rope_store(q, k, v, cos, sin, positions, slots, table, q_out, cache, n_heads, n_kv, hd):
    """Rotates q into q_out and, if k is given, rotates k and writes k and v into the cache pages.
    q, k, v are float32 views [n, heads*hd] with unit inner stride (columns of one product are fine)."""
    _dev(q, k, v, cos, sin, positions, slots, table, q_out, cache)
    n = q.shape[0]
    if not (q.dtype == torch.float32 and q.shape[1] == n_heads * hd and q.stride(1) == 1):
        raise KernelError("rope_store: q must be float32 [n, heads*hd]")
    if not (q_out.shape == (n, n_heads * hd) and q_out.is_contiguous()):
        raise KernelError("rope_store: q_out must be [n, heads*hd], contiguous")
    if cos is not None:
        for t in (cos, sin):
            if not (t.dtype == torch.float32 and t.shape == (n, hd // 2) and t.is_contiguous()):
                raise KernelError("rope_store: cos/sin must be float32 [n, hd/2]")
    page_size = page_stride = 0
    cache_code = _code(q_out, "rope_store: q_out")
    if k is not None:
        for t, name in ((k, "k"), (v, "v")):
            if not (t.dtype == torch.float32 and t.shape == (n, n_kv * hd) and t.stride(1) == 1):
                raise KernelError(f"rope_store: {name} must be float32 [n, kv_heads*hd]")
        page_size = cache.shape[3]
        _check_cache(cache, table, page_size, n_kv, hd, "rope_store")
        page_stride = cache.stride(0)
        cache_code = _code(cache, "rope_store: cache")
        _i32(positions, "rope_store: positions", n)
        _i32(slots, "rope_store: slots", n)
    _call("gi_rope_store", q.data_ptr(), _ptr(k), _ptr(v), q.stride(0), k.stride(0) if k is not None else 0,
          v.stride(0) if v is not None else 0, _ptr(cos), _ptr(sin), _ptr(positions), _ptr(slots),
          _ptr(table) if k is not None else None, table.stride(0) if k is not None else 0, q_out.data_ptr(),
          _code(q_out, "rope_store: q_out"), _ptr(cache) if k is not None else None, cache_code, page_stride, page_size,
          n, n_heads, n_kv, hd, _stream())


def silu_mul(gate_up, out):
    """out[t, i] = silu(gate_up[t, i]) * gate_up[t, inter + i]."""
    _dev(gate_up, out)
    n, inter = out.shape
    if not (gate_up.dtype == torch.float32 and gate_up.shape == (n, 2 * inter) and gate_up.is_contiguous()):
        raise KernelError("silu_mul: gate_up must be float32 [n, 2*inter]")
    if not (out.is_contiguous()):
        raise KernelError("silu_mul: out must be contiguous")
    _call("gi_silu_mul", gate_up.data_ptr(), out.data_ptr(), _code(out, "silu_mul: out"), n, inter, _stream())
    return out


def gather_rows(x, rows, out):
    _dev(x, rows, out)
    k, dim = out.shape
    if not (x.dtype == torch.float32 and x.is_contiguous() and x.shape[1] == dim):
        raise KernelError("gather_rows: x must be contiguous float32 [n, dim]")
    if not (out.dtype == torch.float32 and out.is_contiguous()):
        raise KernelError("gather_rows: out must be contiguous float32")
    _i32(rows, "gather_rows: rows", k)
    _call("gi_gather_rows", x.data_ptr(), rows.data_ptr(), out.data_ptr(), k, dim, _stream())
    return out


def _rows_in_place(name, x, c):
    _dev(x)
    if not (x.dim() == 2 and x.dtype == torch.float32 and x.stride(1) == 1):
        raise KernelError(f"{name}: x must be float32 [n, dim] with unit inner stride")
    _call("gi_" + name, x.data_ptr(), x.shape[0], x.shape[1], x.stride(0), float(c), _stream())
    return x


def scale_rows(x, factor):
    """x *= factor, in place."""
    return _rows_in_place("scale_rows", x, factor)


def softcap_rows(x, cap):
    """x = cap * tanh(x / cap), in place."""
    return _rows_in_place("softcap_rows", x, cap)


def random_normal(out, key: int, offset: float, scale: float):
    """out[i] = offset + scale * z_i, z_i the standard normal number that (key, i) give (`weights.random_init` states the formula);
    out is a contiguous float32 or bfloat16 tensor of any shape, filled in the order of its memory."""
    _dev(out)
    if not out.is_contiguous():
        raise KernelError("random_normal: out must be contiguous")
    _call("gi_random_normal", out.data_ptr(), _code(out, "random_normal: out"), out.numel(), int(key) & 0xFFFFFFFFFFFFFFFF, float(offset), float(scale), _stream())
    return out


def gemm_exact(a, w, out, accumulate=False):
    """out (=|+=) a @ w.T in 32-bit arithmetic with one summation order for every batch size."""
    _dev(a, w, out)
    m, k = a.shape
    n = w.shape[0]
    if not (w.shape == (n, k)):
        raise KernelError(f"gemm: weight is {tuple(w.shape)}, activations are {tuple(a.shape)}")
    if not (out.shape == (m, n)):
        raise KernelError(f"gemm: out is {tuple(out.shape)}, ({m}, {n}) is needed")
    if not (a.stride(1) == 1 and w.stride(1) == 1 and out.stride(1) == 1):
        raise KernelError("gemm: operands need unit inner stride")
    if _profile is not None:
        _profile.note = (f"{n}x{k}", n * k * w.element_size())
    _call("gi_gemm_exact", a.data_ptr(), _code(a, "gemm: a"), w.data_ptr(), _code(w, "gemm: w"), out.data_ptr(), _code(out, "gemm: out"),
          1 if accumulate else 0, m, n, k, a.stride(0), w.stride(0), out.stride(0), _stream())
    return out


def attention_max_head_size() -> int:
    """The largest head the attention kernels take (the exact kernel's limit; the matrix-core kernels take fewer sizes and
    leave the others to it)."""
    return lib().gi_attention_exact_max_head_size()


def _check_paged(cache, table, what):
    """A layer's pages as the general kernels take them: [pages, ...] with whole pages contiguous, whatever the axes behind."""
    if not (cache.dim() >= 2 and cache[0].is_contiguous()):
        raise KernelError(f"{what}: the pages must each be contiguous")
    if not (table.dim() == 2 and table.dtype == torch.int32 and table.stride(1) == 1):
        raise KernelError(f"{what}: the page table must be int32 [slots, pages]")


def attention_exact(q, cache, out, positions, slots, table, n_heads, n_kv, hd, window=None, scale=None, *, page_size=None, value_dim=None,
                    chunk=None, sinks=None, gate=None, cap=None):
    """Each row attends over its request's cached keys up to its own position, no further back than `window` positions and not
    beyond the start of its own chunk of `chunk` positions.  value_dim: channels of a value head (hd if not given); sinks:
    float32 [heads], a score per head that joins the softmax's denominator only; gate: float32 [n, >= heads] (unit inner
    stride), head h's output is multiplied by sigmoid(gate[t, h]); cap: a scaled score s becomes cap * tanh(s / cap)."""
    _dev(q, cache, out, positions, slots, table, sinks, gate)
    if cap is not None and not cap > 0:
        raise KernelError("attention: the scores' cap must be positive")
    n = q.shape[0]
    vd = int(value_dim or hd)
    if not (q.shape == (n, n_heads * hd) and q.is_contiguous() and out.shape == (n, n_heads * vd) and out.is_contiguous()):
        raise KernelError("attention: q must be [n, heads*hd] and out [n, heads*vd], contiguous")
    if page_size is None:
        page_size = cache.shape[3]
        _check_cache(cache, table, page_size, n_kv, hd, "attention")
    else:
        _check_paged(cache, table, "attention")
    if sinks is not None and not (sinks.dtype == torch.float32 and sinks.is_contiguous() and sinks.numel() == n_heads):
        raise KernelError("attention: sinks must be float32 [heads]")
    if gate is not None and not (gate.dtype == torch.float32 and gate.dim() == 2 and gate.shape[0] == n and gate.shape[1] >= n_heads and gate.stride(1) == 1):
        raise KernelError("attention: the heads' gates must be float32 [n, heads] with unit inner stride")
    _i32(positions, "attention: positions", n)
    _i32(slots, "attention: slots", n)
    _call("gi_attention_exact", q.data_ptr(), _code(q, "attention: q"), cache.data_ptr(), _code(cache, "attention: cache"), out.data_ptr(),
          _code(out, "attention: out"), positions.data_ptr(), slots.data_ptr(), table.data_ptr(), table.stride(0), cache.stride(0),
          page_size, n, n_heads, n_kv, hd, vd, int(window or 0), int(chunk or 0), float(scale if scale is not None else hd ** -0.5),
          float(cap or 0.0), _ptr(sinks), _ptr(gate), gate.stride(0) if gate is not None else 0, _stream())
    return out


def rmsnorm_add(y, weight, eps, x):
    """x += weight * (y * rsqrt(mean(y^2) + eps)) per row; x and y float32 [n, dim]."""
    _dev(y, weight, x)
    n, dim = x.shape
    if not (x.dtype == torch.float32 and y.dtype == torch.float32 and y.shape == (n, dim) and x.stride(1) == 1 and y.stride(1) == 1):
        raise KernelError("rmsnorm_add: x and y must be float32 [n, dim] with unit inner stride")
    if not (weight.shape == (dim,) and weight.is_contiguous()):
        raise KernelError("rmsnorm_add: weight must be [dim]")
    _call("gi_rmsnorm_add", y.data_ptr(), weight.data_ptr(), _code(weight, "rmsnorm_add: weight"), x.data_ptr(), n, dim, float(eps), y.stride(0), x.stride(0), _stream())
    return x


def rmsnorm_add_norm(y, weight, eps, x, next_weight, next_eps, out):
    """x += weight * norm(y), and out = next_weight * norm(x) of the rows so made (the norm that reads x next), in one kernel;
    x and y float32 [n, dim], out [n, dim] float32 or bfloat16, the two weights of one dtype."""
    _dev(y, weight, x, next_weight, out)
    n, dim = x.shape
    if not (x.dtype == torch.float32 and y.dtype == torch.float32 and y.shape == (n, dim) and out.shape == (n, dim) and x.stride(1) == 1 and y.stride(1) == 1 and out.stride(1) == 1):
        raise KernelError("rmsnorm_add_norm: x and y must be float32 [n, dim] and out [n, dim], with unit inner stride")
    if not (weight.shape == (dim,) and weight.is_contiguous() and next_weight.shape == (dim,) and next_weight.is_contiguous() and weight.dtype == next_weight.dtype):
        raise KernelError("rmsnorm_add_norm: the weights must be [dim], of one dtype")
    _call("gi_rmsnorm_add_norm", y.data_ptr(), weight.data_ptr(), next_weight.data_ptr(), _code(weight, "rmsnorm_add_norm: weight"), x.data_ptr(), out.data_ptr(),
          _code(out, "rmsnorm_add_norm: out"), n, dim, float(eps), float(next_eps), y.stride(0), x.stride(0), out.stride(0), _stream())
    return out


def norm_rope_store(q, k, v, q_norm, k_norm, eps, cos, sin, rotary_dim, positions, slots, table, q_out, cache, page_size, n_heads, n_kv, hd, vd,
                    biases=None, blend=None, keep=None, neighbours=False, unit_rms=False, norm_last=False, v_scale=1.0, norm_all=False):
    """The general form of `rope_store`: every query and key head is first RMS-normed with q_norm / k_norm [hd] (None: not), then
    the pairs (i, i + rotary_dim/2) of its first rotary_dim channels are turned (cos, sin float32 [n, rotary_dim/2]; None: not);
    queries go to q_out, keys and the values (vd channels a head) into the cache's pages.  k None: the pages are another layer's.
    biases = (q_bias, k_bias, v_bias): float32 vectors added to the products first (each may be None).  blend = (other, weight):
    the values that go into the pages are (1 - weight) v + weight other, other float32 [n, kv_heads*vd] (another layer's values of
    the same rows), weight one float32 number on the device.  keep: float32 [n, kv_heads*vd], gets this layer's values (with
    their bias, before any blending).  neighbours: the pairs turned are (2i, 2i + 1).  unit_rms: every query and key head is divided
    by its root mean square (eps inside the root), without weights.  norm_last: the heads' norm comes behind the rotation.
    v_scale: multiplies the values on their way into the pages.  norm_all: q_norm is [heads*hd] and k_norm [kv_heads*hd], and the norm is
    taken over all heads of a projection at once."""
    if unit_rms and (q_norm is not None or k_norm is not None):
        raise KernelError("norm_rope_store: heads divided by their root mean square have no norm weights")
    _dev(q, k, v, q_norm, k_norm, cos, sin, positions, slots, table, q_out, cache)
    q_bias, k_bias, v_bias = biases if biases is not None else (None, None, None)
    other, weight = blend if blend is not None else (None, None)
    _dev(q_bias, k_bias, v_bias, other, weight, keep)
    for b, width, name in ((q_bias, n_heads * hd, "q"), (k_bias, n_kv * hd, "k"), (v_bias, n_kv * vd, "v")):
        if b is not None and not (b.dtype == torch.float32 and b.is_contiguous() and b.numel() == width):
            raise KernelError(f"norm_rope_store: the {name} bias must be float32 [{width}]")
    for rows, name in ((other, "blended"), (keep, "kept")):
        if rows is not None and not (k is not None and rows.dtype == torch.float32 and rows.dim() == 2 and rows.shape == (q.shape[0], n_kv * vd) and rows.stride(1) == 1):
            raise KernelError(f"norm_rope_store: the {name} values must be float32 [n, kv_heads*vd], beside values of the layer's own")
    if other is not None and not (weight is not None and weight.dtype == torch.float32 and weight.numel() == 1):
        raise KernelError("norm_rope_store: the blend's weight must be one float32 number on the device")
    if k is None and (k_bias is not None or v_bias is not None):
        raise KernelError("norm_rope_store: biases on keys and values need keys and values")
    n = q.shape[0]
    if not (q.dtype == torch.float32 and q.shape[1] == n_heads * hd and q.stride(1) == 1 and q_out.shape == (n, n_heads * hd) and q_out.is_contiguous()):
        raise KernelError("norm_rope_store: q must be float32 [n, heads*hd] and q_out [n, heads*hd], contiguous")
    half = int(rotary_dim) // 2 if cos is not None else 0
    if cos is not None:
        for t in (cos, sin):
            if not (t.dtype == torch.float32 and t.shape == (n, half) and t.is_contiguous()):
                raise KernelError("norm_rope_store: cos/sin must be float32 [n, rotary_dim/2]")
    norm_code = None
    for w, heads in ((q_norm, n_heads), (k_norm, n_kv)):
        if w is not None:
            if not (w.shape == ((heads * hd,) if norm_all else (hd,)) and w.is_contiguous() and (norm_code is None or norm_code == _code(w, "norm_rope_store: norm"))):
                raise KernelError("norm_rope_store: the norm weights must be [hd] (over all heads at once: [heads*hd]), of one dtype")
            norm_code = _code(w, "norm_rope_store: norm")
    if k is not None:
        if not (k.dtype == torch.float32 and k.shape == (n, n_kv * hd) and k.stride(1) == 1 and v.dtype == torch.float32 and v.shape == (n, n_kv * vd) and v.stride(1) == 1):
            raise KernelError("norm_rope_store: k must be float32 [n, kv_heads*hd] and v [n, kv_heads*vd]")
        _check_paged(cache, table, "norm_rope_store")
        if cache.stride(0) < n_kv * page_size * (hd + vd):
            raise KernelError("norm_rope_store: the pages are too small for these heads")
    _i32(positions, "norm_rope_store: positions", n)
    _i32(slots, "norm_rope_store: slots", n)
    cache_code = _code(cache, "norm_rope_store: cache") if k is not None else _code(q_out, "norm_rope_store: q_out")
    rows_r = torch.empty((n, 2), dtype=torch.float32, device=q.device) if norm_all else None          # the rows' 1 / sqrt(mean square + eps), made by a kernel of its own first
    _call("gi_norm_rope_store", q.data_ptr(), _ptr(k), _ptr(v), q.stride(0), k.stride(0) if k is not None else 0, v.stride(0) if v is not None else 0,
          _ptr(q_norm), _ptr(k_norm), norm_code if norm_code is not None else F32, float(eps), _ptr(cos), _ptr(sin), 2 * half, positions.data_ptr(),
          slots.data_ptr(), _ptr(table) if k is not None else None, table.stride(0) if k is not None else 0, q_out.data_ptr(),
          _code(q_out, "norm_rope_store: q_out"), _ptr(cache) if k is not None else None, cache_code, cache.stride(0) if k is not None else 0,
          int(page_size), n, n_heads, n_kv, hd, vd, _ptr(q_bias), _ptr(k_bias), _ptr(v_bias), _ptr(other), other.stride(0) if other is not None else 0,
          _ptr(weight), _ptr(keep), keep.stride(0) if keep is not None else 0, (1 if neighbours else 0) | (2 if unit_rms else 0) | (4 if norm_last else 0) | (8 if norm_all else 0), float(v_scale),
          _ptr(rows_r), _stream())


def xielu(x, out, params):
    """out[t, i] = a z^2 + z/2 for z = x[t, i] > 0, else b (exp(z) - 1 - z) + z/2, with a = softplus(params[0]), b = 1/2 + softplus(params[1]);
    x float32 [n, columns] and out [n, columns] (unit inner stride), params two float32 numbers on the device."""
    _dev(x, out, params)
    n, inter = out.shape
    if not (x.dtype == torch.float32 and x.shape == (n, inter) and x.stride(1) == 1 and out.stride(1) == 1):
        raise KernelError("xielu: x must be float32 [n, columns] and out [n, columns], with unit inner stride")
    if not (params.dtype == torch.float32 and params.is_contiguous() and params.numel() == 2):
        raise KernelError("xielu: the two parameters must be float32 [2]")
    _call("gi_xielu", x.data_ptr(), x.stride(0), out.data_ptr(), _code(out, "xielu: out"), out.stride(0), n, inter, params.data_ptr(), _stream())
    return out


ACTIVATIONS = {"silu": 0, "gelu_tanh": 1, "swish_clamped": 2}
# "swish_clamped" takes a number, `limit`: both halves are clamped first, g <- min(g, limit), u <- clamp(u, -limit, limit), and the
# result is g * sigmoid(1.702 g) * (u + 1).
FUSED_GATE_ACTIVATIONS = ("silu", "gelu_tanh", "swish_clamped")        # those the matrix-core products apply in their own last step


def act_mul(gate_up, out, activation="silu", limit=0.0):
    """out[t, i] = act(gate_up[t, i]) * gate_up[t, inter + i]; act "silu", "gelu_tanh" (the tanh form of GELU), or the clamped form
    "swish_clamped" with its `limit` (see `ACTIVATIONS`)."""
    _dev(gate_up, out)
    n, inter = out.shape
    if activation not in ACTIVATIONS:
        raise KernelError(f"act_mul: unknown activation {activation!r}; known: {', '.join(ACTIVATIONS)}")
    if not (gate_up.dtype == torch.float32 and gate_up.shape == (n, 2 * inter) and gate_up.is_contiguous() and out.is_contiguous()):
        raise KernelError("act_mul: gate_up must be float32 [n, 2*inter], out contiguous")
    _call("gi_act_mul", gate_up.data_ptr(), out.data_ptr(), _code(out, "act_mul: out"), n, inter, ACTIVATIONS[activation], float(limit), _stream())
    return out


def segments(ctx):
    """(first row, number of rows) of every request of the step as int32 device tensors [requests], made on the device from the
    rows' slots and positions (a run of rows ends where the slot changes or the position does not follow): nothing of it comes
    from the host but the number of requests, so a captured pass may use it.  Made once per step, kept in ctx.memo."""
    if "segments" not in ctx.memo:
        n_segs = len(ctx.seg_len)
        both = torch.empty((2, n_segs), dtype=torch.int32, device=ctx.device)
        _i32(ctx.row_slot, "segments: slots", ctx.n_rows)
        _i32(ctx.row_pos, "segments: positions", ctx.n_rows)
        _call("gi_segments", ctx.row_slot.data_ptr(), ctx.row_pos.data_ptr(), ctx.n_rows, both[0].data_ptr(), both[1].data_ptr(), n_segs, _stream())
        ctx.memo["segments"] = (both[0], both[1])
    return ctx.memo["segments"]


def mlstm_state_floats(n_heads, dk, dv) -> int:
    """32-bit numbers of one request's matrix memories, as `mlstm_scan` lays them out for itself: per head and tile of three value
    channels, [dk][4] (three columns of S and the normaliser n) and m padded to four numbers (the library's `gi_mlstm_state_floats`
    says the same; this one needs no library, so that a cache can be planned without one)."""
    return n_heads * (-(-dv // 3)) * (dk * 4 + 4)


MLSTM_MAX_KEY_DIM = 512


def mlstm_max_key_dim() -> int:
    return MLSTM_MAX_KEY_DIM


def mlstm_scan(proj, offsets, i_bias, f_bias, cap, q_scale, seg_start, seg_len, row_slot, state, out, den, n_heads, dk, dv):
    """The matrix memories of a step's requests stepped over the requests' rows, in order (csrc/recurrent.hip states the recurrence).
    proj: float32 [n, columns]; offsets = the first columns of (q, k, v, i, f) in it; out: float32 [n, heads*dv] gets the heads'
    sums S^T q and den: float32 [n, heads] what each head's are to be divided by (the readout is out / den: `head_norm_gate`
    divides on its way); state: float32 [slots, mlstm_state_floats], read at each request's first row of the step and written
    after its last."""
    _dev(proj, i_bias, f_bias, seg_start, seg_len, row_slot, state, out, den)
    if not (den.dtype == torch.float32 and den.shape == (proj.shape[0], n_heads) and den.is_contiguous()):
        raise KernelError("mlstm_scan: den must be float32 [n, heads], contiguous")
    n = proj.shape[0]
    q_off, k_off, v_off, i_off, f_off = (int(o) for o in offsets)
    if not (proj.dtype == torch.float32 and proj.dim() == 2 and proj.stride(1) == 1 and out.dtype == torch.float32 and out.shape == (n, n_heads * dv) and out.stride(1) == 1):
        raise KernelError("mlstm_scan: proj must be float32 [n, columns] and out float32 [n, heads*dv]")
    if max(q_off + n_heads * dk, k_off + n_heads * dk, v_off + n_heads * dv, i_off + n_heads, f_off + n_heads) > proj.shape[1] or min(q_off, k_off, v_off, i_off, f_off) < 0:
        raise KernelError("mlstm_scan: the columns named lie outside proj")
    for t, name in ((i_bias, "i_bias"), (f_bias, "f_bias")):
        if not (t.dtype == torch.float32 and t.is_contiguous() and t.numel() == n_heads):
            raise KernelError(f"mlstm_scan: {name} must be float32 [heads]")
    n_segs = seg_start.numel()
    _i32(seg_start, "mlstm_scan: seg_start", n_segs)
    _i32(seg_len, "mlstm_scan: seg_len", n_segs)
    _i32(row_slot, "mlstm_scan: slots", n)
    if not (state.dtype == torch.float32 and state.dim() == 2 and state.stride(1) == 1 and state.shape[1] >= mlstm_state_floats(n_heads, dk, dv)):
        raise KernelError("mlstm_scan: state must be float32 [slots, mlstm_state_floats]")
    _call("gi_mlstm_scan", proj.data_ptr(), proj.stride(0), q_off, k_off, v_off, i_off, f_off, i_bias.data_ptr(), f_bias.data_ptr(), float(cap), float(q_scale),
          seg_start.data_ptr(), seg_len.data_ptr(), n_segs, row_slot.data_ptr(), state.data_ptr(), state.stride(0), out.data_ptr(), out.stride(0),
          den.data_ptr(), n_heads, dk, dv, _stream())
    return out


GATES = {"sigmoid": 0, "silu": 1}


def head_norm_gate(o, gate, weight, eps, out, n_heads, dv, den=None, gate_activation="sigmoid"):
    """out[t, h*dv + d] = weight[h*dv + d] * o[t, h, d] * rsqrt(mean over d of o[t, h, :]^2 + eps) * sigmoid(gate[t, h*dv + d]);
    o and gate float32 [n, heads*dv] (unit inner stride: columns of a wider product are fine).  den: float32 [n, heads]; o is
    then what the rows hold divided by den[t, h].  weight may be [dv] instead: one for all heads.  gate_activation "silu": the
    last factor is gate * sigmoid(gate)."""
    _dev(o, gate, weight, out, den)
    n = o.shape[0]
    if den is not None and not (den.dtype == torch.float32 and den.shape == (n, n_heads) and den.is_contiguous()):
        raise KernelError("head_norm_gate: den must be float32 [n, heads], contiguous")
    for t, name in ((o, "o"), (gate, "gate")):
        if not (t.dtype == torch.float32 and t.shape == (n, n_heads * dv) and t.stride(1) == 1):
            raise KernelError(f"head_norm_gate: {name} must be float32 [n, heads*dv]")
    shared = weight.numel() == dv and n_heads > 1
    if not (weight.numel() in (n_heads * dv, dv) and weight.is_contiguous() and out.shape == (n, n_heads * dv) and out.stride(1) == 1):
        raise KernelError("head_norm_gate: weight must be [heads*dv] or [dv], and out [n, heads*dv]")
    if gate_activation not in GATES:
        raise KernelError(f"head_norm_gate: unknown gate {gate_activation!r}; known: {', '.join(GATES)}")
    _call("gi_head_norm_gate", o.data_ptr(), o.stride(0), _ptr(den), gate.data_ptr(), gate.stride(0), weight.data_ptr(), _code(weight, "head_norm_gate: weight"),
          out.data_ptr(), _code(out, "head_norm_gate: out"), out.stride(0), n, n_heads, dv, float(eps), 1 if shared else 0, GATES[gate_activation], _stream())
    return out


# ------------------------------------------------------------------------------------------------ the gated delta rule
DELTA_MAX_KEY_DIM, DELTA_MAX_TAPS = 512, 16


def delta_memory_floats(n_heads, dk, dv) -> int:
    """32-bit numbers of one request's memories of the gated delta rule, as `delta_scan` lays them out: per head and tile of four
    value channels, [dk][4]."""
    return n_heads * (-(-dv // 4)) * dk * 4


def delta_state_floats(n_heads, n_kv, dk, dv, n_taps) -> int:
    """... and of its whole state: the memories, then the convolutions' last n_taps - 1 inputs [n_taps - 1][2 n_kv dk + n_heads dv]
    (needs no library, so that a cache can be planned without one)."""
    return delta_memory_floats(n_heads, dk, dv) + (n_taps - 1) * (2 * n_kv * dk + n_heads * dv)


def _delta_checks(what, proj, state, n_heads, n_kv, dk, dv, n_taps):
    if not (proj.dtype == torch.float32 and proj.dim() == 2 and proj.stride(1) == 1):
        raise KernelError(f"{what}: the projections must be float32 [n, columns] with unit inner stride")
    if not (state.dtype == torch.float32 and state.dim() == 2 and state.stride(1) == 1 and state.shape[1] >= delta_state_floats(n_heads, n_kv, dk, dv, n_taps)):
        raise KernelError(f"{what}: state must be float32 [slots, delta_state_floats]")
    if not (0 < dk <= DELTA_MAX_KEY_DIM and 1 <= n_taps <= DELTA_MAX_TAPS and n_heads % n_kv == 0):
        raise KernelError(f"{what}: keys of 1 to {DELTA_MAX_KEY_DIM} channels, 1 to {DELTA_MAX_TAPS} taps and heads in whole groups are served")


def delta_prepare(proj, conv_off, a_off, b_off, taps, a_log, dt_bias, ctx_slots, ctx_positions, state, qkv, gates, n_heads, n_kv, dk, dv, q_scale,
                  single_rows=False):
    """What the gated delta rule needs of every row (csrc/recurrent.hip: delta_prepare_kernel): the columns [conv_off, conv_off +
    2 n_kv dk + n_heads dv) of proj (queries, keys, values) through their short convolutions (taps float32 [channels, n_taps]; a
    request's rows before this step come from its state) and SiLU, queries and keys made unit vectors per head (queries times
    q_scale), into qkv float32 [n, channels]; and gates float32 [n, 2 heads]: the decays exp(-exp(a_log) softplus(proj[a_off + h] +
    dt_bias)), then the step sizes sigmoid(proj[b_off + h]).  single_rows: every row is its request's only row of the step; the
    kernel then also moves every request's tail on by its row, and `delta_tail` is not needed."""
    _dev(proj, taps, a_log, dt_bias, ctx_slots, ctx_positions, state, qkv, gates)
    n, n_conv = proj.shape[0], 2 * n_kv * dk + n_heads * dv
    n_taps = taps.shape[1]
    _delta_checks("delta_prepare", proj, state, n_heads, n_kv, dk, dv, n_taps)
    if not (taps.dtype == torch.float32 and taps.shape == (n_conv, n_taps) and taps.is_contiguous()):
        raise KernelError("delta_prepare: taps must be float32 [2 kv_heads dk + heads dv, n_taps]")
    for t, name in ((a_log, "a_log"), (dt_bias, "dt_bias")):
        if not (t.dtype == torch.float32 and t.is_contiguous() and t.numel() == n_heads):
            raise KernelError(f"delta_prepare: {name} must be float32 [heads]")
    if not (qkv.dtype == torch.float32 and qkv.shape == (n, n_conv) and qkv.is_contiguous() and gates.dtype == torch.float32 and gates.shape == (n, 2 * n_heads) and gates.is_contiguous()):
        raise KernelError("delta_prepare: qkv must be float32 [n, channels] and gates float32 [n, 2 heads], contiguous")
    if min(conv_off, a_off, b_off) < 0 or max(conv_off + n_conv, a_off + n_heads, b_off + n_heads) > proj.shape[1]:
        raise KernelError("delta_prepare: the columns named lie outside proj")
    _i32(ctx_slots, "delta_prepare: slots", n)
    _i32(ctx_positions, "delta_prepare: positions", n)
    _call("gi_delta_prepare", proj.data_ptr(), proj.stride(0), int(conv_off), int(a_off), int(b_off), taps.data_ptr(), n_taps, a_log.data_ptr(), dt_bias.data_ptr(),
          ctx_slots.data_ptr(), ctx_positions.data_ptr(), state.data_ptr(), state.stride(0), qkv.data_ptr(), gates.data_ptr(), n, n_heads, n_kv, dk, dv,
          float(q_scale), 1 if single_rows else 0, _stream())


def delta_tail(proj, conv_off, n_taps, seg_start, seg_len, row_slot, state, n_heads, n_kv, dk, dv):
    """After `delta_prepare` has read them: every request's last n_taps - 1 rows of the convolved columns become its state's tail."""
    _dev(proj, seg_start, seg_len, row_slot, state)
    _delta_checks("delta_tail", proj, state, n_heads, n_kv, dk, dv, n_taps)
    n_segs = seg_start.numel()
    _i32(seg_start, "delta_tail: seg_start", n_segs)
    _i32(seg_len, "delta_tail: seg_len", n_segs)
    _i32(row_slot, "delta_tail: slots", proj.shape[0])
    if conv_off < 0 or conv_off + 2 * n_kv * dk + n_heads * dv > proj.shape[1]:
        raise KernelError("delta_tail: the columns named lie outside proj")
    _call("gi_delta_tail", proj.data_ptr(), proj.stride(0), int(conv_off), int(n_taps), seg_start.data_ptr(), seg_len.data_ptr(), n_segs, row_slot.data_ptr(),
          state.data_ptr(), state.stride(0), n_heads, n_kv, dk, dv, _stream())


def delta_scan(qkv, gates, seg_start, seg_len, row_slot, state, out, n_heads, n_kv, dk, dv):
    """The gated delta rule over every request's rows of the step, in order (csrc/recurrent.hip states it): qkv and gates as
    `delta_prepare` leaves them, out float32 [n, heads*dv] gets the read-outs M^T q; the memories come from the request's state
    slot and go back into it."""
    _dev(qkv, gates, seg_start, seg_len, row_slot, state, out)
    n = qkv.shape[0]
    if not (qkv.dtype == torch.float32 and qkv.dim() == 2 and qkv.stride(1) == 1 and qkv.shape[1] >= 2 * n_kv * dk + n_heads * dv and gates.dtype == torch.float32
            and gates.shape == (n, 2 * n_heads) and gates.is_contiguous() and out.dtype == torch.float32 and out.shape == (n, n_heads * dv) and out.stride(1) == 1):
        raise KernelError("delta_scan: qkv must be float32 [n, channels], gates float32 [n, 2 heads], out float32 [n, heads*dv]")
    if not (state.dtype == torch.float32 and state.dim() == 2 and state.stride(1) == 1 and state.shape[1] >= delta_memory_floats(n_heads, dk, dv)):
        raise KernelError("delta_scan: state must be float32 [slots, at least delta_memory_floats]")
    if not (0 < dk <= DELTA_MAX_KEY_DIM and n_heads % n_kv == 0):
        raise KernelError(f"delta_scan: keys of 1 to {DELTA_MAX_KEY_DIM} channels and heads in whole groups are served")
    n_segs = seg_start.numel()
    _i32(seg_start, "delta_scan: seg_start", n_segs)
    _i32(seg_len, "delta_scan: seg_len", n_segs)
    _i32(row_slot, "delta_scan: slots", n)
    _call("gi_delta_scan", qkv.data_ptr(), qkv.stride(0), gates.data_ptr(), seg_start.data_ptr(), seg_len.data_ptr(), n_segs, row_slot.data_ptr(), state.data_ptr(),
          state.stride(0), out.data_ptr(), out.stride(0), n_heads, n_kv, dk, dv, _stream())
    return out


# --------------------------------------------------------------------------------------------- attention through latents
def latent_prepare(proj, q_rank, kv_rank, rot, q_norm, kv_norm, eps, cos, sin, positions, slots, table, cq, cache, page_size):
    """proj float32 [n, q_rank + kv_rank + rot]: the query latent, RMS-normed with q_norm, into cq [n, q_rank]; the key/value latent,
    RMS-normed with kv_norm, and the last rot channels turned in neighbouring pairs (cos, sin float32 [n, rot/2]), into the row's
    place of its page: the keys [place][kv_rank + rot], and the latent once more behind them with the places innermost, [kv_rank][place]
    (a layer of one key/value head with keys of kv_rank + rot and values of kv_rank channels)."""
    _dev(proj, q_norm, kv_norm, cos, sin, positions, slots, table, cq, cache)
    n = proj.shape[0]
    if not (proj.dtype == torch.float32 and proj.dim() == 2 and proj.stride(1) == 1 and proj.shape[1] >= q_rank + kv_rank + rot):
        raise KernelError("latent_prepare: proj must be float32 [n, q_rank + kv_rank + rot]")
    if not (q_norm.shape == (q_rank,) and kv_norm.shape == (kv_rank,) and q_norm.is_contiguous() and kv_norm.is_contiguous() and q_norm.dtype == kv_norm.dtype):
        raise KernelError("latent_prepare: the norms' weights must be [q_rank] and [kv_rank], of one dtype")
    if not (cq.shape == (n, q_rank) and cq.stride(1) == 1):
        raise KernelError("latent_prepare: cq must be [n, q_rank]")
    if rot:
        for t in (cos, sin):
            if not (t.dtype == torch.float32 and t.shape == (n, rot // 2) and t.is_contiguous()):
                raise KernelError("latent_prepare: cos/sin must be float32 [n, rot/2]")
    _check_paged(cache, table, "latent_prepare")
    if cache.stride(0) < page_size * (2 * kv_rank + rot):
        raise KernelError("latent_prepare: the pages are too small for these latents")
    _i32(positions, "latent_prepare: positions", n)
    _i32(slots, "latent_prepare: slots", n)
    _call("gi_latent_prepare", proj.data_ptr(), proj.stride(0), q_rank, kv_rank, rot, q_norm.data_ptr(), kv_norm.data_ptr(), _code(q_norm, "latent_prepare: norm"),
          float(eps), _ptr(cos), _ptr(sin), positions.data_ptr(), slots.data_ptr(), table.data_ptr(), table.stride(0), cq.data_ptr(), _code(cq, "latent_prepare: cq"),
          cq.stride(0), cache.data_ptr(), _code(cache, "latent_prepare: cache"), cache.stride(0), int(page_size), n, _stream())


def latent_queries(q, cos, sin, plain, folded, n_heads, dim, rot, kv_rank):
    """q float32 [n, heads*(dim + rot)]: every head's first dim channels into plain [n, heads*dim]; its last rot channels, turned in
    neighbouring pairs, into folded [n, heads*(kv_rank + rot)] behind the head's first kv_rank places."""
    _dev(q, cos, sin, plain, folded)
    n = q.shape[0]
    if not (q.dtype == torch.float32 and q.shape == (n, n_heads * (dim + rot)) and q.stride(1) == 1 and plain.shape == (n, n_heads * dim) and plain.stride(1) == 1
            and folded.shape == (n, n_heads * (kv_rank + rot)) and folded.stride(1) == 1):
        raise KernelError("latent_queries: q must be float32 [n, heads*(dim+rot)], plain [n, heads*dim], folded [n, heads*(kv_rank+rot)]")
    if rot:
        for t in (cos, sin):
            if not (t.dtype == torch.float32 and t.shape == (n, rot // 2) and t.is_contiguous()):
                raise KernelError("latent_queries: cos/sin must be float32 [n, rot/2]")
    _call("gi_latent_queries", q.data_ptr(), q.stride(0), _ptr(cos), _ptr(sin), plain.data_ptr(), _code(plain, "latent_queries: plain"), plain.stride(0),
          folded.data_ptr(), _code(folded, "latent_queries: folded"), folded.stride(0), n, n_heads, dim, rot, kv_rank, _stream())


class AttentionPlan:
    """How a step's rows are shared between the two bfloat16 attention kernels: requests that bring
    one row go to the decode kernel, portions of prompts are cut into tiles of up to 128 rows for
    the prompt kernel.  Short portions go to the decode kernel too, row by row (every row attends
    over its own prefix, which the cache holds by then): a tile's workgroup walks the whole context
    in sequence, however few its rows, while the decode kernel cuts each row's context into pieces
    for the whole chip (break-even near 90 rows at the Llama-3.2-1B shape; above SHORT_TOTAL rows
    in all, the rows' repeated reading of the context costs more than the tiles' sequence).
    Made once per step and used by every layer."""
    TILE = 0                             # rows of a prompt tile, 64 or 128; 0: by the step's size
    SMALL_STEP = 768                     # up to this many tiled rows in a step, tiles of 64 rows fill the chip better (measured at 32 heads)
    PAIRS = True                         # a portion's late tiles share workgroups with its early ones
    SHORT, SHORT_TOTAL = 64, 64          # portions of up to SHORT rows count as short; they go row by row while they sum to at most SHORT_TOTAL

    @classmethod
    def all_decode(cls, n_rows, max_context, device):
        """Every row is a request's single new row (what a captured decode step uses: nothing in it depends on the step)."""
        plan = cls.__new__(cls)
        plan.n_decode, plan.n_tiles, plan.max_decode_context, plan.single_rows = n_rows, 0, max_context, True
        plan.decode_rows = None                                  # rows 0 .. n_rows-1
        plan.tiles = torch.empty(0, dtype=torch.int32, device=device)
        plan.n_tile_rows, plan.max_tile_context, plan.tile_first, plan.tile_rows, plan.paired, plan.tile = 0, 0, None, None, False, 128
        return plan

    def __init__(self, seg_start, seg_len, seg_pos0, seg_slot, device, to_device=None):
        dec, tiles, portions, self.max_decode_context = [], [], [], 0
        short_rows = sum(n for n in seg_len if 1 < n <= self.SHORT)
        row_by_row = self.SHORT if short_rows <= self.SHORT_TOTAL else 1
        self.single_rows = all(n == 1 for n in seg_len)          # every row is a request's only new row
        self.tile = self.TILE or (64 if sum(n for n in seg_len if n > row_by_row) <= self.SMALL_STEP else 128)
        for start, n, pos0, slot in zip(seg_start, seg_len, seg_pos0, seg_slot):
            if n <= row_by_row:
                dec.extend(range(start, start + n))
                self.max_decode_context = max(self.max_decode_context, pos0 + n)
            else:
                portions.append([(start + off, min(self.tile, n - off), pos0 + off, slot) for off in range(0, n, self.tile)])
        # Tile i of a portion sees the keys of the tiles before it: the last tile goes with the first, the last but
        # one with the second, ... so that every pair has about the same number of keys to visit and reads them once
        # for both (a tile of no rows fills the middle pair of an odd number).  Without a portion of two tiles, no pairs.
        self.paired = self.PAIRS and any(len(p) > 1 for p in portions)
        for p in portions:
            if not self.paired:
                tiles.extend(p)
                continue
            for i in range((len(p) + 1) // 2):
                late, early = p[len(p) - 1 - i], p[i]
                tiles.extend((late, early if early is not late else (late[0], 0, late[2], late[3])))
        self.n_decode, self.n_tiles = len(dec), len(tiles)
        self.n_tile_rows = sum(t[1] for t in tiles)
        self.max_tile_context = max((t[2] + t[1] for t in tiles), default=0)
        # for sharing a tile's keys out over workgroups: rows before each tile, and the tiles' rows in order
        firsts, count = [], 0
        for t in tiles:
            firsts.append(count)
            count += t[1]
        put = to_device if to_device is not None else (lambda *lists: tuple(torch.tensor(values, dtype=torch.int32).to(device) for values in lists))
        self.decode_rows = self.tile_first = self.tile_rows = None      # no prompt rows: the decode rows are all rows, in order
        self.tiles = torch.empty(0, dtype=torch.int32, device=device)
        if tiles:                            # (every piece starts at a multiple of 16 bytes: the kernel reads a tile's four numbers at once)
            self.tiles, self.tile_first, self.tile_rows, *rest = put([v for t in tiles for v in t], firsts, [r for t in tiles for r in range(t[0], t[0] + t[1])],
                                                                     *([dec] if dec else []))
            self.decode_rows = rest[0] if rest else None


@lru_cache(maxsize=None)
def attention_bf16_supports(hd, page_size, prompt: bool) -> bool:
    return bool(lib().gi_attention_bf16_supports(hd, page_size, 1 if prompt else 0))


PAIRED_TARGET_GROUPS = 256


def prompt_attention_splits(n_groups, n_heads, span, target_groups=512):
    """Workgroups the keys of a tile (or pair of tiles) are shared out over: none while the tiles alone fill the chip
    (two workgroups a compute unit) or the context is short; every share keeps at least 256 keys."""
    groups = n_groups * n_heads
    if groups >= target_groups // 2:
        return 1
    return max(1, min(-(-target_groups // groups), span // 256, 64))


def _decode_piece(span, n_pieces):
    """Positions a wave of the decode kernel takes when a context of `span` is cut into `n_pieces` (multiples of 32, as the kernel cuts)."""
    return (-(-span // n_pieces) + 31) & ~31


@lru_cache(maxsize=None)
def _decode_places(hd, fused, n_waves, gh):
    """Workgroups of `n_waves` waves of the decode kernel that the chip holds at once."""
    per_unit = lib().gi_attention_decode_workgroups_per_unit(hd, 1 if fused else 0, n_waves, gh)
    return lib().gi_compute_units() * (per_unit if per_unit > 0 else max(1, 16 // n_waves))


def _decode_plain_shape(groups, span, max_waves, target_waves=4096, small=False):
    """About `target_waves` waves in all, pieces of at least 64 positions; one split when a workgroup's waves cover them.
    small (a few rows, heads of up to 64 channels, the kernel with rotation inside): pieces down to 32 positions, and workgroups
    of 8 waves while there are few of them (up to 64 groups of heads: half the partial results for the second kernel to merge)."""
    if small:
        target_waves //= 2          # (its waves ask for the next keys while they multiply: half as many, twice as long, measured faster at 4 to 12 rows)
    pieces = max(1, min(-(-target_waves // groups), -(-span // (32 if small else 64))))
    if pieces <= max_waves:
        return (1, pieces)
    n_waves = min(8 if small and groups <= 64 else 4, max_waves)
    return (min(-(-pieces // n_waves), 256), n_waves)


# What the decode kernel's workgroups reach (measured at heads of 64 and 128 channels, 17 to 128 rows, contexts of 1,100 to
# 16,384): a compute unit pulls about 31 GB/s for one workgroup and 27 GB/s for several, however many waves they have (from
# four up), the chip 5.9 TB/s, and a second kernel that merges splits costs about 6 us with the partial results it reads.
_DECODE_UNIT_MB_PER_S, _DECODE_SHARED_UNIT_MB_PER_S, _DECODE_CHIP_MB_PER_S, _DECODE_MERGE_US = 31e3, 27e3, 5.9e6, 6.0


def _decode_single_split(groups, span, hd, max_waves):
    """(1, waves) if one workgroup per (row, group of heads) over the whole context, which needs no second kernel, is expected
    to be no slower than a context cut over several; else None.  Without splits the compute unit with the most workgroups sets
    the time (`groups` over the units, rounded up, each pulling its share of the bytes at a unit's rate); with them the chip's
    rate does, plus the merge.  Of a bracket of contexts three quarters are taken as read.  Four waves where a wave's share
    stays under 200 KB and there is a workgroup for every unit, else eight."""
    units = lib().gi_compute_units()
    mbytes = groups * 0.75 * span * hd * 4 / 1e6
    most = -(-groups // units)                       # workgroups of the busiest compute unit
    single_us = max(most * (mbytes / groups) / (_DECODE_UNIT_MB_PER_S if most == 1 else _DECODE_SHARED_UNIT_MB_PER_S), mbytes / _DECODE_CHIP_MB_PER_S) * 1e6
    if groups < units // 2 or single_us > mbytes / _DECODE_CHIP_MB_PER_S * 1e6 + _DECODE_MERGE_US:
        return None
    n_waves = 8 if groups < units or 0.75 * span / 4 * hd * 4 > 200e3 else 4
    return (1, min(n_waves, max_waves))


@lru_cache(maxsize=None)
def decode_attention_shape(n_decode, n_heads, n_kv, hd, span, target_waves=4096, fused=False):
    """(splits, waves per workgroup) of the decode kernel: about `target_waves` waves in all and pieces of
    at least 64 positions; a single split (no combine kernel) when a workgroup's waves cover them.

    The chip holds so many workgroups of the kernel at once (the runtime's answer for this head size: 16 waves a compute
    unit at 64 channels, 12 at 128); workgroups beyond that run as a further round, and a round with a few workgroups in it
    costs as much as a full one (65 requests of 8 key/value heads: 520 workgroups of 8 waves on 512 places took 73 us a layer
    against 50 at 64).  So where the plain rule leaves a last round less than half full (less than a third where it has one
    split: there is no combine kernel to save then, and fewer pieces mean longer waves), or workgroups of 5 to 7 waves (which
    measured slower than either neighbour), the context is cut into as many pieces as fit in one round instead, in workgroups
    of 8 or 4 waves (of 3 or 2 where those leave fewer than 6 pieces), with as few splits as that allows: 65 rows 73 -> 57 us a layer, 96 rows 90 -> 74, 40 rows 46 -> 38,
    56 rows 2.10 -> 1.92 ms a step (heads of 64 channels); 65 rows 127 -> 111 us (heads of 128).  The small batches whose kernel
    also rotates and stores the new key keep the plain rule at heads of 64 channels: their workgroups are short, and 8 and 16 rows
    measured 5 and 3 % slower with one round.  What helps them is more and shorter pieces in fewer, larger workgroups (`small` in
    `_decode_plain_shape`; attention and combine kernel together, context 2,100: 1 row 11.4 -> 9.9 us a layer, 4 rows 13.8 -> 12.2,
    6 rows 15.8 -> 14.8, 8 rows 17.5 -> 17.0; context 1,100: 8 rows 12.9 -> 11.8).  At 128 channels that kernel's registers leave room for 8 waves a compute unit, and
    there one round is the faster cut whenever the plain rule needs more (8 rows: 30 -> 27 us a layer at a context of 2,100, 35 ->
    29 at 3,000; the step of the 8B shape 4.82 -> 4.79 ms at 8 rows, 5.47 -> 5.31 at 16).

    Since the kernel's waves ask for the next keys while they multiply (page numbers through the scalar unit, no wait for loads
    that are not needed yet), a wave is cheap to run for long, and from 17 rows on a context that is not cut at all is often the
    faster one: no partial results, no second kernel (`_decode_single_split` says when: 24 rows 27 -> 21 us a layer at a context
    of 2,100, 32 rows 31 -> 25, 64 rows 50 -> 47 with four waves instead of eight, 96 rows 76 -> 69; 24 rows at heads of 128
    channels 48 -> 38).  The rules above decide the rest."""
    group = n_heads // n_kv
    groups = n_decode * n_kv * ((group + 15) // 16)
    max_waves = min(8, lib().gi_attention_decode_max_waves(hd))
    base = _decode_plain_shape(groups, span, max_waves, target_waves, small=fused and hd <= 64)
    if target_waves != 4096:
        return base
    if not fused or n_decode > 16:                   # (more than 16 rows: whichever kernel serves them)
        single = _decode_single_split(groups, span, hd, max_waves)
        if single is not None:
            return single
    if fused and hd < 128:
        return base
    gh = min(group, 16)
    units = lib().gi_compute_units()
    places = lambda n_waves: min(_decode_places(hd, fused, n_waves, gh), units) if fused else _decode_places(hd, fused, n_waves, gh)
    rounds = groups * base[0] / places(base[1])
    if fused:                        # (heads of 128 channels: 8 waves a compute unit, and a second round costs what it brings; with the
        if rounds <= 1:              # waves asking ahead, a workgroup for every compute unit is enough: 4 rows 17.2 -> 14.7 us a layer)
            return base
    else:
        short_last_round = rounds > 1 and 0 < rounds - int(rounds) < (0.5 if base[0] > 1 else 0.3)
        if not (short_last_round or 5 <= base[1] <= 7):
            return base
    def most_pieces(widths):
        best = None
        for n_waves in widths:
            if n_waves > max_waves:
                continue
            splits = min(places(n_waves) // groups, 256)         # as many as still fit in one round
            while splits > 1 and _decode_piece(span, splits * n_waves) < 64:
                splits -= 1
            if splits >= 1 and (best is None or splits * n_waves > best[0] * best[1] or (splits * n_waves == best[0] * best[1] and splits < best[0])):
                best = (splits, n_waves)
        return best
    best = most_pieces((8, 4))
    if best is None or best[0] * best[1] < 6:        # narrow workgroups only where wide ones leave few pieces: many small ones run slower than the same pieces in wide ones
        best = most_pieces((8, 4, 3, 2))
    return best or base


def attention_bf16(q, cache, out, plan: AttentionPlan, positions, slots, table, n_heads, n_kv, hd, window=None, scale=None,
                   target_waves: int = 4096, products=None, chunk=None, sinks=None, gate=None, cap=None):
    """Attention of a step's rows with the matrix-core kernels (bfloat16 cache and out).

    `q` holds the rotated queries in bfloat16 and the cache the rows' keys and values; or, for a step
    of single decoded rows only, `q` is None and `products = (q, k, v, cos, sin)` holds the unrotated
    float32 products and the rotation's tables (k, v None: the pages are another layer's; cos, sin
    None: no rotation): the decode kernel then rotates, writes the cache and attends in one launch.

    chunk, sinks, gate: as `attention_exact` takes them (a mask cut into chunks, a score per head that joins the softmax's
    denominator only, a gate per row and head on the output)."""
    n = out.shape[0]
    _dev(q, cache, out, positions, slots, table, sinks, gate)
    if sinks is not None and not (sinks.dtype == torch.float32 and sinks.is_contiguous() and sinks.numel() == n_heads):
        raise KernelError("attention: sinks must be float32 [heads]")
    if gate is not None and not (gate.dtype == torch.float32 and gate.dim() == 2 and gate.shape[0] == n and gate.shape[1] >= n_heads and gate.stride(1) == 1):
        raise KernelError("attention: the heads' gates must be float32 [n, heads] with unit inner stride")
    chunk = int(chunk or 0)
    if cap is not None and not cap > 0:
        raise KernelError("attention: the scores' cap must be positive")
    extras = (chunk, _ptr(sinks), _ptr(gate), gate.stride(0) if gate is not None else 0, float(cap or 0.0))
    seen = lambda context, slack: min([context] + ([window + slack] if window else []) + ([chunk + slack] if chunk else []))
    for t, name in ((q, "q"), (cache, "cache"), (out, "out")):
        if not (t is None or t.dtype == torch.bfloat16):
            raise KernelError(f"attention_bf16: {name} must be bfloat16")
    if not (out.shape == (n, n_heads * hd) and out.is_contiguous() and (q is None or (q.shape == out.shape and q.is_contiguous()))):
        raise KernelError( "attention: q and out must be [n, heads*hd], contiguous")
    page_size = cache.shape[3]
    _check_cache(cache, table, page_size, n_kv, hd, "attention")
    _i32(positions, "attention: positions", n)
    _i32(slots, "attention: slots", n)
    window = int(window or 0)
    scale = float(scale if scale is not None else hd ** -0.5)
    if not ((q is None) != (products is None)):
        raise KernelError("attention_bf16: give rotated queries or the unrotated products")
    qf = kf = vf = cos = sin = None
    if products is not None:
        if not (plan.n_tiles == 0):
            raise KernelError("attention_bf16: unrotated products serve steps of single decoded rows only")
        qf, kf, vf, cos, sin = products
        _dev(qf, kf, vf, cos, sin)
        if not (qf.dtype == torch.float32 and qf.shape == (n, n_heads * hd) and qf.stride(1) == 1):
            raise KernelError("attention: q must be float32 [n, heads*hd]")
        for t, name in ((kf, "k"), (vf, "v")):
            if not (t is None or (t.dtype == torch.float32 and t.shape == (n, n_kv * hd) and t.stride(1) == 1)):
                raise KernelError( f"attention: {name} must be float32 [n, kv_heads*hd]")
        for t in (cos, sin):
            if not (t is None or (t.dtype == torch.float32 and t.shape == (n, hd // 2) and t.is_contiguous())):
                raise KernelError("attention: cos/sin must be float32 [n, hd/2]")
    if plan.n_tiles:
        n_splits = prompt_attention_splits(plan.n_tiles // 2 if plan.paired else plan.n_tiles, n_heads, seen(plan.max_tile_context, plan.tile),
                                           target_groups=PAIRED_TARGET_GROUPS if plan.paired else 512)      # a pair's workgroup has twice the waves
        n_part = plan.n_tile_rows * n_heads * n_splits * (hd + 2) if n_splits > 1 else 0
        part = torch.empty(n_part, dtype=torch.float32, device=out.device) if n_part else None
        _call("gi_attention_prompt_bf16", q.data_ptr(), cache.data_ptr(), out.data_ptr(), plan.tiles.data_ptr(), plan.n_tiles, plan.tile,
              1 if plan.paired else 0, table.data_ptr(), table.stride(0), cache.stride(0), page_size, n_heads, n_kv, hd, window, scale, n_splits,
              _ptr(plan.tile_first), _ptr(plan.tile_rows), plan.n_tile_rows, _ptr(part), n_part, *extras, _stream())
    if plan.n_decode:
        span = seen(plan.max_decode_context, 31)
        n_splits, n_waves = decode_attention_shape(plan.n_decode, n_heads, n_kv, hd, span, target_waves, products is not None)
        n_part = plan.n_decode * n_heads * n_splits * (hd + 2) if n_splits > 1 else 0
        part = torch.empty(n_part, dtype=torch.float32, device=out.device) if n_part else None
        _call("gi_attention_decode_bf16", _ptr(q), _ptr(qf), _ptr(kf), _ptr(vf), qf.stride(0) if qf is not None else 0,
              kf.stride(0) if kf is not None else 0, vf.stride(0) if vf is not None else 0, _ptr(cos), _ptr(sin), cache.data_ptr(),
              out.data_ptr(), _ptr(part), n_part, _ptr(plan.decode_rows), plan.n_decode, positions.data_ptr(), slots.data_ptr(),
              table.data_ptr(), table.stride(0), cache.stride(0), page_size, n_heads, n_kv, hd, window, scale, n_splits, n_waves, *extras, _stream())
    return out


def _plan_of(ctx):
    if "attention_plan" not in ctx.memo:
        ctx.memo["attention_plan"] = AttentionPlan(ctx.seg_start, ctx.seg_len, ctx.seg_pos0, ctx.seg_slot, ctx.device, ctx.to_device)
    return ctx.memo["attention_plan"]


def attention(q, cache, out, ctx, table, n_heads, n_kv, hd, window=None):
    """Attention of a step's rows; the kernel is chosen by the storage dtype and the batch's shape."""
    page_size = cache.shape[3]
    if q.dtype == torch.bfloat16 and cache.dtype == torch.bfloat16 and out.dtype == torch.bfloat16:
        plan = _plan_of(ctx)
        if (not plan.n_tiles or attention_bf16_supports(hd, page_size, True)) and (not plan.n_decode or attention_bf16_supports(hd, page_size, False)):
            return attention_bf16(q, cache, out, plan, ctx.row_pos, ctx.row_slot, table, n_heads, n_kv, hd, window)
    return attention_exact(q, cache, out, ctx.row_pos, ctx.row_slot, table, n_heads, n_kv, hd, window)


def attention_general(q, cache, out, ctx, table, n_heads, n_kv, hd, *, page_size, value_dim=None, window=None, chunk=None, scale=None, sinks=None, gate=None,
                      cap=None):
    """Attention of a step's rows for layers with any of: value heads of another size, a scale of their own, a mask cut into
    chunks, sinks, a gate per head, capped scores."""
    vd = int(value_dim or hd)
    if (vd == hd and cache.dim() == 5 and q.dtype == torch.bfloat16 and cache.dtype == torch.bfloat16 and out.dtype == torch.bfloat16
            and (gate is None or gate.dtype == torch.float32) and (cap is None or hd <= 128)):          # (capped scores on the matrix cores: tested up to heads of 128)
        plan = _plan_of(ctx)
        if (not plan.n_tiles or attention_bf16_supports(hd, page_size, True)) and (not plan.n_decode or attention_bf16_supports(hd, page_size, False)):
            return attention_bf16(q, cache, out, plan, ctx.row_pos, ctx.row_slot, table, n_heads, n_kv, hd, window, scale, chunk=chunk, sinks=sinks, gate=gate, cap=cap)
    return attention_exact(q, cache, out, ctx.row_pos, ctx.row_slot, table, n_heads, n_kv, hd, window, scale, page_size=page_size,
                           value_dim=value_dim, chunk=chunk, sinks=sinks, gate=gate, cap=cap)


# Up to so many rows the decode kernel rotates and writes the pages itself.  It saves the rotation kernel's launch wherever the
# q/k/v product does not rotate and store in its own epilogue (which it does from 33 rows on, and for long k from 17): +2..3 % a
# step at 1 and 8 rows, and at 17 to 32 rows of the Llama-3.2-1B shape (24 rows 1.323 -> 1.290 ms).
FUSED_DECODE_MAX_ROWS = 32


def attention_from_products(q, k, v, cos, sin, cache, out, ctx, table, n_heads, n_kv, hd, window=None) -> bool:
    """Rotation, cache write and attention in one launch, from the unrotated float32 products, when
    every row of the step is a request's single new row, the rows are few and the matrix-core decode
    kernel takes the sizes.  Returns False (nothing done) otherwise: the caller then rotates and stores first."""
    if not (cache.dtype == torch.bfloat16 and out.dtype == torch.bfloat16 and q.dtype == torch.float32):
        return False
    plan = _plan_of(ctx)
    if plan.n_tiles or not plan.single_rows or not attention_bf16_supports(hd, cache.shape[3], False):      # rows of one portion need each other's keys in the cache
        return False
    if plan.n_decode > FUSED_DECODE_MAX_ROWS:
        return False
    if q.stride(0) % 4 or q.data_ptr() % 16 or (k is not None and (k.stride(0) % 4 or k.data_ptr() % 16)):
        return False
    attention_bf16(None, cache, out, plan, ctx.row_pos, ctx.row_slot, table, n_heads, n_kv, hd, window, products=(q, k, v, cos, sin))
    return True


def gemm_bf16_supports(a, w, out) -> bool:
    """Shapes and alignments the matrix-core kernels take; the exact kernel serves the rest."""
    k = a.shape[1]
    return (a.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and k % 8 == 0 and a.stride(1) == 1 and w.stride(1) == 1
            and a.stride(0) % 8 == 0 and w.stride(0) % 8 == 0 and a.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0
            and (out.dtype == torch.float32 or out.dtype == torch.bfloat16) and out.stride(1) == 1)


# What the library says about a shape does not change while the process lives, and a step asks it some hundred times: the answers
# are kept (a question costs a call through ctypes, about a microsecond of the host's time each).
@lru_cache(maxsize=None)
def _scratch_floats(m, n, k) -> int:
    return lib().gi_gemm_bf16_scratch_floats(m, n, k)


@lru_cache(maxsize=None)
def gemm_bf16_norm_parts(m, n, k) -> int:
    """The pieces per row in which a product [m, k] x [n, k] that adds onto rows writes their sums of squares when it hands
    the next norm on (`gemm_bf16(..., norm_out=...)`); 0 if a product of these sizes cannot."""
    return lib().gi_gemm_bf16_norm_parts(m, n, k)


@lru_cache(maxsize=None)
def gemm_bf16_takes_norm(m, n, k, gated=False) -> bool:
    """Whether a product of these sizes can read rows whose norm was handed on (`gemm_bf16(..., norm_in=...)`) by a product
    of as many rows."""
    return bool(lib().gi_gemm_bf16_takes_norm(m, n, k, 1 if gated else 0))


def gemm_bf16(a, w, out, accumulate=False, gated=False, checked=False, norm_in=None, norm_out=None, gate_limit=0.0):
    """out (=|+=) a @ w.T with bfloat16 operands on the matrix cores, float32 sums.
    gated: w is [gate; up] interleaved in groups of 16 rows and out = act(a @ gate.T) * (a @ up.T), bfloat16 [m, n/2]; act is
    SiLU (gated = True or "silu"), the tanh form of GELU (gated = "gelu_tanh") or the clamped form (gated = "swish_clamped", with
    `gate_limit`; see `ACTIVATIONS`).

    An RMS norm between two products of a few rows, without a kernel of its own:
    norm_out = (g, scaled, squares), with accumulate: beside out += a @ w.T, scaled = bfloat16(g * out) and squares
    [m, gemm_bf16_norm_parts(m, n, k)] = the pieces of the rows' sums of out^2;
    norm_in = (squares, eps): a is such a `scaled`, and the results are multiplied by rsqrt(sum of the row's pieces / k + eps)."""
    _dev(a, w, out)
    m, k = a.shape
    n = w.shape[0]
    if not (w.shape == (n, k)):
        raise KernelError(f"gemm: weight is {tuple(w.shape)}, activations are {tuple(a.shape)}")
    if not (out.shape == (m, n // 2 if gated else n)):
        raise KernelError(f"gemm: out is {tuple(out.shape)}, ({m}, {n // 2 if gated else n}) is needed")
    if not (checked or gemm_bf16_supports(a, w, out)):
        raise KernelError("gemm_bf16: operands must be bfloat16 with K and row strides multiples of 8, 16-byte aligned")
    n_scratch = _scratch_floats(m, n, k)                             # partial sums where k is split over workgroups
    scratch = torch.empty(n_scratch, dtype=torch.float32, device=a.device) if n_scratch else None
    if gated and gated is not True and gated not in ACTIVATIONS:
        raise KernelError(f"gemm: unknown activation {gated!r} of a gated product; known: {', '.join(ACTIVATIONS)}")
    gate_code = 0 if not gated else 1 + (0 if gated is True else ACTIVATIONS[gated])        # 1: SiLU, 2: GELU (tanh form)
    if _profile is not None:
        _profile.note = (f"{n}x{k}{' gated' if gated else ''}", n * k * w.element_size())
    if norm_in is not None or norm_out is not None:
        squares_in, eps = norm_in if norm_in is not None else (None, 0.0)
        g, scaled, squares_out = norm_out if norm_out is not None else (None, None, None)
        if squares_in is not None and not (squares_in.dtype == torch.float32 and squares_in.is_contiguous() and squares_in.dim() == 2 and squares_in.shape[0] == m):
            raise KernelError("gemm: the pieces of the sums of squares must be float32 [m, pieces]")
        if norm_out is not None:
            parts = gemm_bf16_norm_parts(m, n, k)
            if not (parts and accumulate and out.dtype == torch.float32 and g.dtype == torch.float32 and g.is_contiguous() and g.numel() == n
                    and scaled.dtype == torch.bfloat16 and scaled.shape == (m, n) and scaled.stride(1) == 1
                    and squares_out.dtype == torch.float32 and squares_out.is_contiguous() and squares_out.shape == (m, parts)):
                raise KernelError("gemm: handing a norm on needs a product of a few rows that adds onto float32 rows, float32 weights of the norm, "
                                  "bfloat16 [m, n] for the scaled rows and float32 [m, gemm_bf16_norm_parts] for the sums of squares")
            _dev(g, scaled, squares_out)
        _call("gi_gemm_bf16_handing", a.data_ptr(), w.data_ptr(), out.data_ptr(), _code(out, "gemm: out"), 1 if accumulate else 0, gate_code, float(gate_limit),
              m, n, k, a.stride(0), w.stride(0), out.stride(0), _ptr(scratch), n_scratch, _ptr(squares_in), squares_in.shape[1] if squares_in is not None else 0, float(eps),
              _ptr(g), _ptr(scaled), scaled.stride(0) if scaled is not None else 0, _ptr(squares_out), _stream())
        return out
    _call("gi_gemm_bf16", a.data_ptr(), w.data_ptr(), out.data_ptr(), _code(out, "gemm: out"), 1 if accumulate else 0, gate_code, float(gate_limit),
          m, n, k, a.stride(0), w.stride(0), out.stride(0), _ptr(scratch), n_scratch, _stream())
    return out


@lru_cache(maxsize=None)
def gemm_bf16_qkv_rope_store_takes(m, n, k, hd) -> bool:
    """Whether `gemm_bf16_qkv_rope_store` takes a q/k/v product of m rows, n = (heads + 2 kv heads) * hd columns and k."""
    return bool(lib().gi_gemm_bf16_qkv_rope_store_takes(m, n, k, hd))


@lru_cache(maxsize=None)
def gemm_bf16_qkv_rope_store_max_parts(m, n, k) -> int:
    """The most pieces of a row's sum of squares (`norm_in`) that `gemm_bf16_qkv_rope_store` reads for these sizes."""
    return lib().gi_gemm_bf16_qkv_rope_store_max_parts(m, n, k)


def gemm_bf16_qkv_rope_store(a, w, cos, sin, positions, slots, table, q_out, cache, n_heads, n_kv, hd, norm_in=None):
    """The q/k/v product a @ w.T of an attention layer whose results do not come back: the queries go, rotated, into q_out
    (bfloat16 [m, heads*hd]), the keys (rotated) and the values into the cache's pages, as `rope_store` puts them.
    cos, sin: float32 [m, hd/2] or None; norm_in as for `gemm_bf16`."""
    _dev(a, w, cos, sin, positions, slots, table, q_out, cache)
    m, k = a.shape
    n = w.shape[0]
    if not (gemm_bf16_supports(a, w, q_out) and w.shape == (n, k) and n == (n_heads + 2 * n_kv) * hd and gemm_bf16_qkv_rope_store_takes(m, n, k, hd)):
        raise KernelError(f"gemm (q/k/v): a product of {m} x {n} x {k} with heads of {hd} is not taken")
    if not (q_out.dtype == torch.bfloat16 and q_out.shape == (m, n_heads * hd) and q_out.is_contiguous() and cache.dtype == torch.bfloat16):
        raise KernelError("gemm (q/k/v): q_out must be bfloat16 [m, heads*hd], contiguous, and the cache bfloat16")
    if cos is not None:
        for t in (cos, sin):
            if not (t.dtype == torch.float32 and t.shape == (m, hd // 2) and t.is_contiguous()):
                raise KernelError("gemm (q/k/v): cos/sin must be float32 [m, hd/2]")
    page_size = cache.shape[3]
    _check_cache(cache, table, page_size, n_kv, hd, "gemm (q/k/v)")
    _i32(positions, "gemm (q/k/v): positions", m)
    _i32(slots, "gemm (q/k/v): slots", m)
    squares_in, eps = norm_in if norm_in is not None else (None, 0.0)
    if squares_in is not None and not (squares_in.dtype == torch.float32 and squares_in.is_contiguous() and squares_in.dim() == 2 and squares_in.shape[0] == m):
        raise KernelError("gemm: the pieces of the sums of squares must be float32 [m, pieces]")
    n_scratch = _scratch_floats(m, n, k)
    scratch = torch.empty(n_scratch, dtype=torch.float32, device=a.device) if n_scratch else None
    if _profile is not None:
        _profile.note = (f"{n}x{k}", n * k * w.element_size())
    _call("gi_gemm_bf16_qkv_rope_store", a.data_ptr(), w.data_ptr(), m, n, k, a.stride(0), w.stride(0), _ptr(scratch), n_scratch,
          _ptr(squares_in), squares_in.shape[1] if squares_in is not None else 0, float(eps), _ptr(cos), _ptr(sin), positions.data_ptr(),
          slots.data_ptr(), table.data_ptr(), table.stride(0), q_out.data_ptr(), cache.data_ptr(), cache.stride(0), page_size, n_heads, n_kv, hd, _stream())
    return q_out


def interleave_gate_up(gate, up):
    """[gate; up] in groups of 16 rows: 16 gate rows, the 16 up rows of the same outputs, and so on."""
    i, d = gate.shape
    if not (i % 16 == 0 and up.shape == gate.shape):
        raise KernelError("interleave_gate_up: the intermediate size must be a multiple of 16")
    return torch.stack([gate.view(i // 16, 16, d), up.view(i // 16, 16, d)], dim=1).reshape(2 * i, d).contiguous()


def argmax(logits, out):
    _dev(logits, out)
    n, vocab = logits.shape
    if not (logits.dtype == torch.float32 and logits.stride(1) == 1):
        raise KernelError("argmax: logits must be float32 with unit inner stride")
    _i32(out, "argmax: out", n)
    chunks = lib().gi_argmax_chunks(vocab)
    part_v = torch.empty(n * chunks, dtype=torch.float32, device=logits.device)
    part_i = torch.empty(n * chunks, dtype=torch.int32, device=logits.device)
    _call("gi_argmax", logits.data_ptr(), out.data_ptr(), part_v.data_ptr(), part_i.data_ptr(), n, vocab, logits.stride(0), _stream())
    return out


def sample_temperature(logits, temperature, uniform, out):
    _dev(logits, temperature, uniform, out)
    n, vocab = logits.shape
    if not (logits.dtype == torch.float32 and logits.stride(1) == 1):
        raise KernelError("sample: logits must be float32 with unit inner stride")
    for t, name in ((temperature, "temperature"), (uniform, "uniform")):
        if not (t.dtype == torch.float32 and t.is_contiguous() and t.numel() >= n):
            raise KernelError(f"sample: {name} must be float32 [n]")
    _i32(out, "sample: out", n)
    chunks = lib().gi_argmax_chunks(vocab)
    part_m = torch.empty(n * chunks, dtype=torch.float32, device=logits.device)
    part_s = torch.empty(n * chunks, dtype=torch.float64, device=logits.device)
    _call("gi_sample_temperature", logits.data_ptr(), temperature.data_ptr(), uniform.data_ptr(), out.data_ptr(), part_m.data_ptr(),
          part_s.data_ptr(), n, vocab, logits.stride(0), _stream())
    return out


def sample_filtered(logits, temperature, top_k, top_p, uniform, out):
    """Top-k, then top-p, then the draw, for rows that each have one of the two filters (top_k in 1..vocab-1, or
    top_p < 1): a row without a filter is drawn in index order, which `sample_temperature` does."""
    _dev(logits, temperature, top_k, top_p, uniform, out)
    n, vocab = logits.shape
    if not (logits.dtype == torch.float32 and logits.stride(1) == 1):
        raise KernelError("sample: logits must be float32 with unit inner stride")
    for t, name in ((temperature, "temperature"), (top_p, "top_p"), (uniform, "uniform")):
        if not (t.dtype == torch.float32 and t.is_contiguous() and t.numel() >= n):
            raise KernelError(f"sample: {name} must be float32 [n]")
    _i32(top_k, "sample: top_k", n)
    _i32(out, "sample: out", n)
    chunks = lib().gi_argmax_chunks(vocab)
    part_m = torch.empty(n * chunks, dtype=torch.float32, device=logits.device)
    part_s = torch.empty(n * chunks, dtype=torch.float64, device=logits.device)
    kept = torch.empty(n * vocab, dtype=torch.float32, device=logits.device)
    tops = torch.empty(n * lib().gi_sample_filtered_histogram_bytes() // 8, dtype=torch.int64, device=logits.device)
    _call("gi_sample_filtered", logits.data_ptr(), temperature.data_ptr(), top_k.data_ptr(), top_p.data_ptr(), uniform.data_ptr(),
          out.data_ptr(), part_m.data_ptr(), part_s.data_ptr(), kept.data_ptr(), tops.data_ptr(), n, vocab, logits.stride(0), _stream())
    return out


# ------------------------------------------------------------------------------------------------ probes
def _timed_ms(launch, repeats):
    """Median time of `launch()` over `repeats` runs, by device events, after one run that is not timed."""
    launch()
    times = []
    for _ in range(repeats):
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        launch()
        stop.record()
        stop.synchronize()
        times.append(start.elapsed_time(stop))
    return sorted(times)[len(times) // 2]


# (workgroups of 256 threads per compute unit, loads of 16 bytes in flight per thread) of the plain read.  On an MI355X few
# waves with many loads each read fastest (measured over 1 to 64 workgroups a unit and 4, 8, 16 loads: 6.3 TB/s with one
# workgroup and 8 loads, 6.2 with two and 4; 5.3 to 5.8 with 4 to 16 workgroups; 6.0 with 32 and 64); a copy reaches 5.1 to 5.3.
STREAM_SHAPES = ((1, 8), (2, 4), (1, 16), (64, 4))


def measured_read_bandwidth(device="cuda:0", n_bytes: int = 2 << 30, repeats: int = 5, copy: bool = False, shapes=STREAM_SHAPES) -> float:
    """GB/s at which a plain kernel of this library reads `n_bytes` of device memory (much more than the caches hold);
    with `copy`, reads and writes them (bytes moved = 2 * n_bytes): the best of a few shapes of the kernel (`STREAM_SHAPES`)."""
    src = torch.empty(n_bytes // 4, dtype=torch.int32, device=device).fill_(1)
    dst = torch.empty_like(src) if copy else None
    best = 0.0
    for blocks_per_unit, in_flight in shapes:
        n_blocks = lib().gi_compute_units() * blocks_per_unit
        sink = torch.empty(n_blocks * 256, dtype=torch.int32, device=device)
        ms = _timed_ms(lambda: _call("gi_probe_stream", src.data_ptr(), _ptr(dst), n_bytes, sink.data_ptr(), n_blocks, in_flight, _stream()), repeats)
        best = max(best, (2 if copy else 1) * n_bytes / (ms * 1e-3) / 1e9)
    return best


def measured_mfma_rate(device="cuda:0", iters: int = 20000, repeats: int = 5) -> float:
    """TFLOP/s of a loop of bfloat16 matrix instructions (32x32x16, eight independent sums a wave, eight waves a compute unit)."""
    n_blocks = 256 * 2
    sink = torch.empty(n_blocks * 256, dtype=torch.float32, device=device)
    ms = _timed_ms(lambda: _call("gi_probe_mfma", iters, sink.data_ptr(), n_blocks, _stream()), repeats)
    return lib().gi_probe_mfma_flops(iters, n_blocks) / (ms * 1e-3) / 1e12


def heads_product(a, w, out, n_heads, out_head_stride=None):
    """out[t, h*stride + n] = sum_k a[t, h*k_dim + k] * w[h, n, k] for every head in one launch, on the matrix cores: a bfloat16
    [rows, heads*k_dim], w bfloat16 [heads, n_out, k_dim] contiguous, out [rows, >= heads*stride] bfloat16 or float32 (stride: n_out
    if not given).  False, and nothing done, where the kernel does not take the operands (the caller then multiplies head by head)."""
    _dev(a, w, out)
    rows, k_dim, n_out = a.shape[0], w.shape[2], w.shape[1]
    stride = int(out_head_stride or n_out)
    if not (a.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and w.is_contiguous() and w.shape[0] == n_heads and a.shape[1] == n_heads * k_dim and a.stride(1) == 1
            and out.stride(1) == 1 and out.dtype in (torch.bfloat16, torch.float32) and k_dim % 8 == 0 and a.stride(0) % 8 == 0 and a.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0
            and out.shape[0] == rows and out.shape[1] >= (n_heads - 1) * stride + n_out):
        return False
    if _profile is not None:
        _profile.note = (f"{n_heads}x{n_out}x{k_dim}", w.numel() * w.element_size())
    _call("gi_heads_product", a.data_ptr(), a.stride(0), w.data_ptr(), out.data_ptr(), _code(out, "heads_product: out"), out.stride(0), stride, rows, n_heads, k_dim, n_out, _stream())
    return True


@lru_cache(maxsize=None)
def latent_attention_bf16_supports(kd, vd, page_size) -> bool:
    return bool(lib().gi_latent_attention_supports(kd, vd, page_size))


def latent_attention_prepare():
    """Once, outside any captured pass: the prompt kernel's LDS (more than the default limit) is asked for."""
    if lib().gi_latent_attention_tiles_prepare() != 0:
        raise KernelError(lib().gi_last_error().decode())


def latent_attention_bf16(q, cache, out, ctx, table, n_heads, kd, vd, page_size, window=None, scale=1.0):
    """Attention of a step's rows over latent pages (one key/value head for all query heads: keys [place][kd], then the values
    [vd][place]) on the matrix cores; q bfloat16 [n, heads*kd], out bfloat16 [n, heads*vd].  The rows of prompts go by the attention
    plan's tiles: a workgroup takes a few consecutive rows with all their heads and stages the keys they see once in LDS.  Single
    rows, and the rows of short portions, are a wave per 16 heads and share of their context each; with few of them the context is
    shared out further and a second kernel adds the shares."""
    _dev(q, cache, out, table)
    n = q.shape[0]
    if not (q.dtype == torch.bfloat16 and cache.dtype == torch.bfloat16 and out.dtype == torch.bfloat16 and q.shape == (n, n_heads * kd) and q.is_contiguous()
            and out.shape == (n, n_heads * vd) and out.is_contiguous()):
        raise KernelError("latent_attention: q must be bfloat16 [n, heads*kd] and out bfloat16 [n, heads*vd], contiguous, over a bfloat16 cache")
    _check_paged(cache, table, "latent_attention")
    _i32(ctx.row_pos, "latent_attention: positions", n)
    _i32(ctx.row_slot, "latent_attention: slots", n)
    plan = _plan_of(ctx)                  # (its longest contexts are the bracket's in a captured pass: the same for every replay)
    by_tiles = plan.n_tiles > 0 and bool(lib().gi_latent_attention_tiles_supports(n_heads, kd, vd, int(page_size)))
    if by_tiles:
        _call("gi_latent_attention_tiles_bf16", q.data_ptr(), cache.data_ptr(), out.data_ptr(), plan.tiles.data_ptr(), plan.n_tiles, plan.tile, table.data_ptr(),
              table.stride(0), cache.stride(0), int(page_size), n_heads, kd, vd, int(window or 0), float(scale), _stream())
        if not plan.n_decode:
            return out
        n_single, rows, span = plan.n_decode, plan.decode_rows, plan.max_decode_context
    else:
        n_single, rows, span = n, None, max(plan.max_decode_context, plan.max_tile_context, 1)
    if window:
        span = min(span, int(window) + 31)
    groups = n_single * (-(-n_heads // 16))
    n_splits = max(1, min(16, 2048 // groups, (span + 63) // 64))
    n_part = n_single * n_heads * n_splits * (vd + 2) if n_splits > 1 else 0
    part = torch.empty(n_part, dtype=torch.float32, device=out.device) if n_part else None
    _call("gi_latent_attention_bf16", q.data_ptr(), cache.data_ptr(), out.data_ptr(), _ptr(part), n_part, _ptr(rows), ctx.row_pos.data_ptr(), ctx.row_slot.data_ptr(),
          table.data_ptr(), table.stride(0), cache.stride(0), int(page_size), n_single, n_heads, kd, vd, int(window or 0), float(scale), n_splits, _stream())
    return out


# --------------------------------------------------------------------------- rows side by side, weighted sums, a vector on every row
def _f32_rows(t, what, n=None, width=None):
    if t is None:
        return
    if not (t.dtype == torch.float32 and t.dim() == 2 and t.stride(1) == 1 and (n is None or t.shape[0] == n) and (width is None or t.shape[1] == width)):
        raise KernelError(f"{what} must be float32 [{n if n is not None else 'n'}, {width if width is not None else 'width'}] with unit inner stride")


def concat_rows(a, b, out):
    """out[t] = [a[t]; b[t]] (b None: a alone), float32 rows stored as `out`'s dtype."""
    _dev(a, b, out)
    n, wa = a.shape
    wb = 0 if b is None else b.shape[1]
    _f32_rows(a, "concat_rows: a")
    _f32_rows(b, "concat_rows: b", n)
    if not (out.shape == (n, wa + wb) and out.stride(1) == 1):
        raise KernelError("concat_rows: out must be [n, columns of both] with unit inner stride")
    _call("gi_concat_rows", a.data_ptr(), a.stride(0), wa, _ptr(b), b.stride(0) if b is not None else 0, wb, out.data_ptr(), _code(out, "concat_rows: out"),
          out.stride(0), n, _stream())
    return out


def add_weighted(x, a, scale_a, b=None, scale_b=0.0):
    """x += scale_a * a + scale_b * b (float32 rows; b may be None)."""
    _dev(x, a, b)
    n, dim = x.shape
    _f32_rows(x, "add_weighted: x")
    _f32_rows(a, "add_weighted: a", n, dim)
    _f32_rows(b, "add_weighted: b", n, dim)
    _call("gi_add_weighted", x.data_ptr(), x.stride(0), a.data_ptr(), a.stride(0), float(scale_a), _ptr(b), b.stride(0) if b is not None else 0, float(scale_b), n, dim, _stream())
    return x


def add_vector(x, v):
    """x[t] += v for every row."""
    _dev(x, v)
    n, dim = x.shape
    _f32_rows(x, "add_vector: x")
    if not (v.shape == (dim,) and v.is_contiguous()):
        raise KernelError("add_vector: the vector must be [dim], contiguous")
    _call("gi_add_vector", x.data_ptr(), x.stride(0), v.data_ptr(), _code(v, "add_vector: v"), n, dim, _stream())
    return x


def gate_token_columns(u, table, first, tokens, out, activation="gelu_tanh"):
    """out[t, c] = act(u[t, c]) * table[tokens[t], first + c]."""
    _dev(u, table, tokens, out)
    n, dim = u.shape
    _f32_rows(u, "gate_token_columns: u")
    if activation not in ACTIVATIONS:
        raise KernelError(f"gate_token_columns: unknown activation {activation!r}; known: {', '.join(ACTIVATIONS)}")
    if not (table.dim() == 2 and table.stride(1) == 1 and 0 <= first and first + dim <= table.shape[1] and out.shape == (n, dim) and out.stride(1) == 1):
        raise KernelError("gate_token_columns: the table must hold the columns asked for, out must be [n, dim]")
    _i32(tokens, "gate_token_columns: tokens", n)
    _call("gi_gate_token_columns", u.data_ptr(), u.stride(0), table.data_ptr(), _code(table, "gate_token_columns: table"), table.stride(0), int(first), tokens.data_ptr(),
          out.data_ptr(), _code(out, "gate_token_columns: out"), out.stride(0), n, dim, ACTIVATIONS[activation], _stream())
    return out


def gate_token_columns_rows(x, w, table, first, tokens, out, activation="gelu_tanh"):
    """out[t, j] = act(w[j] . x[t]) * table[tokens[t], first + j] in one launch, for a few rows: x float32 [n, width], read as a product
    reads rows (rounded to bfloat16 where w is bfloat16); w [dim, width]; out [n, dim] of w's dtype."""
    _dev(x, w, table, tokens, out)
    n, width = x.shape
    dim = w.shape[0]
    _f32_rows(x, "gate_token_columns_rows: x")
    if activation not in ACTIVATIONS:
        raise KernelError(f"gate_token_columns_rows: unknown activation {activation!r}; known: {', '.join(ACTIVATIONS)}")
    if not (w.shape == (dim, width) and w.stride(1) == 1 and table.dim() == 2 and table.stride(1) == 1 and 0 <= first and first + dim <= table.shape[1]
            and out.shape == (n, dim) and out.stride(1) == 1 and w.dtype == table.dtype == out.dtype):
        raise KernelError("gate_token_columns_rows: w [dim, width], a table that holds the columns asked for and out [n, dim], all of one dtype, are needed")
    _i32(tokens, "gate_token_columns_rows: tokens", n)
    _call("gi_gate_token_columns_rows", x.data_ptr(), x.stride(0), w.data_ptr(), _code(w, "gate_token_columns_rows: w"), w.stride(0), width, table.data_ptr(),
          _code(table, "gate_token_columns_rows: table"), table.stride(0), int(first), tokens.data_ptr(), out.data_ptr(), _code(out, "gate_token_columns_rows: out"),
          out.stride(0), n, dim, ACTIVATIONS[activation], 1 if w.dtype == torch.bfloat16 else 0, _stream())
    return out


# ------------------------------------------------------------------------------------------------------------ the selective scan
SSM_MAX_TAPS, SSM_MAX_STATES = 16, 256


def ssm_state_floats(inner, n_state, n_taps) -> int:
    """32-bit numbers of one request's state: S [inner][n_state], then the convolution's last n_taps - 1 inputs [n_taps - 1][inner]."""
    return inner * n_state + (n_taps - 1) * inner


def _ssm_state(state, inner, n_state, n_taps, what):
    if not (state.dtype == torch.float32 and state.dim() == 2 and state.stride(1) == 1 and state.shape[1] >= ssm_state_floats(inner, n_state, n_taps)):
        raise KernelError(f"{what}: the state must be float32 [slots, {ssm_state_floats(inner, n_state, n_taps)}]")


def ssm_conv(pre, taps, bias, ctx_slots, ctx_positions, state, x, x_low, n_state, move_tail=False):
    """x = SiLU(convolution of `pre` [n, inner] over each request's rows + bias), float32, and the same once more as `x_low`'s dtype
    (None: not).  taps float32 [inner, n_taps]; rows before a step come from the request's state.  move_tail: a step of single rows,
    whose kernel also moves every request's tail on."""
    _dev(pre, taps, bias, ctx_slots, ctx_positions, state, x, x_low)
    n, inner = x.shape
    n_taps = taps.shape[1]
    _f32_rows(pre, "ssm_conv: the projection", n, inner)
    if not (x.dtype == torch.float32 and x.is_contiguous() and (x_low is None or (x_low.shape == (n, inner) and x_low.is_contiguous()))):
        raise KernelError("ssm_conv: x (and its copy) must be [n, inner], contiguous")
    if not (taps.dtype == torch.float32 and taps.shape == (inner, n_taps) and taps.is_contiguous() and bias.dtype == torch.float32 and bias.shape == (inner,) and bias.is_contiguous()):
        raise KernelError("ssm_conv: taps must be float32 [inner, taps] and the bias float32 [inner]")
    if not 1 <= n_taps <= SSM_MAX_TAPS:
        raise KernelError(f"ssm_conv: {n_taps} taps are outside what the kernel takes (1 to {SSM_MAX_TAPS})")
    _ssm_state(state, inner, n_state, n_taps, "ssm_conv")
    _i32(ctx_slots, "ssm_conv: slots", n)
    _i32(ctx_positions, "ssm_conv: positions", n)
    _call("gi_ssm_conv", pre.data_ptr(), pre.stride(0), taps.data_ptr(), n_taps, bias.data_ptr(), state.data_ptr(), state.stride(0), 1 if move_tail else 0,
          ctx_slots.data_ptr(), ctx_positions.data_ptr(), x.data_ptr(), _ptr(x_low), _code(x_low, "ssm_conv: copy") if x_low is not None else F32, n, inner, n_state, _stream())


def ssm_tail(pre, n_taps, seg_start, seg_len, row_slot, state, inner, n_state):
    """Every request's last n_taps - 1 convolution inputs, moved on behind `ssm_conv`."""
    _dev(pre, seg_start, seg_len, row_slot, state)
    _f32_rows(pre, "ssm_tail: the projection", None, inner)
    _ssm_state(state, inner, n_state, n_taps, "ssm_tail")
    _call("gi_ssm_tail", pre.data_ptr(), pre.stride(0), n_taps, seg_start.data_ptr(), seg_len.data_ptr(), seg_start.numel(), row_slot.data_ptr(), state.data_ptr(),
          state.stride(0), inner, n_state, _stream())


SSM_CHUNK_ROWS = 64            # rows of a chunk where a long run of rows is cut into chunks that run at once
SSM_CHUNKS_FROM = 128          # rows of a step's longest request from which that is done


def ssm_scan(x, dt_pre, dt_bias, low, b_off, c_off, z, a_log, d_skip, seg_start, seg_len, row_slot, state, out, n_state, rows_per_request=None, out_scale=1.0, dt_proj=None):
    """The recurrence over every request's rows, from its state slot and back into it; out [n, inner] = (read-out + D x) * SiLU(z).
    x float32 [n, inner] contiguous; dt_pre, z float32 [n, inner] (any row stride); low float32 [n, >= offsets + n_state] holds B and
    C of every row at the two offsets; dt_bias, d_skip float32 [inner]; a_log float32 [inner, n_state].
    rows_per_request: the requests' numbers of rows as the host knows them (what seg_len holds).  Given, with results stored as
    bfloat16 and a request of SSM_CHUNKS_FROM rows or more, the rows are cut into chunks of SSM_CHUNK_ROWS that run at once (every
    chunk from a zero state first, then the states the chunks start from, then every chunk with its results): the same sums in
    another order, so the results differ by 32-bit rounding from those of rows taken one after the other.
    out_scale multiplies what is stored.
    dt_proj = (w_dt, offset) with dt_pre None: the kernel makes the step sizes' product itself, dt_pre = low[:, offset : offset + rank] @
    w_dt.T, w_dt bfloat16 [inner, rank]; for steps of a few rows whose results are stored as bfloat16."""
    _dev(x, dt_pre, dt_bias, low, z, a_log, d_skip, seg_start, seg_len, row_slot, state, out)
    n, inner = x.shape
    w_dt, dt_off = dt_proj if dt_proj is not None else (None, 0)
    if (dt_pre is None) == (w_dt is None):
        raise KernelError("ssm_scan: either the step sizes or the matrix that makes them")
    if w_dt is not None:
        _dev(w_dt)
        if not (w_dt.dtype == torch.bfloat16 and w_dt.dim() == 2 and w_dt.shape[0] == inner and w_dt.stride(1) == 1 and out.dtype == torch.bfloat16
                and 0 <= dt_off and dt_off + w_dt.shape[1] <= low.shape[1]):
            raise KernelError("ssm_scan: the step sizes' matrix must be bfloat16 [inner, rank], its columns within `low`, the results bfloat16")
        if rows_per_request is None or max(rows_per_request) != 1:
            raise KernelError("ssm_scan: the step sizes' product inside the kernel is for steps of single rows (rows_per_request says so)")
    else:
        _f32_rows(dt_pre, "ssm_scan: the step sizes", n, inner)
    _f32_rows(z, "ssm_scan: the gate", n, inner)
    _f32_rows(low, "ssm_scan: B and C", n)
    if not (x.dtype == torch.float32 and x.is_contiguous() and out.shape == (n, inner) and out.stride(1) == 1):
        raise KernelError("ssm_scan: x must be float32 [n, inner], contiguous, and out [n, inner]")
    if not 1 <= n_state <= SSM_MAX_STATES or max(b_off, c_off) + n_state > low.shape[1] or min(b_off, c_off) < 0:
        raise KernelError(f"ssm_scan: {n_state} states at columns {b_off} and {c_off} of {low.shape[1]} are outside what the kernel takes")
    for v, shape, name in ((dt_bias, (inner,), "dt_bias"), (d_skip, (inner,), "D"), (a_log, (inner, n_state), "A_log")):
        if not (v.dtype == torch.float32 and v.shape == shape and v.is_contiguous()):
            raise KernelError(f"ssm_scan: {name} must be float32 {list(shape)}")
    _ssm_state(state, inner, n_state, 1, "ssm_scan")
    _i32(row_slot, "ssm_scan: slots", n)
    n_chunks, ends, sums = 0, None, None
    if rows_per_request is not None and out.dtype == torch.bfloat16 and max(rows_per_request) >= SSM_CHUNKS_FROM and w_dt is None:
        if len(rows_per_request) != seg_start.numel() or sum(rows_per_request) != n:
            raise KernelError("ssm_scan: the requests' numbers of rows do not add up to the step's rows")
        n_chunks = sum(-(-int(r) // SSM_CHUNK_ROWS) for r in rows_per_request)
        ends = torch.empty((n_chunks, inner, n_state), dtype=torch.float32, device=x.device)
        sums = torch.empty((n_chunks, inner), dtype=torch.float32, device=x.device)
    _call("gi_ssm_scan", x.data_ptr(), _ptr(dt_pre), dt_pre.stride(0) if dt_pre is not None else 0, dt_bias.data_ptr(), low.data_ptr(), low.stride(0), int(b_off), int(c_off), z.data_ptr(),
          z.stride(0), a_log.data_ptr(), d_skip.data_ptr(), seg_start.data_ptr(), seg_len.data_ptr(), seg_start.numel(), row_slot.data_ptr(), state.data_ptr(),
          state.stride(0), out.data_ptr(), _code(out, "ssm_scan: out"), out.stride(0), inner, n_state, n_chunks, SSM_CHUNK_ROWS, _ptr(ends), _ptr(sums), float(out_scale),
          _ptr(w_dt), w_dt.stride(0) if w_dt is not None else 0, int(dt_off), w_dt.shape[1] if w_dt is not None else 0,
          1 if rows_per_request is not None and max(rows_per_request) == 1 else 0, _stream())
    return out


# ------------------------------------------------------------------------------------------------------------------ routed experts
ROUTER_SCORES = {"sigmoid": 0, "softmax": 1}
ROUTER_MAX_EXPERTS, ROUTER_MAX_TOP = 1024, 64
EXPERT_ROW_GROUP = 16          # rows of a group where an expert's gates and up products lie in one matrix (`interleave_gate_up`)
EXPERT_TILE_ROWS = 128         # rows of a tile of the product for grouped rows (the library's gi_experts_tile_rows)
EXPERTS_GROUPED_FROM = 8       # (row, choice) items from which the experts' rows are grouped for the matrix cores


def _router_groups(what, n_experts, top, groups):
    n_groups, keep = (1, 1) if groups is None else (int(groups[0]), int(groups[1]))
    if not (n_groups >= 1 and n_experts % n_groups == 0 and 1 <= keep <= n_groups and top <= keep * (n_experts // n_groups)):
        raise KernelError(f"{what}: {n_experts} experts in {n_groups} groups of which {keep} are kept cannot give {top} a row")
    return n_groups, keep


def route_top(logits, top, ids, weights, score="sigmoid", renormalize=False, groups=None, floor=0.0):
    """ids int32 [n, top], weights float32 [n, top]: per row the `top` experts with the largest scores (the lower index wins a tie)
    and their scores, divided by their sum + `floor` if `renormalize`.  groups = (count, keep): the experts form `count` equal groups
    of neighbours, a group scores what its best expert scores, and only experts of the `keep` best groups can be chosen."""
    _dev(logits, ids, weights)
    n, n_experts = logits.shape
    _f32_rows(logits, "route_top: logits")
    if score not in ROUTER_SCORES:
        raise KernelError(f"route_top: unknown score {score!r}; known: {', '.join(ROUTER_SCORES)}")
    if not (1 <= top <= min(n_experts, ROUTER_MAX_TOP) and n_experts <= ROUTER_MAX_EXPERTS):
        raise KernelError(f"route_top: top {top} of {n_experts} experts is outside what the kernel takes")
    if not (ids.dtype == torch.int32 and ids.shape == (n, top) and ids.is_contiguous() and weights.dtype == torch.float32 and weights.shape == (n, top) and weights.is_contiguous()):
        raise KernelError("route_top: ids must be int32 [n, top] and weights float32 [n, top], contiguous")
    _call("gi_route_top", logits.data_ptr(), logits.stride(0), n, n_experts, top, ROUTER_SCORES[score], 1 if renormalize else 0, float(floor),
          *_router_groups("route_top", n_experts, top, groups), ids.data_ptr(), weights.data_ptr(), _stream())


def _expert_stack(w, rows, cols, what):
    if not (w.dim() == 3 and w.shape[1:] == (rows, cols) and w.is_contiguous()):
        raise KernelError(f"{what} must be [experts, {rows}, {cols}], contiguous")


def experts_gate_up(h, w_gate, w_up, ids, weights, mid, weigh_input=True, activation="silu", limit=0.0):
    """mid[(row, choice)] = act(W_gate[e] a) * (W_up[e] a), a = the row of h (times the choice's weight if `weigh_input`, stored as
    h's dtype), e = ids[row, choice]; one wave per output, for the few rows of decoding steps.  w_up None: w_gate is one stack
    [experts, 2 ff, width] of 16 gate rows, the 16 up rows of the same outputs, and so on (`interleave_gate_up` per expert)."""
    _dev(h, w_gate, w_up, ids, weights, mid)
    n, width = h.shape
    top = ids.shape[1]
    group = 0 if w_up is not None else EXPERT_ROW_GROUP
    ff = w_gate.shape[1] if w_up is not None else w_gate.shape[1] // 2
    _expert_stack(w_gate, ff if w_up is not None else 2 * ff, width, "experts_gate_up: the gates")
    if w_up is not None:
        _expert_stack(w_up, ff, width, "experts_gate_up: the up products")
    elif ff % EXPERT_ROW_GROUP:
        raise KernelError(f"experts_gate_up: gates and up products in one stack come in groups of {EXPERT_ROW_GROUP} rows")
    if not (h.stride(1) == 1 and mid.shape == (n * top, ff) and mid.stride(1) == 1 and (w_up is None or w_gate.dtype == w_up.dtype) and ids.dtype == torch.int32
            and ids.is_contiguous() and ids.shape == (n, top) and weights.dtype == torch.float32 and weights.shape == (n, top) and weights.is_contiguous()):
        raise KernelError("experts_gate_up: h [n, width], mid [n * top, ff], ids int32 and weights float32 [n, top] are needed")
    _call("gi_experts_gate_up", h.data_ptr(), _code(h, "experts_gate_up: h"), h.stride(0), w_gate.data_ptr(), _ptr(w_up), _code(w_gate, "experts_gate_up: weights"),
          ids.data_ptr(), weights.data_ptr(), 1 if weigh_input else 0, mid.data_ptr(), _code(mid, "experts_gate_up: mid"), mid.stride(0), n, top, width, ff,
          ACTIVATIONS[activation], float(limit), group, _stream())
    return mid


def experts_down(mid, w_down, ids, weights, x, accumulate=True, weigh_output=False):
    """x[row] (+)= sum over the row's choices of W_down[e] mid[(row, choice)] (times the choice's weight if `weigh_output`)."""
    _dev(mid, w_down, ids, weights, x)
    n, width = x.shape
    top, ff = ids.shape[1], w_down.shape[2]
    _expert_stack(w_down, width, ff, "experts_down: the down products")
    _f32_rows(x, "experts_down: x")
    if not (mid.shape == (n * top, ff) and mid.stride(1) == 1 and ids.dtype == torch.int32 and ids.shape == (n, top) and ids.is_contiguous()
            and weights.dtype == torch.float32 and weights.shape == (n, top) and weights.is_contiguous()):
        raise KernelError("experts_down: mid [n * top, ff], ids int32 and weights float32 [n, top] are needed")
    _call("gi_experts_down", mid.data_ptr(), _code(mid, "experts_down: mid"), mid.stride(0), w_down.data_ptr(), _code(w_down, "experts_down: weights"), ids.data_ptr(),
          weights.data_ptr(), 1 if weigh_output else 0, x.data_ptr(), x.stride(0), 1 if accumulate else 0, n, top, width, ff, _stream())
    return x


def route_rows(h, router, top, ids, weights, score="sigmoid", renormalize=False, logits=None, groups=None, floor=0.0, extra=None):
    """The router's product and its choice in one launch: logits = h @ router.T with 32-bit sums in an order that the width alone
    fixes, then as `route_top` (with its `groups` and `floor`).  logits: float32 [n, experts] to keep them in, or None.  extra:
    float32 [n, k]: the router's matrix has k more rows behind the experts', whose products with the rows go there (no expert's
    logits: they take no part in the choice)."""
    _dev(h, router, ids, weights, logits, extra)
    n, width = h.shape
    n_extra = 0 if extra is None else extra.shape[1]
    if extra is not None:
        _f32_rows(extra, "route_rows: the products behind the experts'", n)
    n_experts = router.shape[0] - n_extra
    if score not in ROUTER_SCORES:
        raise KernelError(f"route_rows: unknown score {score!r}; known: {', '.join(ROUTER_SCORES)}")
    if not (1 <= top <= min(n_experts, ROUTER_MAX_TOP) and n_experts <= ROUTER_MAX_EXPERTS):
        raise KernelError(f"route_rows: top {top} of {n_experts} experts is outside what the kernel takes")
    if not (h.stride(1) == 1 and router.shape == (n_experts + n_extra, width) and router.stride(1) == 1 and ids.dtype == torch.int32 and ids.shape == (n, top) and ids.is_contiguous()
            and weights.dtype == torch.float32 and weights.shape == (n, top) and weights.is_contiguous()):
        raise KernelError("route_rows: h [n, width], the router [experts, width], ids int32 and weights float32 [n, top] are needed")
    if logits is not None:
        _f32_rows(logits, "route_rows: logits", n, n_experts)
    _call("gi_route_rows", h.data_ptr(), _code(h, "route_rows: h"), h.stride(0), router.data_ptr(), _code(router, "route_rows: the router"), router.stride(0), n, width,
          n_experts, top, ROUTER_SCORES[score], 1 if renormalize else 0, float(floor), *_router_groups("route_rows", n_experts, top, groups), ids.data_ptr(), weights.data_ptr(),
          _ptr(logits), logits.stride(0) if logits is not None else 0, n_extra, _ptr(extra), extra.stride(0) if extra is not None else 0, _stream())


def gemm_bf16_grouped(a, w, out, tile_group, gated=False, gate_limit=0.0):
    """out[rows of tile t] = a[rows of tile t] @ w[tile_group[t]].T for every tile t of 128 rows with tile_group[t] >= 0: bfloat16 on
    the matrix cores.  a [m, k] with m a multiple of 128, w [groups, n, k], out float32 or bfloat16 [m, n], or, gated (as
    `gemm_bf16`), bfloat16 [m, n / 2].  Tiles with a negative entry are left as they are."""
    _dev(a, w, out, tile_group)
    m, k = a.shape
    n = w.shape[1]
    if not (a.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and w.dim() == 3 and w.shape[2] == k and w.is_contiguous() and a.stride(1) == 1 and out.stride(1) == 1
            and out.shape == (m, n // 2 if gated else n) and m % EXPERT_TILE_ROWS == 0):
        raise KernelError("gemm_bf16_grouped: a bfloat16 [m, k] (m a multiple of 128), w bfloat16 [groups, n, k] and out [m, n] (gated: [m, n / 2]) are needed")
    _i32(tile_group, "gemm_bf16_grouped: the tiles' groups", m // EXPERT_TILE_ROWS)
    if gated and gated is not True and gated not in ACTIVATIONS:
        raise KernelError(f"gemm_bf16_grouped: unknown activation {gated!r} of a gated product")
    gate_code = 0 if not gated else 1 + (0 if gated is True else ACTIVATIONS[gated])
    if _profile is not None:
        _profile.note = (f"{m}x{n}x{k}{' gated' if gated else ''}", 0)
    _call("gi_gemm_bf16_grouped", a.data_ptr(), w.data_ptr(), out.data_ptr(), _code(out, "gemm_bf16_grouped: out"), gate_code, float(gate_limit), m, n, k, a.stride(0), w.stride(1),
          out.stride(0), tile_group.data_ptr(), w.stride(0), _stream())
    return out


def experts_grouped_supported(h, w_gate, w_up, w_down) -> bool:
    """Whether `routed_experts` can take many rows through the product for grouped rows: bfloat16 throughout, gates and up products
    in one stack, and sizes the tiles take."""
    if w_up is not None or not (h.dtype == w_gate.dtype == w_down.dtype == torch.bfloat16):
        return False
    width, ff = h.shape[1], w_down.shape[2]
    return width % 64 == 0 and ff % 64 == 0 and width >= 128 and 2 * ff >= 128 and h.stride(0) % 8 == 0 and h.data_ptr() % 16 == 0


def routed_experts(h, w_gate, w_up, w_down, ids, weights, x, accumulate=True, weigh="input", activation="silu", limit=0.0):
    """x[row] (+)= sum over the row's choices of expert(a): the whole mixture behind the router's choice.  weigh "input": a = weight * h[row]
    (stored as h's dtype); "output": a = h[row] and the weight multiplies the expert's result.  w_up None: w_gate holds both (see
    `experts_gate_up`).  Few items, or 32-bit operands: every item walks its expert's matrices.  Many in bfloat16: the items' rows are
    put in the order of their experts and all experts' products are two launches on the matrix cores."""
    if weigh not in ("input", "output"):
        raise KernelError(f"routed_experts: the weights weigh an expert's 'input' or its 'output', not {weigh!r}")
    n, top = ids.shape
    n_experts, width = w_down.shape[0], w_down.shape[1]
    ff = w_down.shape[2]
    if n * top >= EXPERTS_GROUPED_FROM and activation in FUSED_GATE_ACTIVATIONS and experts_grouped_supported(h, w_gate, w_up, w_down):
        _dev(h, w_gate, w_down, ids, weights, x)
        _f32_rows(x, "routed_experts: x", n, width)
        if not (ids.dtype == torch.int32 and ids.is_contiguous() and weights.dtype == torch.float32 and weights.shape == (n, top) and weights.is_contiguous()
                and w_gate.shape == (n_experts, 2 * ff, width) and h.shape == (n, width)):
            raise KernelError("routed_experts: ids int32 and weights float32 [n, top], gates and up products [experts, 2 ff, width] are needed")
        tile = EXPERT_TILE_ROWS
        n_tiles = max(1, (n * top + n_experts * (tile - 1)) // tile)
        dev = h.device
        book = torch.empty(n_experts + n * top + n_tiles, dtype=torch.int32, device=dev)
        count, place, tile_expert = book[:n_experts], book[n_experts:n_experts + n * top], book[n_experts + n * top:]
        _call("gi_experts_place", ids.data_ptr(), n * top, n_experts, count.data_ptr(), place.data_ptr(), tile_expert.data_ptr(), n_tiles, _stream())
        rows = torch.empty((n_tiles * tile, width), dtype=torch.bfloat16, device=dev)
        _call("gi_experts_gather", h.data_ptr(), h.stride(0), place.data_ptr(), weights.data_ptr(), 1 if weigh == "input" else 0, n, top, rows.data_ptr(), rows.stride(0),
              width, _stream())
        mid = torch.empty((n_tiles * tile, ff), dtype=torch.bfloat16, device=dev)
        gemm_bf16_grouped(rows, w_gate, mid, tile_expert, gated=True if activation == "silu" else activation, gate_limit=limit)
        y = torch.empty((n_tiles * tile, width), dtype=torch.float32, device=dev)
        gemm_bf16_grouped(mid, w_down, y, tile_expert)
        _call("gi_experts_combine", y.data_ptr(), y.stride(0), place.data_ptr(), weights.data_ptr(), 1 if weigh == "output" else 0, n, top, x.data_ptr(), x.stride(0),
              width, 1 if accumulate else 0, _stream())
        return x
    mid_dtype = torch.float32 if w_down.dtype == torch.float32 else h.dtype
    mid = torch.empty((n * top, ff), dtype=mid_dtype, device=h.device)
    experts_gate_up(h, w_gate, w_up, ids, weights, mid, weigh_input=weigh == "input", activation=activation, limit=limit)
    experts_down(mid, w_down, ids, weights, x, accumulate=accumulate, weigh_output=weigh == "output")
    return x


# ---------------------------------------------------------------- several copies of the residual stream, the row before a row
def streams_max() -> int:
    return lib().gi_streams_max()


def streams_spread(x0, x, n_streams):
    """Every one of the n copies in x [rows, n * width] <- x0 [rows, width] (float32)."""
    _dev(x0, x)
    rows, width = x0.shape
    _f32_rows(x0, "streams_spread: the rows", rows, width)
    _f32_rows(x, "streams_spread: the copies", rows, n_streams * width)
    _call("gi_streams_spread", x0.data_ptr(), x0.stride(0), x.data_ptr(), x.stride(0), rows, n_streams, width, _stream())
    return x


def streams_norm_shift(x, n_streams, out, *, read=None, norm_weight=None, eps=0.0, shift=None, state=None, positions=None, slots=None, mode=1):
    """x float32 [rows, n * width]: u = sum_s read[s] x_s (read None: the plain sum), h = norm_weight * u / sqrt(mean(u^2) + eps)
    (norm_weight None: h = u), and, with `shift` float32 [width], out = h + (h_before - h) * shift with h_before the h of the
    request's row before (zeros at position 0; the step's previous row, or the request's slot of `state` float32 [slots, width]).
    mode 1 writes out, mode 2 lets every request's last row of the step write its h into its slot, 3 both: in one launch only if
    every request brings one row."""
    _dev(x, out, read, norm_weight, shift, state, positions, slots)
    rows = x.shape[0]
    width = x.shape[1] // n_streams
    _f32_rows(x, "streams_norm_shift: x", rows, n_streams * width)
    if not 1 <= n_streams <= streams_max():
        raise KernelError(f"streams_norm_shift: 1 to {streams_max()} copies of the stream are taken, not {n_streams}")
    if mode & 1 and not (out is not None and out.shape == (rows, width) and out.stride(1) == 1):
        raise KernelError("streams_norm_shift: out must be [rows, width] with unit inner stride")
    for v, n, what in ((read, n_streams, "the copies' weights"), (shift, width, "the blend's weights")):
        if v is not None and not (v.dtype == torch.float32 and v.is_contiguous() and v.numel() == n):
            raise KernelError(f"streams_norm_shift: {what} must be float32 [{n}]")
    if norm_weight is not None and not (norm_weight.shape == (width,) and norm_weight.is_contiguous()):
        raise KernelError("streams_norm_shift: the norm's weights must be [width]")
    if shift is not None:
        if not (state is not None and state.dtype == torch.float32 and state.dim() == 2 and state.shape[1] == width and state.stride(1) == 1):
            raise KernelError("streams_norm_shift: the state must be float32 [slots, width]")
        _i32(positions, "streams_norm_shift: positions", rows)
        _i32(slots, "streams_norm_shift: slots", rows)
    elif mode != 1:
        raise KernelError("streams_norm_shift: without a blend there is no state to write")
    _call("gi_streams_norm_shift", x.data_ptr(), x.stride(0), n_streams, width, _ptr(read), _ptr(norm_weight), _code(norm_weight, "streams_norm_shift: norm") if norm_weight is not None else F32,
          float(eps), _ptr(shift), _ptr(state), state.stride(0) if state is not None else 0, _ptr(positions), _ptr(slots), _ptr(out) if mode & 1 else None,
          _code(out, "streams_norm_shift: out") if out is not None else F32, out.stride(0) if out is not None else width, rows, int(mode), _stream())
    return out


def streams_write(x, n_streams, y, mix, write, mult=1.0):
    """x float32 [rows, n * width] in place: copy t <- sum_s mix[s, t] copy_s + mult * write[t] * y, all copies at once from the old
    ones; mix float32 [n, n] (None: every copy keeps itself), write float32 [n] (None: ones), y float32 [rows, width]."""
    _dev(x, y, mix, write)
    rows = x.shape[0]
    width = x.shape[1] // n_streams
    _f32_rows(x, "streams_write: x", rows, n_streams * width)
    _f32_rows(y, "streams_write: y", rows, width)
    if not 1 <= n_streams <= streams_max():
        raise KernelError(f"streams_write: 1 to {streams_max()} copies of the stream are taken, not {n_streams}")
    if mix is not None and not (mix.dtype == torch.float32 and mix.is_contiguous() and mix.shape == (n_streams, n_streams)):
        raise KernelError("streams_write: the mixing matrix must be float32 [n, n]")
    if write is not None and not (write.dtype == torch.float32 and write.is_contiguous() and write.numel() == n_streams):
        raise KernelError("streams_write: the writing weights must be float32 [n]")
    _call("gi_streams_write", x.data_ptr(), x.stride(0), n_streams, width, y.data_ptr(), y.stride(0), _ptr(mix), _ptr(write), float(mult), rows, _stream())
    return x


def streams_write_norm_takes(n_streams, width) -> bool:
    """Whether `streams_write_norm` takes these sizes (a few copies, a width the kernel keeps in registers)."""
    return bool(lib().gi_streams_write_norm_takes(int(n_streams), int(width)))


def streams_write_norm(x, n_streams, y, mix, write, mult, read, norm_weight, eps, out):
    """`streams_write` and, of the new copies, out = norm_weight * u / sqrt(mean(u^2) + eps) with u = sum_t read[t] x_t (read None: the
    plain sum): a half's result into the copies and the next half's input out of them, in one kernel."""
    _dev(x, y, mix, write, read, norm_weight, out)
    rows = x.shape[0]
    width = x.shape[1] // n_streams
    _f32_rows(x, "streams_write_norm: x", rows, n_streams * width)
    _f32_rows(y, "streams_write_norm: y", rows, width)
    if not streams_write_norm_takes(n_streams, width):
        raise KernelError(f"streams_write_norm: {n_streams} copies of {width} channels are not taken")
    if mix is not None and not (mix.dtype == torch.float32 and mix.is_contiguous() and mix.shape == (n_streams, n_streams)):
        raise KernelError("streams_write_norm: the mixing matrix must be float32 [n, n]")
    for v, what in ((write, "writing"), (read, "reading")):
        if v is not None and not (v.dtype == torch.float32 and v.is_contiguous() and v.numel() == n_streams):
            raise KernelError(f"streams_write_norm: the {what} weights must be float32 [n]")
    if not (norm_weight.shape == (width,) and norm_weight.is_contiguous() and out.shape == (rows, width) and out.stride(1) == 1):
        raise KernelError("streams_write_norm: the norm's weights must be [width] and out [rows, width]")
    if x.stride(0) % 4 or y.stride(0) % 4 or out.stride(0) % 4 or x.data_ptr() % 16 or y.data_ptr() % 16 or out.data_ptr() % 16:
        raise KernelError("streams_write_norm: rows must start at multiples of 16 bytes")
    _call("gi_streams_write_norm", x.data_ptr(), x.stride(0), n_streams, width, y.data_ptr(), y.stride(0), _ptr(mix), _ptr(write), float(mult), _ptr(read),
          norm_weight.data_ptr(), _code(norm_weight, "streams_write_norm: norm"), float(eps), out.data_ptr(), _code(out, "streams_write_norm: out"), out.stride(0), rows, _stream())
    return out


def head_gate(a, gate, n_heads, vd):
    """a [rows, heads * vd] in place: head h of row t multiplied by sigmoid(gate[t, h]); gate float32 [rows, >= heads] (unit inner stride)."""
    _dev(a, gate)
    rows = a.shape[0]
    if not (a.shape == (rows, n_heads * vd) and a.stride(1) == 1 and gate.dtype == torch.float32 and gate.dim() == 2 and gate.shape[0] == rows and gate.shape[1] >= n_heads
            and gate.stride(1) == 1):
        raise KernelError("head_gate: a must be [rows, heads*vd] and the gates float32 [rows, heads], with unit inner stride")
    _call("gi_head_gate", a.data_ptr(), _code(a, "head_gate: a"), a.stride(0), gate.data_ptr(), gate.stride(0), rows, n_heads, vd, _stream())
    return a


def add_rows_gated(x, y, g):
    """x[t] += sigmoid(g[t]) * y[t]; x, y float32 [rows, width], g float32 [rows] (any stride)."""
    _dev(x, y, g)
    rows, width = x.shape
    _f32_rows(x, "add_rows_gated: x", rows, width)
    _f32_rows(y, "add_rows_gated: y", rows, width)
    if not (g.dtype == torch.float32 and g.numel() == rows and g.dim() <= 2):
        raise KernelError("add_rows_gated: the gates must be float32, one a row")
    _call("gi_add_rows_gated", x.data_ptr(), x.stride(0), y.data_ptr(), y.stride(0), g.data_ptr(), g.stride(0), rows, width, _stream())
    return x
