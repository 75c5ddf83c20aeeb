"""`torch.library` registration of the fused VQ GEMM, so that graphs traced by `torch.compile` /
`torch.export` can hold it as one opaque node:

    torch.ops.vq_gemm_amd.vq_linear(x, codes, codebook, bias=None) -> Tensor

`x` is fp16 [..., K], `codes` [N, K/vec] uint8/uint16, `codebook` fp16 [E, vec] or [G, E, vec],
`bias` fp16 [N] or None; the result is fp16 [..., N].  The device implementation calls the HIP
library through its C ABI (the current stream, no synchronisation); the fake implementation only
propagates shapes.  There is no CPU implementation: CPU tensors are refused.
"""
from __future__ import annotations

from typing import Optional

import torch

from . import cabi


# What the automatic choice wants as scratch for a shape (bytes; 0 for all but the split-K shapes), remembered per shape and
# state of the tuning table, and one scratch buffer per device and stream, grown on demand: a layer's forward makes neither
# a host-side cost-model pass nor an allocation per call.  (Launches on one stream run in order, so they can share the buffer.)
_ws_need: dict = {}
_ws_pool: dict = {}


def _workspace_for(M, K, N, v, E, G, bits, device):
    key = (M, K, N, v, E, G, bits, cabi.tuning_generation)
    need = _ws_need.get(key)
    if need is None:
        if len(_ws_need) > 4096:
            _ws_need.clear()
        need = _ws_need[key] = cabi.workspace_bytes_b(M, K, N, v, E, G, bits, cabi.VARIANT_AUTO)
    if need <= 0:
        return None
    slot = (device.index, torch.cuda.current_stream(device).cuda_stream)
    ws = _ws_pool.get(slot)
    if ws is None or ws.numel() < need:
        ws = _ws_pool[slot] = torch.empty(need, dtype=torch.uint8, device=device)
    return ws


def _out_shape(x: torch.Tensor, codes: torch.Tensor, codebook: torch.Tensor):
    if codes.dim() != 2 or codebook.dim() not in (2, 3) or x.dim() < 1:
        raise ValueError("vq_linear: x [..., K], codes [N, K/vec], codebook [E, vec] or [G, E, vec]")
    if codes.dtype not in (torch.uint8, torch.uint16):
        raise ValueError(f"vq_linear: codes must be uint8 or uint16, got {codes.dtype}")
    if x.shape[-1] != codes.shape[1] * codebook.shape[-1]:
        raise ValueError(f"vq_linear: x has {x.shape[-1]} features, codes x vec give {codes.shape[1] * codebook.shape[-1]}")
    return (*x.shape[:-1], codes.shape[0])


@torch.library.custom_op("vq_gemm_amd::vq_linear", mutates_args=(), device_types="cuda")
def vq_linear(x: torch.Tensor, codes: torch.Tensor, codebook: torch.Tensor,
              bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    shape = _out_shape(x, codes, codebook)
    if x.dtype != torch.float16 or codebook.dtype != torch.float16:
        raise ValueError("vq_linear: x and codebook must be float16")
    x2 = x.reshape(-1, x.shape[-1]).contiguous()
    codes, codebook = codes.contiguous(), codebook.contiguous()
    bias = None if bias is None else bias.contiguous()
    g, e, v = cabi._cb_dims(codebook)
    ws = _workspace_for(x2.shape[0], x2.shape[1], codes.shape[0], v, e, g, 8 * codes.element_size(), x2.device)
    if ws is None:
        # (no kernel the automatic choice would take wants scratch for this shape: the plain entry point)
        return cabi.e2e_gemm_b(x2, codes, codebook, bias=bias).view(shape)
    # the entry point with a sized workspace: the automatic choice may split K
    return cabi.e2e_gemm_b_ws(x2, codes, codebook, bias=bias, workspace=ws).view(shape)


@vq_linear.register_fake
def _vq_linear_fake(x, codes, codebook, bias=None):
    return x.new_empty(_out_shape(x, codes, codebook))


@torch.library.custom_op("vq_gemm_amd::vq_linear_packed", mutates_args=(), device_types="cuda")
def vq_linear_packed(x: torch.Tensor, codes_packed: torch.Tensor, codebook: torch.Tensor,
                     bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """`vq_linear` on a code matrix in the decode kernel's packed layout (`cabi.pack_codes_b`):
    the decode kernel only, for the shapes `cabi.decode_packed_supports` accepts."""
    shape = _out_shape(x, codes_packed, codebook)
    if x.dtype != torch.float16 or codebook.dtype != torch.float16:
        raise ValueError("vq_linear_packed: x and codebook must be float16")
    x2 = x.reshape(-1, x.shape[-1]).contiguous()
    y = cabi.e2e_gemm_b(x2, codes_packed.contiguous(), codebook.contiguous(), variant=cabi.VARIANT_DECODE_PACKED,
                        bias=None if bias is None else bias.contiguous())
    return y.view(shape)


@vq_linear_packed.register_fake
def _vq_linear_packed_fake(x, codes_packed, codebook, bias=None):
    return x.new_empty(_out_shape(x, codes_packed, codebook))


@torch.library.custom_op("vq_gemm_amd::silu_mul", mutates_args=(), device_types="cuda")
def silu_mul(gate_up: torch.Tensor) -> torch.Tensor:
    """silu(gate_up[..., :N]) * gate_up[..., N:] for fp16 gate_up [..., 2N]."""
    if gate_up.dtype != torch.float16 or gate_up.shape[-1] % 2 != 0:
        raise ValueError("silu_mul: expected an fp16 tensor with an even last dimension")
    a = gate_up.reshape(-1, gate_up.shape[-1]).contiguous()
    return cabi.silu_mul(a).view(*gate_up.shape[:-1], gate_up.shape[-1] // 2)


@silu_mul.register_fake
def _silu_mul_fake(gate_up):
    if gate_up.shape[-1] % 2 != 0:
        raise ValueError("silu_mul: expected an even last dimension")
    return gate_up.new_empty((*gate_up.shape[:-1], gate_up.shape[-1] // 2))


@torch.library.custom_op("vq_gemm_amd::vq_gated_linear", mutates_args=(), device_types="cuda")
def vq_gated_linear(x: torch.Tensor, codes: torch.Tensor, codebook: torch.Tensor,
                    bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """silu(x @ Wg.T) * (x @ Wu.T) in one fused VQ GEMM: `codes` [2H, K/vec] hold the gate and the up rows
    interleaved in groups of 16 (`vq_gemm_amd.quantize.interleave_gate_up`), the result is fp16 [..., H].  Every
    fused kernel carries the epilogue, so no call allocates a workspace."""
    shape = _out_shape(x, codes, codebook)
    if x.dtype != torch.float16 or codebook.dtype != torch.float16:
        raise ValueError("vq_gated_linear: x and codebook must be float16")
    if codes.shape[0] % 32 != 0:
        raise ValueError("vq_gated_linear: the interleaved gate/up rows come in whole groups of 32")
    x2 = x.reshape(-1, x.shape[-1]).contiguous()
    y = cabi.e2e_gemm_b_gated(x2, codes.contiguous(), codebook.contiguous(), bias=None if bias is None else bias.contiguous())
    return y.view(*shape[:-1], shape[-1] // 2)


@vq_gated_linear.register_fake
def _vq_gated_linear_fake(x, codes, codebook, bias=None):
    shape = _out_shape(x, codes, codebook)
    return x.new_empty((*shape[:-1], shape[-1] // 2))
