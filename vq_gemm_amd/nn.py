"""`VQLinear`: a linear layer whose weight is held as codes + codebooks and multiplied by the
fused VQ GEMM (geometry B), the call site after the path.

Inference only (no gradient flows to codes or codebooks).  The product runs in the HIP library
through its C ABI, the optional bias is added inside the kernel before the result is rounded; the
call is registered with `torch.library` (`torch.ops.vq_gemm_amd.vq_linear`) so that a traced graph
holds it as one node.  Nothing falls back to the CPU.
"""
from __future__ import annotations

import torch

from . import cabi
from .quantize import kmeans_quantize, residual_quantize
from .torch_ops import silu_mul, vq_gated_linear, vq_linear, vq_linear_packed


class VQLinear(torch.nn.Module):
    """y = x @ W.T + bias with W[n, j*vec + t] = codebook[n // (N/G)][codes[n, j]][t].

    With `k_repeat` = S > 1 the codes hold S additive stages side by side along K (see
    `vq_gemm_amd.quantize.residual_quantize`): the layer's weight is the sum of the S [N, K] blocks of
    the dequantised [N, S*K] matrix, and the input is repeated S times along K before the one fused
    GEMM, so that all stages accumulate in the same fp32 sums.
    """

    def __init__(self, codes: torch.Tensor, codebook: torch.Tensor, bias: torch.Tensor | None = None, k_repeat: int = 1):
        super().__init__()
        if codes.dtype not in (torch.uint8, torch.uint16) or codes.dim() != 2:
            raise ValueError("codes must be a [N, K/vec] uint8 or uint16 tensor")
        if codebook.dtype != torch.float16 or codebook.dim() not in (2, 3):
            raise ValueError("codebook must be an fp16 [E, vec] or [G, E, vec] tensor")
        self.register_buffer("codes", codes.contiguous())
        self.register_buffer("codebook", codebook.contiguous())
        self.register_buffer("bias", None if bias is None else bias.to(torch.float16).contiguous())
        if k_repeat < 1 or (codes.shape[1] * codebook.shape[-1]) % k_repeat != 0:
            raise ValueError("k_repeat must divide the dequantised row length")
        self.k_repeat = k_repeat
        self.out_features = codes.shape[0]
        self.in_features = codes.shape[1] * codebook.shape[-1] // k_repeat
        if self.bias is not None and self.bias.shape != (self.out_features,):
            raise ValueError("bias must have one entry per output feature")
        self.register_buffer("codes_packed", None, persistent=False)  # derived from `codes`: not part of the state
        self._packed_from = None  # (version counter, address) of `codes` when `codes_packed` was made

    def prepack_for_decode(self) -> "VQLinear":
        """Keep a second copy of the codes in the decode kernel's packed layout (`cabi.pack_codes_b`;
        as large as the codes, 1/16 of the fp16 weight for 8-vectors with 8-bit codes).  Inputs short
        enough for the decode kernel then read that copy: one contiguous run per wave load instead
        of sixteen row pieces, 10-25 % less time once a workgroup has several tiles, the same result
        bit for bit.  Taller inputs keep using the plain matrix."""
        try:
            self.codes_packed = cabi.pack_codes_b(self.codes, self.codebook.shape[-1])
        except cabi.VqGemmError as e:
            raise ValueError("the packed layout needs K % 256 == 0, out_features % 16 == 0 and vec in (2, 4, 8)") from e
        self._packed_from = self._codes_key()
        return self

    def _codes_key(self):
        # (a tensor made under torch.inference_mode() keeps no version counter and cannot be updated in
        # place outside that mode: its address, shape and device identify its contents)
        c = self.codes
        version = -1 if c.is_inference() else c._version
        return (version, c.data_ptr(), tuple(c.shape), str(c.device))

    def _fresh_packed_codes(self):
        """The packed copy, re-made first if `codes` changed since it was packed (`load_state_dict`,
        an in-place update, a move to another device): short and tall inputs must multiply by the
        same weights."""
        if self._packed_from != self._codes_key() or self.codes_packed.device != self.codes.device:
            self.prepack_for_decode()
        return self.codes_packed

    @classmethod
    def from_float(cls, weight: torch.Tensor, vec: int = 8, entries: int = 256, n_codebooks: int = 1,
                   bias: torch.Tensor | None = None, iters: int = 10, seed: int = 0, residual_stages: int = 1) -> "VQLinear":
        """Quantise an fp16 weight [N, K] on the GPU (Lloyd iterations around the HIP encoder), in
        `residual_stages` additive stages of `entries` vectors each."""
        if residual_stages > 1:
            codes, codebook, _ = residual_quantize(weight.to(torch.float16), vec, entries, residual_stages, n_codebooks,
                                                   iters, seed)
            return cls(codes, codebook, bias, k_repeat=residual_stages)
        codes, codebook, _ = kmeans_quantize(weight.to(torch.float16), vec, entries, n_codebooks, iters, seed)
        return cls(codes, codebook, bias)

    def dequantized_weight(self) -> torch.Tensor:
        """The weight the layer multiplies by, [N, K] fp16 (the fp32 sum of the stages, rounded once)."""
        w = cabi.dequant_b(self.codes, self.codebook)
        if self.k_repeat == 1:
            return w
        return w.view(self.out_features, self.k_repeat, self.in_features).float().sum(dim=1).half()

    @torch.no_grad()
    def forward(self, x: torch.Tensor) -> torch.Tensor:
        if x.dtype != torch.float16 or x.shape[-1] != self.in_features:
            raise ValueError(f"expected an fp16 input with {self.in_features} features")
        if self.k_repeat > 1:
            x = x.repeat(*([1] * (x.dim() - 1)), self.k_repeat)
        if self.codes_packed is not None:
            g, e, v = cabi._cb_dims(self.codebook)
            dims = (x.numel() // x.shape[-1], x.shape[-1], self.out_features, v, e, g, 8 * self.codes.element_size())
            if cabi.select_variant_b(*dims) == cabi.VARIANT_DECODE and cabi.decode_packed_supports(*dims):
                return vq_linear_packed(x, self._fresh_packed_codes(), self.codebook, self.bias)
        return vq_linear(x, self.codes, self.codebook, self.bias)

    def extra_repr(self) -> str:
        g = 1 if self.codebook.dim() == 2 else self.codebook.shape[0]
        return (f"in_features={self.in_features}, out_features={self.out_features}, vec={self.codebook.shape[-1]}, "
                f"entries={self.codebook.shape[-2]}, codebooks={g}, stages={self.k_repeat}, bias={self.bias is not None}")


class VQGatedMLP(torch.nn.Module):
    """down(silu(x @ Wg.T) * (x @ Wu.T)) with all three weights vector-quantised.

    `gate_up` holds the gate rows and the up rows of the pair as one [2*H, K] weight.  With `interleaved=True`
    (what `from_float` builds) they alternate in groups of 16 rows (`vq_gemm_amd.quantize.interleave_gate_up`) and one
    fused VQ GEMM with the gated epilogue gives silu(gate) * up directly: the [M, 2*H] product never exists in
    memory.  With `interleaved=False` the gate rows are stacked on the up rows: the plain fused GEMM writes both
    products and an element-wise kernel follows.  `down` ([K_out, H]) is an ordinary `VQLinear`.
    """

    def __init__(self, gate_up: VQLinear, down: VQLinear, interleaved: bool = False):
        super().__init__()
        if gate_up.out_features % 2 != 0 or gate_up.out_features // 2 != down.in_features:
            raise ValueError("gate_up must have twice as many output features as down has input features")
        if interleaved and (gate_up.out_features % 32 != 0 or gate_up.k_repeat != 1):
            raise ValueError("the interleaved layout needs a multiple of 32 gate_up rows and a single quantisation stage")
        self.gate_up = gate_up
        self.down = down
        self.interleaved = interleaved

    @classmethod
    def from_float(cls, gate: torch.Tensor, up: torch.Tensor, down: torch.Tensor, vec: int = 8, entries: int = 256,
                   n_codebooks: int = 1, iters: int = 10, seed: int = 0) -> "VQGatedMLP":
        """Quantise fp16 weights gate [H, K], up [H, K], down [K_out, H]; the pair is interleaved for the gated epilogue."""
        from .quantize import interleave_gate_up
        gu = VQLinear.from_float(interleave_gate_up(gate.to(torch.float16), up.to(torch.float16)), vec, entries, n_codebooks,
                                 None, iters, seed)
        return cls(gu, VQLinear.from_float(down, vec, entries, n_codebooks, None, iters, seed + 1), interleaved=True)

    @torch.no_grad()
    def forward(self, x: torch.Tensor) -> torch.Tensor:
        if self.interleaved:
            gu = self.gate_up
            if x.dtype != torch.float16 or x.shape[-1] != gu.in_features:
                raise ValueError(f"expected an fp16 input with {gu.in_features} features")
            return self.down(vq_gated_linear(x, gu.codes, gu.codebook, gu.bias))
        return self.down(silu_mul(self.gate_up(x)))
