"""Packed MXFP4 tensors as objects, and their file format.

The real-kernel path of the reference keeps three byte tensors per quantized operand -- ``e2m1 [M, K/2]``,
``e8m0 [M, K/32]`` and clip-mask bits ``[M, K/8]`` (notebooks/benchmark_mxfp4.ipynb, ``fusedQuantizeMx_op`` and
``CudaGemm.forward``'s ``ctx.save_for_backward``) -- and hands them to QuTLASS / FP-Quant style consumers
(README.md, "Quantized inference").  This module gives those tensors a documented layout, a container and a
(de)serialiser so that saved activations, weights and checkpoints can be exchanged.

Format (version 1)
  * ``e2m1``  uint8 ``[R, C/2]``: byte ``j`` of row ``r`` holds element ``2j`` in its low nibble and ``2j+1`` in its
    high nibble; a nibble is sign (bit 3) and magnitude code 0..7 for 0, .5, 1, 1.5, 2, 3, 4, 6 (OCP MX E2M1).
    With ``layout = "tiled"`` the same bytes are stored as ``[R/16][C/128][16 rows][64 bytes]`` (what the GEMM of
    this library reads fastest); ``to_layout`` converts either way.
  * ``e8m0``  uint8 ``[R, C/32]``: biased exponent of the group of 32 elements; the group's scale is
    ``2^(byte - 127)``, times 4/3 (the fp32 value of ``1 / 0.75``) when ``scale_kind = "absmax"``.
  * ``mask``  uint8 ``[R, C/8]`` (optional): bit ``i`` of byte ``j`` is 1 where element ``8j + i`` was not clipped.
  * values are those of the *rotated* tensor ``x.view(-1, hd) @ H`` with ``H = hd^-1/2 * Sylvester * diag(signs)``;
    ``hadamard_dim`` and ``sign_bits`` (bit ``j`` set = column ``j`` negated) say which rotation.

A file is a ``safetensors`` archive with entries ``<name>.e2m1``, ``<name>.e8m0``, ``<name>.mask`` and one JSON
metadata string (key ``quartet_mxfp4``) carrying the attributes of every tensor.

``scales_to_blocked`` / ``scales_from_blocked`` convert the plain scale matrix to and from the 128 x 4 blocked
order that NVIDIA block-scaled GEMMs (and QuTLASS's ``to_blocked``) take.  QuTLASS is not part of the reference's
sources, so that order follows NVIDIA's published description of the layout rather than reference code.
"""
import ctypes
import json
from dataclasses import dataclass
from typing import Dict, Optional

import torch

from . import _lib
from . import kernels as K

FORMAT_VERSION = 1
_METADATA_KEY = "quartet_mxfp4"
_LAYOUTS = ("rowmajor", "tiled")
_SCALE_KINDS = ("quest", "absmax")


@dataclass
class PackedTensor:
    """One quantized ``[rows, cols]`` operand; see the module docstring for the meaning of each field."""
    codes: torch.Tensor
    scales: torch.Tensor
    maskbits: Optional[torch.Tensor]
    rows: int
    cols: int
    layout: str = "rowmajor"
    hadamard_dim: int = 32
    sign_bits: int = 0
    scale_kind: str = "quest"

    def __post_init__(self):
        if self.layout not in _LAYOUTS:
            raise ValueError(f"layout must be one of {_LAYOUTS}, got {self.layout!r}")
        if self.scale_kind not in _SCALE_KINDS:
            raise ValueError(f"scale_kind must be one of {_SCALE_KINDS}, got {self.scale_kind!r}")
        if self.cols % 32 or self.rows < 0:
            raise ValueError(f"a packed tensor needs cols % 32 == 0, got [{self.rows}, {self.cols}]")
        if self.layout == "tiled" and (self.rows % 16 or self.cols % 128):
            raise ValueError(f"the tiled layout needs rows % 16 == 0 and cols % 128 == 0, got [{self.rows}, {self.cols}]")
        want = {"codes": (self.rows, self.cols // 2), "scales": (self.rows, self.cols // 32),
                "maskbits": (self.rows, self.cols // 8)}
        for name, shape in want.items():
            t = getattr(self, name)
            if t is None and name == "maskbits":
                continue
            if t.dtype != torch.uint8 or tuple(t.shape) != shape:
                raise ValueError(f"{name} must be uint8 of shape {shape}, got {t.dtype} {tuple(t.shape)}")

    @property
    def post_scale(self):
        """What ``code * 2^(e8m0 - 127)`` is multiplied by to give the value."""
        return K.FOUR_THIRDS if self.scale_kind == "absmax" else 1.0

    def to_layout(self, layout):
        """Same tensor with its code bytes in the other order (a permutation of bytes; any device)."""
        if layout not in _LAYOUTS:
            raise ValueError(f"layout must be one of {_LAYOUTS}, got {layout!r}")
        if layout == self.layout:
            return self
        if (self.rows % 16 or self.cols % 128) and layout == "tiled":
            raise ValueError(f"the tiled layout needs rows % 16 == 0 and cols % 128 == 0, got [{self.rows}, {self.cols}]")
        codes = K.tile_codes(self.codes) if layout == "tiled" else K.untile_codes(self.codes)
        return PackedTensor(codes, self.scales, self.maskbits, self.rows, self.cols, layout, self.hadamard_dim,
                            self.sign_bits, self.scale_kind)

    def to(self, device):
        mv = lambda t: None if t is None else t.to(device)
        return PackedTensor(mv(self.codes), mv(self.scales), mv(self.maskbits), self.rows, self.cols, self.layout,
                            self.hadamard_dim, self.sign_bits, self.scale_kind)

    def clip_mask(self):
        """Boolean ``[rows, cols]`` mask (True = kept), or None when no mask was stored."""
        if self.maskbits is None:
            return None
        shifts = torch.arange(8, device=self.maskbits.device, dtype=torch.uint8)
        return ((self.maskbits[..., None] >> shifts) & 1).bool().view(self.rows, self.cols)

    def dequantize(self, dtype=torch.float32):
        """Values of the rotated tensor (GPU kernel)."""
        rm = self.to_layout("rowmajor")
        return K.dequantize_mxfp4(rm.codes.contiguous(), rm.scales.contiguous(), self.post_scale, dtype)

    def reconstruct(self, dtype=torch.float32):
        """De-quantize and undo the rotation: the pseudo-quantized tensor in the original basis (GPU kernels)."""
        return K.masked_hadamard_bwd(self.dequantize(dtype), self.hadamard_dim, dtype, self.sign_bits, None)

    def _attributes(self):
        return {"rows": self.rows, "cols": self.cols, "layout": self.layout, "hadamard_dim": self.hadamard_dim,
                "sign_bits": f"{self.sign_bits:#x}", "scale_kind": self.scale_kind, "mask": self.maskbits is not None}


def pack_quest(x, hadamard_dim=32, sign_bits=0, tiled=False):
    """Forward quantizer of the layer (quest scale, round to nearest, clip mask) on a 2-D GPU tensor."""
    codes, scales, mask, _ = K.quantize_mxfp4(x.contiguous(), hadamard_dim, sign_bits, K.QM_QUEST_RTN, want_mask=True, tiled=tiled)
    return PackedTensor(codes, scales, mask, x.shape[0], x.shape[1], "tiled" if tiled else "rowmajor", hadamard_dim,
                        sign_bits, "quest")


def pack_absmax(x, hadamard_dim=32, sign_bits=0, stochastic=False, seed=0, tiled=False):
    """Gradient-side quantizer (absmax scale, optional stochastic rounding from `seed`) on a 2-D GPU tensor."""
    mode = K.QM_ABSMAX_SR if stochastic else K.QM_ABSMAX_RTN
    codes, scales, _, _ = K.quantize_mxfp4(x.contiguous(), hadamard_dim, sign_bits, mode, seed=seed, tiled=tiled)
    return PackedTensor(codes, scales, None, x.shape[0], x.shape[1], "tiled" if tiled else "rowmajor", hadamard_dim,
                        sign_bits, "absmax")


def from_operand_buffer(buffer, rows, cols, tiled, quantizer):
    """The packed tensor inside one of the byte buffers that ``kernels.linear_forward`` returns (views, no copy): what
    the layer keeps of x or of W for its backward pass.  `quantizer` is the forward quantizer that produced it."""
    off = (ctypes.c_size_t * 3)()
    _lib.check(_lib.lib().qm_packed_operand_offsets(rows, cols, off), "qm_packed_operand_offsets")

    def view(start, width):
        return buffer[start:start + rows * width].view(rows, width)
    return PackedTensor(view(off[0], cols // 2), view(off[1], cols // 32), view(off[2], cols // 8), rows, cols,
                        "tiled" if tiled else "rowmajor", quantizer.hadamard_dim, quantizer.sign_bits, "quest")


def pack_model_weights(model, tiled=False) -> Dict[str, PackedTensor]:
    """Quantized weights of every ``QuantizedLinear`` of `model` whose weight quantizer is the forward MXFP4 quantizer,
    keyed by parameter name (``transformer.h.0.attn.c_attn.weight`` ...): what a layer's forward pass multiplies with,
    ready for ``save_packed`` -- the quantized checkpoint an inference engine with FP4 GEMMs consumes.  Each tensor is
    in its layer's rotated basis (``hadamard_dim``, ``sign_bits``): activations must be rotated the same way."""
    from .linear import QuantizedLinear
    from .quantizers import QuestMXFP4Quantizer
    out = {}
    for name, m in model.named_modules():
        if isinstance(m, QuantizedLinear) and type(m.weight_quantizer) is QuestMXFP4Quantizer and not m.weight_quantizer.is_dense:
            w_q = m.weight_quantizer
            ok = tiled and m.weight.shape[0] % 16 == 0 and m.weight.shape[1] % 128 == 0 and w_q.hadamard_dim == 32
            out[f"{name}.weight"] = pack_quest(m.weight.detach(), w_q.hadamard_dim, w_q.sign_bits, tiled=ok)
    return out


def save_packed(path, tensors: Dict[str, PackedTensor], extra_metadata: Optional[Dict[str, str]] = None):
    """Write packed tensors to a safetensors file."""
    from safetensors.torch import save_file
    blobs, attrs = {}, {}
    for name, t in tensors.items():
        if "." in name and name.rsplit(".", 1)[1] in ("e2m1", "e8m0", "mask"):
            raise ValueError(f"tensor name {name!r} collides with the entry suffixes")
        blobs[f"{name}.e2m1"] = t.codes.detach().cpu().contiguous()
        blobs[f"{name}.e8m0"] = t.scales.detach().cpu().contiguous()
        if t.maskbits is not None:
            blobs[f"{name}.mask"] = t.maskbits.detach().cpu().contiguous()
        attrs[name] = t._attributes()
    metadata = dict(extra_metadata or {})
    metadata[_METADATA_KEY] = json.dumps({"version": FORMAT_VERSION, "tensors": attrs}, sort_keys=True)
    save_file(blobs, str(path), metadata=metadata)


def load_packed(path, device="cpu") -> Dict[str, PackedTensor]:
    """Read a file written by ``save_packed`` (safetensors: nothing in the file is executed)."""
    from safetensors import safe_open
    out = {}
    with safe_open(str(path), framework="pt", device=str(device)) as f:
        meta = f.metadata() or {}
        if _METADATA_KEY not in meta:
            raise ValueError(f"{path} holds no '{_METADATA_KEY}' metadata: not a packed-tensor file")
        desc = json.loads(meta[_METADATA_KEY])
        if desc.get("version") != FORMAT_VERSION:
            raise ValueError(f"{path}: format version {desc.get('version')} is not supported (this reader: {FORMAT_VERSION})")
        for name, a in desc["tensors"].items():
            mask = f.get_tensor(f"{name}.mask") if a["mask"] else None
            out[name] = PackedTensor(f.get_tensor(f"{name}.e2m1"), f.get_tensor(f"{name}.e8m0"), mask, a["rows"], a["cols"],
                                     a["layout"], a["hadamard_dim"], int(a["sign_bits"], 16), a["scale_kind"])
    return out


def scales_to_blocked(scales):
    """Plain ``[R, G]`` scale bytes -> the flat 128 x 4 blocked order of NVIDIA block-scaled GEMMs: rows padded to a
    multiple of 128 and groups to a multiple of 4 (zero bytes), each 128 x 4 block stored as 32 rows of 16 bytes
    where byte ``4 * (r // 32) + g`` of row ``r % 32`` is the scale of block row ``r`` and block column ``g``."""
    R, G = scales.shape
    rb, gb = -(-R // 128), -(-G // 4)
    padded = torch.zeros((rb * 128, gb * 4), dtype=scales.dtype, device=scales.device)
    padded[:R, :G] = scales
    blocks = padded.view(rb, 128, gb, 4).permute(0, 2, 1, 3)
    return blocks.reshape(-1, 4, 32, 4).transpose(1, 2).reshape(-1, 32, 16).flatten()


def scales_from_blocked(blocked, rows, groups):
    """Inverse of ``scales_to_blocked`` for a ``[rows, groups]`` scale matrix."""
    rb, gb = -(-rows // 128), -(-groups // 4)
    if blocked.numel() != rb * gb * 512:
        raise ValueError(f"expected {rb * gb * 512} blocked scale bytes for [{rows}, {groups}], got {blocked.numel()}")
    blocks = blocked.view(-1, 32, 4, 4).transpose(1, 2).reshape(rb, gb, 128, 4).permute(0, 2, 1, 3)
    return blocks.reshape(rb * 128, gb * 4)[:rows, :groups].contiguous()
