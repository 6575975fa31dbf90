"""GEMM operands derived from a quantised linear's stored state, shared by the dynamic and the static module.

The GEMM reads the weight as bytes ``[N, pad128(K)]`` and the weight scale as an fp32 vector ``[N]``.  The stored
state (``qweight`` [N, K], ``weight_scale`` [1, N] or [1]) already has that form when K is a multiple of 128 and the
scale is per channel; otherwise a zero-padded copy / the scalar written out per channel is kept beside the state,
never saved, rebuilt when the state changes, and built ahead of the first forward wherever the state is set
(conversion, ``load_state_dict``, ``.to(device)``).
"""
from __future__ import annotations

import torch
from torch import Tensor

from ... import ops


def _capturing(t: Tensor) -> bool:
    return t.device.type == "cuda" and torch.cuda.is_current_stream_capturing()


def _refresh_after_load(module, incompatible_keys) -> None:
    module.refresh_derived()


class DerivedOperands:
    """Mixin for a module with ``qweight``, ``weight_scale`` and ``out_features``."""

    def _init_derived(self) -> None:
        self._packed = None  # (key, K-padded byte view of qweight)
        self._sw_vec = None  # (key, per-tensor weight scale once per output channel)
        self.register_load_state_dict_post_hook(_refresh_after_load)

    def _apply(self, fn, recurse=True):
        out = super()._apply(fn, recurse)  # .to(device) / .cuda(): the derived operands follow the state
        if not torch.compiler.is_compiling():
            self.refresh_derived()
        return out

    def refresh_derived(self) -> None:
        """Builds the derived operands now, so that a forward launches nothing but its kernels.  A module that
        does not live on a ROCm device (yet) builds them at its first forward there."""
        self._packed = self._sw_vec = None
        if self.qweight.device.type == "cuda":
            self._gemm_weight()
            self._weight_scale_vector()

    def _gemm_weight(self) -> Tensor:
        """qweight as the byte matrix [N, pad128(K)] the GEMM reads."""
        qw = self.qweight.detach()
        if qw.dtype != torch.int8:
            qw = qw.view(torch.uint8)
        k = qw.shape[1]
        kp = ops.pad_k(k)
        if kp == k and qw.is_contiguous():
            return qw
        if ops.is_tracing(qw):
            # a traced graph cannot key a cache on the storage address: pad inside the graph
            return torch.nn.functional.pad(qw, (0, kp - k)).contiguous()
        key = (self.qweight.data_ptr(), self.qweight._version, str(qw.device))
        if self._packed is None or self._packed[0] != key:
            buf = torch.zeros((qw.shape[0], kp), dtype=qw.dtype, device=qw.device)
            buf[:, :k] = qw
            if _capturing(qw):
                # recorded, not executed: the buffer belongs to the graph's pool and holds data only after a
                # replay, so it must not be kept for later eager calls
                return buf
            self._packed = (key, buf)
        return self._packed[1]

    def _weight_scale_vector(self) -> Tensor:
        """weight_scale as the fp32 [N] vector the GEMM reads."""
        ws = self.weight_scale
        if ws.numel() != 1:
            return ws.view(-1)
        if ops.is_tracing(ws):
            return ops.broadcast_f32(ws.reshape(1).contiguous(), self.out_features)
        key = (ws.data_ptr(), ws._version, str(ws.device))
        if self._sw_vec is None or self._sw_vec[0] != key:
            vec = ops.broadcast_f32(ws.reshape(1).contiguous(), self.out_features)
            if _capturing(ws):
                return vec
            self._sw_vec = (key, vec)
        return self._sw_vec[1]

    def _check_device(self, dev) -> None:
        if self.qweight.device != dev:
            raise RuntimeError(f"Expected all tensors to be on the same device, but the input is on {dev} and this "
                               f"module's qweight on {self.qweight.device} (move the quantised model with .to(device))")
