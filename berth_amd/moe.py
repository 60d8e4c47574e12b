"""Host-side owner of one MoE layer's device buffers: the router, E routed
experts of three EXL3 linears each, and an optional always-on shared expert —
the `Ffn::Moe{router, shared, experts}` of crates/berth-plan/src/plan.rs:24-59
with every tensor resident in HBM (the reference's VRAM / pinned-RAM / SSD
placement, crates/berth-plan/src/place.rs:189-232, collapses to "all VRAM" on a
288 GB device)."""
from __future__ import annotations

import ctypes as C

import numpy as np
import torch

from . import kernels as K
from .device import Exl3Linear, Gpu, InputError
from .kernels import Codebook, ExpertLinStruct


class MoeLayer:
    def __init__(self, gpu: Gpu, router: np.ndarray, experts, top_k: int, shared=None,
                 bias: np.ndarray | None = None, renorm: bool = True,
                 codebook: Codebook = Codebook.MUL1):
        """router fp16 [H][E]; experts: list of (gate, up, down) Exl3Linear; shared:
        optional (gate, up, down)."""
        self.hidden, self.num_experts = router.shape
        if len(experts) != self.num_experts:
            raise InputError("moe: router width and expert count differ")
        g0 = experts[0][0]
        self.intermediate = g0.size_n
        self.k_bits = g0.k_bits
        self.codebook = codebook
        self.top_k = top_k
        self.renorm = renorm
        for g, u, d in experts:
            if (g.size_k, g.size_n, u.size_k, u.size_n, d.size_k, d.size_n) != \
               (self.hidden, self.intermediate, self.hidden, self.intermediate, self.intermediate, self.hidden) \
               or g.k_bits != self.k_bits or u.k_bits != self.k_bits or d.k_bits != self.k_bits:
                raise InputError("moe: expert shapes / bit rates must be uniform")
        self.experts = experts
        self.router = gpu.upload(router.view(np.uint16))
        self.bias = None if bias is None else torch.from_numpy(np.ascontiguousarray(bias, dtype=np.float32)).to(gpu.device)
        table = (ExpertLinStruct * (3 * self.num_experts))()
        for e, trio in enumerate(experts):
            for i, lin in enumerate(trio):
                table[3 * e + i] = ExpertLinStruct(lin.trellis.data_ptr(), lin.suh.data_ptr(), lin.svh.data_ptr())
        raw = np.frombuffer(bytes(table), dtype=np.uint8).copy()
        self.table = torch.from_numpy(raw).to(gpu.device)
        self.shared = shared
        self.shared_I = shared[0].size_n if shared else 0
        self._shared_host = None
        if shared:
            arr = (ExpertLinStruct * 3)()
            for i, lin in enumerate(shared):
                arr[i] = ExpertLinStruct(lin.trellis.data_ptr(), lin.suh.data_ptr(), lin.svh.data_ptr())
            self._shared_host = arr
        self._ws = None
        self._ws_tokens = 0

    def trellis_bytes(self) -> int:
        n = sum(lin.trellis_bytes() for trio in self.experts for lin in trio)
        if self.shared:
            n += sum(lin.trellis_bytes() for lin in self.shared)
        return n

    def _workspace(self, gpu: Gpu, T: int):
        if self._ws is None or T > self._ws_tokens:
            nbytes = K.moe.workspace_bytes(T, self.hidden, self.num_experts, self.top_k, self.intermediate,
                                           self.shared_I)
            self._ws = torch.zeros(nbytes, dtype=torch.uint8, device=gpu.device)
            self._ws_tokens = T
        return self._ws

    def forward(self, gpu: Gpu, x: torch.Tensor, out: torch.Tensor, T: int,
                idx_out: torch.Tensor | None = None, w_out: torch.Tensor | None = None) -> None:
        """x fp16 [T][H] -> out fp32 [T][H]."""
        if x.numel() < T * self.hidden or out.numel() < T * self.hidden:
            raise InputError("moe: buffer too small")
        ws = self._workspace(gpu, T)
        K.moe.layer(x.data_ptr(), self.router.data_ptr(), None if self.bias is None else self.bias.data_ptr(),
                    self.table.data_ptr(),
                    None if self._shared_host is None else C.cast(self._shared_host, C.c_void_p),
                    out.data_ptr(), None if idx_out is None else idx_out.data_ptr(),
                    None if w_out is None else w_out.data_ptr(), ws.data_ptr(), ws.numel(),
                    T, self.hidden, self.num_experts, self.top_k, self.intermediate, self.shared_I,
                    self.k_bits, self.codebook, self.renorm, gpu.raw_stream())
