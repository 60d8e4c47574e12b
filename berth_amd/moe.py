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
from .device import Exl3Linear, Gpu, InputError, WeightsError, find_linear, read_float_tensor
from .kernels import Codebook, ExpertLinStruct


class StackedLinear:
    """An EXL3 linear that stacks `blocks` equal linears along K: tile rows
    [b * K/16, (b+1) * K/16) and input scales [b * K, (b+1) * K) belong to block b; the output
    scale spans the columns once, or once per block.  `window` copies one block's rows,
    restricted to a column range, into an ordinary linear.  This is how a checkpoint's
    `experts.gate_up_proj` / `experts.down_proj` pair (crates/berth-plan/tests/plan.rs:111-118)
    is read; the reference names those tensors but never opens one, so the stacking order is
    this loader's assumption."""

    def __init__(self, ckpt, prefix: str, blocks: int):
        linear = find_linear(ckpt, prefix)
        if linear.k.is_half():
            raise WeightsError(f"{prefix}: half-integer rate")
        if linear.input_scale.is_packed() or linear.output_scale.is_packed():
            raise WeightsError(f"{prefix}: packed signs in a stacked expert tensor")
        if linear.bias is not None:
            raise WeightsError(f"{prefix}: bias is present and is not applied")
        self.prefix, self.blocks = prefix, blocks
        self.codebook = Codebook(linear.kernel_codebook)
        self.trellis = linear.trellis.read_array(np.uint16)
        tiles_k_all, self.tiles_n, _ = self.trellis.shape
        if blocks < 1 or tiles_k_all % blocks:
            raise WeightsError(f"{prefix}: {tiles_k_all} tile rows do not split into {blocks} experts")
        self.tiles_k = tiles_k_all // blocks
        self.suh = linear.input_scale.tensor.read_array(np.float16).ravel()
        self.svh = linear.output_scale.tensor.read_array(np.float16).ravel()
        n = self.tiles_n * 16
        if self.suh.size != tiles_k_all * 16 or self.svh.size not in (n, n * blocks):
            raise WeightsError(f"{prefix}: scales do not match the stacked tensor")
        self.svh_per_block = blocks > 1 and self.svh.size == n * blocks
        self.size_k, self.size_n = self.tiles_k * 16, n

    def window(self, gpu: Gpu, name: str, block: int, n0: int, n: int) -> Exl3Linear:
        if not 0 <= block < self.blocks or n0 < 0 or n < 16 or n0 % 16 or n % 16 or n0 + n > self.size_n:
            raise WeightsError(f"{self.prefix}: window {name} lies outside the stacked tensor")
        rows = slice(block * self.tiles_k, (block + 1) * self.tiles_k)
        tr = np.ascontiguousarray(self.trellis[rows, n0 // 16:(n0 + n) // 16])
        sv0 = (block * self.size_n if self.svh_per_block else 0) + n0
        return Exl3Linear(gpu, name, tr, self.suh[block * self.size_k:(block + 1) * self.size_k].copy(),
                          self.svh[sv0:sv0 + n].copy(), self.codebook)


class MoeLayer:
    def __init__(self, gpu: Gpu, router: np.ndarray, experts, top_k: int, shared=None,
                 bias: np.ndarray | None = None, renorm: bool = True,
                 codebook: Codebook = Codebook.MUL1, shared_gate: np.ndarray | None = None):
        """router fp16 [H][E]; experts: list of (gate, up, down) Exl3Linear; shared:
        optional (gate, up, down); shared_gate: optional [H] weights of the per-token scale
        sigmoid(x . shared_gate) on the shared expert's row (kept in fp32)."""
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
        self.shared_gate = None
        if shared_gate is not None:
            if not shared:
                raise InputError("moe: a shared-expert gate without a shared expert")
            sg = np.ascontiguousarray(shared_gate, dtype=np.float32).ravel()
            if sg.size != self.hidden:
                raise InputError(f"moe: shared-expert gate has {sg.size} weights for hidden size {self.hidden}")
            self.shared_gate = torch.from_numpy(sg).to(gpu.device)
        self._ws = None
        self._ws_tokens = 0

    @classmethod
    def load(cls, gpu: Gpu, ckpt, layer: int, ffn, renorm: bool = True) -> "MoeLayer":
        """Layer `layer`'s MoE block from a `berth_amd.exl3.Checkpoint`, sized by the plan's
        `Ffn` record (`berth_amd.plan`; crates/berth-plan/src/plan.rs:45-57; tensor names as in
        crates/berth-plan/tests/plan.rs:96-120 and tests/from_exl3_bytes.rs), with
        {mlp} = model.language_model.layers.<layer>.mlp:
          {mlp}.gate.weight                       router, [experts][hidden] in F16 / BF16 / F32 as a
                                                  linear layer stores it; transposed to [hidden][experts]
          {mlp}.experts.<e>.{gate,up,down}_proj   one EXL3 linear per routed expert and projection, or
          {mlp}.experts.{gate_up,down}_proj       the stacked pair (StackedLinear; gate columns, then up)
          {mlp}.shared_expert.{gate,up,down}_proj the always-on expert
          {mlp}.shared_expert_gate.weight         optional [1][hidden] (or [hidden]) in F16 / BF16 / F32:
                                                  the always-on expert's row of token t is scaled by
                                                  sigmoid(x[t] . weight); the reference never opens this
                                                  tensor, so the formula is this loader's assumption
        Refused: a plan layer that is not MoE, sizes that differ from the plan's, a quantized
        router and a bias on an expert linear (the grouped launches have no place for it)."""
        if not ffn.is_moe:
            raise InputError(f"moe: layer {layer} is planned with a dense MLP")
        mlp = f"model.language_model.layers.{layer}.mlp"
        E, I, SI = ffn.router.num_experts, ffn.experts.intermediate_size, ffn.shared.intermediate_size
        if any(lin.prefix == f"{mlp}.gate" for lin in ckpt.linears()):
            raise WeightsError(f"{mlp}.gate: a quantized router is not handled")
        gate = ckpt.tensors.get(f"{mlp}.gate.weight")
        if gate is None:
            raise WeightsError(f"tensor {mlp}.gate.weight is missing")
        if len(gate.shape) != 2 or gate.shape[0] != E:
            raise WeightsError(f"{gate.name}: expected [{E}][hidden]")
        H = int(gate.shape[1])
        router = np.ascontiguousarray(read_float_tensor(gate).reshape(E, H).T.astype(np.float16))
        shared_gate = None
        sgt = ckpt.tensors.get(f"{mlp}.shared_expert_gate.weight")
        if sgt is not None:
            if int(np.prod(sgt.shape)) != H or len(sgt.shape) > 2:
                raise WeightsError(f"{sgt.name}: expected [1][{H}]")
            shared_gate = read_float_tensor(sgt).ravel()

        def checked(prefix, k, n):
            lin = Exl3Linear.load(gpu, ckpt, prefix)
            if (lin.size_k, lin.size_n) != (k, n):
                raise WeightsError(f"{prefix}: {lin.size_k}x{lin.size_n} where the plan has {k}x{n}")
            if lin.bias is not None:
                raise WeightsError(f"{prefix}: bias is present and is not applied")
            return lin

        pool = f"{mlp}.experts"
        experts = []
        if any(lin.prefix == f"{pool}.gate_up_proj" for lin in ckpt.linears()):
            gate_up, down = StackedLinear(ckpt, f"{pool}.gate_up_proj", E), StackedLinear(ckpt, f"{pool}.down_proj", E)
            if (gate_up.size_k, gate_up.size_n, down.size_k, down.size_n) != (H, 2 * I, I, H):
                raise WeightsError(f"{pool}: stacked tensors are {gate_up.size_k}x{gate_up.size_n} and "
                                   f"{down.size_k}x{down.size_n} per expert where the plan has {H}x{2 * I} and {I}x{H}")
            for e in range(E):
                experts.append((gate_up.window(gpu, f"{pool}.{e}.gate_proj", e, 0, I),
                                gate_up.window(gpu, f"{pool}.{e}.up_proj", e, I, I),
                                down.window(gpu, f"{pool}.{e}.down_proj", e, 0, H)))
        else:
            for e in range(E):
                experts.append((checked(f"{pool}.{e}.gate_proj", H, I), checked(f"{pool}.{e}.up_proj", H, I),
                                checked(f"{pool}.{e}.down_proj", I, H)))
        sh = f"{mlp}.shared_expert"
        shared = (checked(f"{sh}.gate_proj", H, SI), checked(f"{sh}.up_proj", H, SI), checked(f"{sh}.down_proj", SI, H))
        g0 = experts[0][0]
        if any(lin.k_bits != g0.k_bits or lin.codebook != g0.codebook for lin in shared):
            raise InputError("moe: the shared expert must use the routed experts' bit rate and codebook")
        return cls(gpu, router, experts, ffn.router.experts_per_tok, shared=shared, renorm=renorm,
                   codebook=g0.codebook, shared_gate=shared_gate)

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
                    self.k_bits, self.codebook, self.renorm, gpu.raw_stream(),
                    None if self.shared_gate is None else self.shared_gate.data_ptr())
