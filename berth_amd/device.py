"""Host-side owners of device buffers for the EXL3 linear path, mirroring
crates/berth-engine/src/device.rs:14-367 (`Gpu`, `Exl3Linear`, `RowScratch`) and
crates/berth-engine/src/mlp.rs:25-334 (`MlpLayer`); `load` constructors read an
EXL3 checkpoint directory through `berth_amd.exl3`.  torch is used for device
memory and the stream only; every computation goes through the C ABI.
"""
from __future__ import annotations

import numpy as np
import torch

from . import kernels as K
from .kernels import Codebook, OutDtype

MAX_RECONSTRUCT_N = 32768   # crates/berth-engine/src/device.rs:193


class InputError(ValueError):
    """crates/berth-engine `Error::Input`."""


class WeightsError(ValueError):
    """crates/berth-engine `Error::Weights`: a checkpoint the engine does not handle."""


def find_linear(ckpt, prefix: str):
    """The checkpoint's EXL3 linear with this prefix (device.rs:167-173)."""
    for lin in ckpt.linears():
        if lin.prefix == prefix:
            return lin
    raise WeightsError(f"{prefix} is not an EXL3 linear")


def read_float_tensor(info) -> np.ndarray:
    """An F16 / BF16 / F32 checkpoint tensor as fp32 values (the dtypes a bias may have:
    crates/berth-exl3/src/linear.rs:219-231)."""
    name = info.dtype.as_str()
    if name == "F32":
        return info.read_array(np.float32).ravel().copy()
    if name == "F16":
        return info.read_array(np.float16).ravel().astype(np.float32)
    if name == "BF16":
        return (info.read_array(np.uint16).ravel().astype(np.uint32) << 16).view(np.float32)
    raise WeightsError(f"{info.name}: expected a float tensor, got {name}")


class Gpu:
    """Device 0 and the stream every launch goes on (device.rs:14-43)."""

    def __init__(self, device: int = 0):
        if not torch.cuda.is_available():
            raise RuntimeError("no HIP device")
        self.device = torch.device("cuda", device)
        torch.cuda.set_device(self.device)
        self.stream = torch.cuda.current_stream(self.device)
        self.sm_count = K.device_sms(device)

    def raw_stream(self):
        """The stream launches go on: torch's current stream of the device (the one
        captured when a HIP graph is being recorded)."""
        return torch.cuda.current_stream(self.device).cuda_stream or None

    def zeroed(self, nbytes: int) -> torch.Tensor:
        return torch.zeros(nbytes, dtype=torch.uint8, device=self.device)

    def upload(self, array: np.ndarray) -> torch.Tensor:
        a = np.ascontiguousarray(array)
        if a.dtype == np.uint16:
            a = a.view(np.int16)
        return torch.from_numpy(a).to(self.device)

    def synchronize(self):
        torch.cuda.synchronize(self.device)


def ptr(t: torch.Tensor) -> int:
    return t.data_ptr()


def _out_dtype(out: OutDtype):
    return torch.float32 if out == OutDtype.F32 else torch.float16


class RowScratch:
    """Scratch shared by every linear of a prefill chunk (device.rs:176-212)."""

    def __init__(self, gpu: Gpu, max_rows: int, max_k: int, max_n: int):
        self.a_had = torch.zeros(max_rows * max_k, dtype=torch.float16, device=gpu.device)
        self.weight = torch.zeros(max_k * min(max_n, MAX_RECONSTRUCT_N), dtype=torch.float16,
                                  device=gpu.device)
        self.max_rows, self.max_k, self.max_n = max_rows, max_k, max_n


class Exl3Linear:
    """One EXL3 linear on the device: trellis, fp16 Hadamard scales, and the
    fp16 scratch the kernel writes the rotated input to (device.rs:77-367)."""

    def __init__(self, gpu: Gpu, prefix: str, trellis: np.ndarray, suh: np.ndarray, svh: np.ndarray,
                 codebook: Codebook = Codebook.MUL1):
        if trellis.ndim != 3 or trellis.shape[2] % 16:
            raise InputError(f"{prefix}: trellis must be (K/16, N/16, 16*bits)")
        self.prefix = prefix
        self.k_bits = trellis.shape[2] // 16
        self.size_k = int(suh.size)
        self.size_n = int(svh.size)
        if trellis.shape[0] * 16 != self.size_k or trellis.shape[1] * 16 != self.size_n:
            raise InputError(f"{prefix}: trellis shape does not match suh / svh")
        self.codebook = codebook
        self.trellis = gpu.upload(trellis.view(np.uint16))
        self.suh = gpu.upload(suh.view(np.uint16))
        self.svh = gpu.upload(svh.view(np.uint16))
        self.a_had = torch.zeros(self.size_k, dtype=torch.float16, device=gpu.device)
        self.bias = None

    @classmethod
    def from_device(cls, prefix: str, trellis: torch.Tensor, suh: torch.Tensor, svh: torch.Tensor, k_bits: int,
                    codebook: Codebook = Codebook.MUL1, a_had: torch.Tensor | None = None) -> "Exl3Linear":
        """Adopt tensors that already live on the device (16-bit element types:
        trellis (K/16)(N/16)(16 k_bits) words, suh [K], svh [N]); a_had may be shared
        between linears that never run concurrently."""
        self = cls.__new__(cls)
        self.prefix, self.k_bits, self.codebook = prefix, int(k_bits), codebook
        self.size_k, self.size_n = int(suh.numel()), int(svh.numel())
        if self.size_k % 128 or self.size_n % 128 or \
           trellis.numel() != (self.size_k // 16) * (self.size_n // 16) * 16 * self.k_bits or \
           trellis.element_size() != 2 or suh.element_size() != 2 or svh.element_size() != 2:
            raise InputError(f"{prefix}: trellis shape does not match suh / svh")
        self.trellis, self.suh, self.svh = trellis, suh, svh
        self.a_had = a_had if a_had is not None else torch.zeros(self.size_k, dtype=torch.float16, device=trellis.device)
        self.bias = None
        return self

    def set_bias(self, gpu: Gpu, bias: np.ndarray) -> None:
        """A bias of `size_n` values, kept in fp32 and added to every output row after the
        linear.  The reference classifies the tensor (crates/berth-exl3/src/linear.rs:131-133)
        and its engine refuses it (mlp.rs:67-75): what is added here follows y = W x + b."""
        if bias.size != self.size_n:
            raise WeightsError(f"{self.prefix}: bias has {bias.size} values for {self.size_n} outputs")
        self.bias = gpu.upload(np.ascontiguousarray(bias, dtype=np.float32).ravel())

    def _add_bias(self, gpu: Gpu, c: torch.Tensor, rows: int, out: OutDtype) -> None:
        if self.bias is not None:
            K.ops.add_bias(ptr(c), ptr(self.bias), rows, self.size_n, out == OutDtype.F32, gpu.raw_stream())

    @classmethod
    def from_packed_signs(cls, gpu: Gpu, prefix: str, trellis: np.ndarray, su: np.ndarray, sv: np.ndarray,
                          codebook: Codebook = Codebook.MUL1) -> "Exl3Linear":
        """A linear stored with packed sign tensors `su` [K/16] / `sv` [N/16] (int16
        words, one bit per channel: crates/berth-exl3/src/linear.rs:122-141): the
        words are uploaded and expanded to fp16 +-1 on the device."""
        halves = []
        for name, words in (("su", su), ("sv", sv)):
            raw = np.ascontiguousarray(words).view(np.uint8).ravel()
            d_raw = torch.from_numpy(raw.copy()).to(gpu.device)
            out = torch.zeros(raw.size * 8, dtype=torch.float16, device=gpu.device)
            K.unpack_signs(ptr(d_raw), ptr(out), raw.size, gpu.raw_stream())
            halves.append(out)
        gpu.synchronize()
        return cls.from_device(prefix, gpu.upload(trellis.view(np.uint16)).reshape(-1), halves[0], halves[1],
                               trellis.shape[2] // 16, codebook)

    @classmethod
    def load(cls, gpu: Gpu, ckpt, prefix: str) -> "Exl3Linear":
        """`<prefix>.trellis`, `.suh` / `.svh` (or packed `.su` / `.sv`, expanded on the
        device) and an optional `.bias` from a `berth_amd.exl3.Checkpoint`
        (device.rs:92-125).  Half-integer rates are refused as in the reference; packed
        signs, which the reference refuses at this point, are accepted."""
        linear = find_linear(ckpt, prefix)
        if linear.k.is_half():
            raise WeightsError(f"{prefix}: half-integer rate")
        halves = []
        for scale in (linear.input_scale, linear.output_scale):
            raw = scale.tensor.read_array(np.uint8).ravel()
            if scale.is_packed():
                d_raw = torch.from_numpy(raw).to(gpu.device)
                out = torch.zeros(raw.size * 8, dtype=torch.float16, device=gpu.device)
                K.unpack_signs(ptr(d_raw), ptr(out), raw.size, gpu.raw_stream())
                gpu.synchronize()
            else:
                out = gpu.upload(raw.view(np.uint16))
            halves.append(out)
        tiles_k, tiles_n, _ = linear.trellis.shape
        if tiles_k * 16 != halves[0].numel() or tiles_n * 16 != halves[1].numel():
            raise WeightsError(f"{prefix}: trellis {tiles_k}x{tiles_n} tiles do not match "
                               f"{halves[0].numel()} x {halves[1].numel()} scales")
        trellis = gpu.upload(linear.trellis.read_array(np.uint16).ravel())
        self = cls.from_device(prefix, trellis, halves[0], halves[1], linear.k.twice // 2,
                               Codebook(linear.kernel_codebook))
        if linear.bias is not None:
            self.set_bias(gpu, read_float_tensor(linear.bias))
        return self

    def trellis_bytes(self) -> int:
        return self.trellis.numel() * 2

    # device.rs:127-165
    def forward(self, gpu: Gpu, a: torch.Tensor, c: torch.Tensor, out: OutDtype) -> None:
        if a.numel() * a.element_size() < self.size_k * 2 or \
           c.numel() * c.element_size() < self.size_n * (4 if out == OutDtype.F32 else 2):
            raise InputError(f"{self.prefix}: buffer too small")
        K.exl3_linear(ptr(a), ptr(self.trellis), ptr(c), ptr(self.suh), ptr(self.a_had), ptr(self.svh),
                      1, self.size_k, self.size_n, self.k_bits, self.codebook, out, gpu.raw_stream())
        self._add_bias(gpu, c, 1, out)

    # device.rs:210-272
    def forward_rows(self, gpu: Gpu, scratch: RowScratch, a: torch.Tensor, c: torch.Tensor, rows: int,
                     out: OutDtype) -> None:
        if rows < 2:
            raise InputError(f"{self.prefix}: forward_rows needs rows > 1")
        if rows > scratch.max_rows or self.size_k > scratch.max_k or self.size_n > scratch.max_n:
            raise InputError(f"{self.prefix}: {rows} x {self.size_k} x {self.size_n} exceeds the row scratch")
        if a.numel() * a.element_size() < rows * self.size_k * 2 or \
           c.numel() * c.element_size() < rows * self.size_n * (4 if out == OutDtype.F32 else 2):
            raise InputError(f"{self.prefix}: buffer too small")
        weight = ptr(scratch.weight) if rows > 144 else None
        K.prefill_lin.exl3_linear(ptr(a), ptr(self.trellis), ptr(c), ptr(self.suh), ptr(scratch.a_had),
                                  ptr(self.svh), weight, rows, self.size_k, self.size_n, self.k_bits,
                                  self.codebook, out, gpu.raw_stream())
        self._add_bias(gpu, c, rows, out)

    # device.rs:288-366
    def forward_n(self, gpu: Gpu, a_had: torch.Tensor, a: torch.Tensor, c: torch.Tensor, rows: int,
                  out: OutDtype) -> None:
        if rows == 1:
            return self.forward(gpu, a, c, out)
        if rows == 0 or rows > 144:
            raise InputError(f"{self.prefix}: forward_n rows {rows} are outside 1..=144")
        need = rows * self.size_k * 2
        if a_had.numel() * a_had.element_size() < need or a.numel() * a.element_size() < need or \
           c.numel() * c.element_size() < rows * self.size_n * (4 if out == OutDtype.F32 else 2):
            raise InputError(f"{self.prefix}: buffer too small")
        if self.k_bits == 6:
            K.exl3_linear(ptr(a), ptr(self.trellis), ptr(c), ptr(self.suh), ptr(a_had), ptr(self.svh),
                          rows, self.size_k, self.size_n, self.k_bits, self.codebook, out, gpu.raw_stream())
        else:
            K.prefill_lin.exl3_linear(ptr(a), ptr(self.trellis), ptr(c), ptr(self.suh), ptr(a_had),
                                      ptr(self.svh), None, rows, self.size_k, self.size_n, self.k_bits,
                                      self.codebook, out, gpu.raw_stream())
        self._add_bias(gpu, c, rows, out)


class Exl3MultiLinear:
    """Several EXL3 linears that share one input, launched as one sliced
    `exl3_mgemm` (the qkv bundles of crates/berth-engine/src/attn.rs:1934-1973 and
    gdn.rs:1102-1130; list layout from crates/berth-kernels/src/ops.rs:264-293):
    every source is cut into slices of the greatest common width.  Any row count: one
    row runs the streaming kernel, 2..8 the dot-product kernel, more the MFMA kernels
    (the reference sends 9..32 rows through the same call, prefill.rs:81-85)."""

    def __init__(self, gpu: Gpu, sources: list[Exl3Linear]):
        import math
        k = {s.size_k for s in sources}
        bits = {s.k_bits for s in sources}
        cbs = {s.codebook for s in sources}
        if len(k) != 1 or len(bits) != 1 or len(cbs) != 1:
            raise InputError("multi-linear: sources must share in-features, bit rate and codebook")
        self.sources = sources
        self.size_k, self.k_bits, self.codebook = k.pop(), bits.pop(), cbs.pop()
        width = 0
        for s in sources:
            width = math.gcd(width, s.size_n)
        if width % 128:
            raise InputError("multi-linear: slice width must be a multiple of 128")
        self.width = width
        b, svh, stride, src, n0s = [], [], [], [], []
        tile_bytes = 16 * self.k_bits * 2
        for si, s in enumerate(sources):
            for n0 in range(0, s.size_n, width):
                b.append(s.trellis.data_ptr() + (n0 // 16) * tile_bytes)
                svh.append(s.svh.data_ptr() + n0 * 2)
                stride.append(s.size_n)
                src.append(si)
                n0s.append(n0)
        self.slices = len(b)
        self._src, self._n0 = src, n0s
        i64 = lambda v: torch.tensor(v, dtype=torch.int64, device=gpu.device)
        i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=gpu.device)
        self.b_list, self.svh_list = i64(b), i64(svh)
        self.suh_list = i64([s.suh.data_ptr() for s in sources])
        self.size_n_list, self.n_stride_list, self.had_src_list = i32([width] * len(b)), i32(stride), i32(src)
        self.a_had = torch.zeros(len(sources) * self.size_k, dtype=torch.float16, device=gpu.device)
        self._c_key, self._c_ptrs = None, None
        # the same lists on the host: one-row launches pass them by value (berth_ops_mgemm_hostlists)
        self._h = {"b": np.array(b, dtype=np.uint64), "svh": np.array(svh, dtype=np.uint64),
                   "suh": np.array([s.suh.data_ptr() for s in sources], dtype=np.uint64),
                   "size_n": np.array([width] * len(b), dtype=np.int32), "stride": np.array(stride, dtype=np.int32),
                   "src": np.array(src, dtype=np.int32)}
        self._h_c = None
        self.host_lists = self.slices <= 16

    def forward(self, gpu: Gpu, a: torch.Tensor, outs: list[torch.Tensor], out: OutDtype, rows: int = 1,
                by_value: bool = True) -> None:
        """a fp16 [rows][K]; outs[i] [rows][N_i] of `out` for source i.  `by_value` False
        keeps the lists in device memory whatever the row count."""
        if rows < 1:
            raise InputError("multi-linear: rows must be positive")
        if rows * self.size_k > self.a_had.numel() // len(self.sources):
            self.a_had = torch.zeros(len(self.sources) * rows * self.size_k, dtype=torch.float16, device=gpu.device)
        esz = 4 if out == OutDtype.F32 else 2
        key = tuple(o.data_ptr() for o in outs) + (esz,)
        if key != self._c_key:
            ptrs = [outs[s].data_ptr() + n0 * esz for s, n0 in zip(self._src, self._n0)]
            self._c_ptrs = torch.tensor(ptrs, dtype=torch.int64, device=gpu.device)
            self._h_c = np.array(ptrs, dtype=np.uint64)
            self._c_key = key
        # lists by value: one row through the streaming kernel, more than 8 rows through the MFMA
        # kernels (2..8 rows read the device lists)
        if by_value and ((rows == 1 and self.host_lists) or (rows > 8 and self.slices <= 16)):
            h = self._h
            try:
                K.ops.exl3_mgemm_hostlists(ptr(a), h["b"].ctypes.data, ptr(outs[0]), h["suh"].ctypes.data, ptr(self.a_had),
                                           h["svh"].ctypes.data, rows, self.size_k, self.width, self.k_bits, self.codebook,
                                           out, 1, self.slices, h["size_n"].ctypes.data, self._h_c.ctypes.data,
                                           h["stride"].ctypes.data, h["src"].ctypes.data, len(self.sources),
                                           gpu.raw_stream())
                return
            except K.LaunchError as err:
                if rows > 1 or "host lists" not in str(err):
                    raise
                self.host_lists = False         # too small for the streaming kernel: device lists from now on
        K.ops.exl3_mgemm(ptr(a), ptr(self.b_list), ptr(outs[0]), ptr(self.suh_list), ptr(self.a_had),
                         ptr(self.svh_list), rows, self.size_k, self.width, self.k_bits, self.codebook, out,
                         1, self.slices, ptr(self.size_n_list), ptr(self._c_ptrs), ptr(self.n_stride_list),
                         ptr(self.had_src_list), len(self.sources), gpu.raw_stream())


class MlpLayer:
    """gate -> up -> silu_mul -> down (mlp.rs:118-150 decode, :219-303 prefill)."""

    def __init__(self, gpu: Gpu, gate: Exl3Linear, up: Exl3Linear, down: Exl3Linear, max_rows: int = 1):
        self.gate, self.up, self.down = gate, up, down
        self.hidden = gate.size_k
        self.intermediate = gate.size_n
        if up.size_k != self.hidden or up.size_n != self.intermediate or \
           down.size_k != self.intermediate or down.size_n != self.hidden:
            raise InputError("mlp: projection shapes do not chain")
        self.g = torch.zeros(max_rows * self.intermediate, dtype=torch.float16, device=gpu.device)
        self.u = torch.zeros(max_rows * self.intermediate, dtype=torch.float16, device=gpu.device)
        self.x_had = self.act_had = None      # rotated inputs of the fused call, allocated on first use
        # the one-call path takes one bit rate and codebook for the three linears
        self.uniform = gate.k_bits == up.k_bits == down.k_bits and gate.codebook == up.codebook == down.codebook
        self.has_bias = any(l.bias is not None for l in (gate, up, down))

    @classmethod
    def load(cls, gpu: Gpu, ckpt, layer: int, max_rows: int = 1) -> "MlpLayer":
        """Layer `layer`'s MLP weights (mlp.rs:52-56)."""
        return cls.load_prefixed(gpu, ckpt, f"model.language_model.layers.{layer}.mlp", max_rows)

    @classmethod
    def load_prefixed(cls, gpu: Gpu, ckpt, prefix: str, max_rows: int = 1) -> "MlpLayer":
        """`{prefix}.gate_proj`, `.up_proj`, `.down_proj` (mlp.rs:58-112).  The reference refuses
        a bias here (mlp.rs:67-75); this loader keeps it, and `forward` then takes the four-call
        path, where each linear adds its own."""
        parts = [f"{prefix}.gate_proj", f"{prefix}.up_proj", f"{prefix}.down_proj"]
        gate, up, down = (Exl3Linear.load(gpu, ckpt, part) for part in parts)
        if (gate.size_k, gate.size_n) != (up.size_k, up.size_n):
            raise WeightsError(f"{prefix}: gate is {gate.size_k}x{gate.size_n}, up is {up.size_k}x{up.size_n}")
        if (down.size_k, down.size_n) != (gate.size_n, gate.size_k):
            raise WeightsError(f"{prefix}: down is {down.size_k}x{down.size_n}, gate is {gate.size_k}x{gate.size_n}")
        if gate.size_n < 2 or gate.size_n % 2:
            raise WeightsError(f"{prefix}: intermediate {gate.size_n} must be positive and even")
        return cls(gpu, gate, up, down, max_rows)

    def forward(self, gpu: Gpu, x: torch.Tensor, y: torch.Tensor, fused: bool = True, rows: int = 1) -> None:
        """x fp16 [rows][hidden] -> y fp32 [rows][hidden].  fused: one `berth_exl3_mlp` call (two
        launches up to 8 rows); otherwise the reference's four calls for one row (mlp.rs:118-150)."""
        if fused and self.uniform and not self.has_bias:
            if rows * self.intermediate > self.g.numel() or x.numel() < rows * self.hidden or \
               y.numel() < rows * self.hidden:
                raise InputError(f"{self.gate.prefix}: buffer too small")
            if self.x_had is None or self.x_had.numel() < rows * self.hidden:
                self.x_had = torch.zeros(rows * self.hidden, dtype=torch.float16, device=x.device)
                self.act_had = torch.zeros(self.g.numel(), dtype=torch.float16, device=x.device)
            lins = [(ptr(l.trellis), ptr(l.suh), ptr(l.svh)) for l in (self.gate, self.up, self.down)]
            K.exl3_mlp(ptr(x), lins, ptr(self.g), ptr(self.u), ptr(self.x_had), ptr(self.act_had), ptr(y), rows,
                       self.hidden, self.intermediate, self.gate.k_bits, self.gate.codebook, gpu.raw_stream())
            return
        self.gate.forward(gpu, x, self.g, OutDtype.F16)
        self.up.forward(gpu, x, self.u, OutDtype.F16)
        K.ops.silu_mul(ptr(self.g), ptr(self.u), ptr(self.u), self.intermediate, 0.0, gpu.raw_stream())
        self.down.forward(gpu, self.u, y, OutDtype.F32)

    def forward_block(self, gpu: Gpu, x: torch.Tensor, residual: torch.Tensor, residual_out: torch.Tensor,
                      norm_weight: torch.Tensor, y: torch.Tensor, epsilon: float = 1e-6, constant_bias: float = 1.0,
                      constant_scale: float = 1.0, weight_bf16: bool = True, rows: int = 1) -> None:
        """The FFN block around the MLP in one call (`berth_exl3_mlp_block`): residual_out =
        residual + x; y = mlp(rms_norm(residual_out)) + residual_out.  x, residual, residual_out
        and y fp32 [rows][hidden]."""
        if not self.uniform or self.has_bias:
            raise InputError(f"{self.gate.prefix}: the block call takes one bit rate and codebook and no bias")
        if rows * self.intermediate > self.g.numel():
            raise InputError(f"{self.gate.prefix}: buffer too small")
        if self.x_had is None or self.x_had.numel() < rows * self.hidden:
            self.x_had = torch.zeros(rows * self.hidden, dtype=torch.float16, device=x.device)
            self.act_had = torch.zeros(self.g.numel(), dtype=torch.float16, device=x.device)
        if getattr(self, "h_norm", None) is None or self.h_norm.numel() < rows * self.hidden:
            self.h_norm = torch.zeros(rows * self.hidden, dtype=torch.float16, device=x.device)
        norm = K.RmsNorm(ptr(norm_weight), epsilon, constant_bias, constant_scale, int(weight_bf16))
        lins = [(ptr(l.trellis), ptr(l.suh), ptr(l.svh)) for l in (self.gate, self.up, self.down)]
        K.exl3_mlp_block(ptr(x), ptr(residual), ptr(residual_out), norm, lins, ptr(self.h_norm), ptr(self.g), ptr(self.u),
                         ptr(self.x_had), ptr(self.act_had), ptr(y), rows, self.hidden, self.intermediate,
                         self.gate.k_bits, self.gate.codebook, gpu.raw_stream())

    def prefill(self, gpu: Gpu, scratch: RowScratch, x: torch.Tensor, y: torch.Tensor, rows: int) -> None:
        """x fp16 [rows][hidden] -> y fp32 [rows][hidden]."""
        if rows * self.intermediate > self.g.numel():
            raise InputError("mlp: rows exceed the layer scratch")
        self.gate.forward_rows(gpu, scratch, x, self.g, rows, OutDtype.F16)
        self.up.forward_rows(gpu, scratch, x, self.u, rows, OutDtype.F16)
        K.ops.silu_mul(ptr(self.g), ptr(self.u), ptr(self.u), rows * self.intermediate, 0.0, gpu.raw_stream())
        self.down.forward_rows(gpu, scratch, self.u, y, rows, OutDtype.F32)
