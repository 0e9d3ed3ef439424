"""Linear layers (reference: tinyvllm/layers/linear.py:10-184).

Same class names, weight layout (``[out, in]``, ``nn.Linear`` order) and ``weight_loader``
protocol as the reference; this build runs one GPU, so the tensor-parallel rank is 0 of 1 and
there is no all-reduce.  ``quantize_()`` swaps the bf16 weight for an int8 weight plus a
per-output-channel fp32 scale; ``forward`` then runs the weight-only int8 GEMM.  On the GPU the int8
weight is kept in the library's tile order (``ops.pack_w8``, done once by ``pack_()``): ``qweight``
is the row-major ``[out, in]`` tensor until then, ``qpacked`` the packed one afterwards.
"""
import torch
from torch import nn

from .. import ops


def quantize_per_channel(weight: torch.Tensor):
    """Symmetric int8: ``scale[n] = max|W[n,:]| / 127``, ``Wq = clamp(round(W / scale), -127, 127)``."""
    w = weight.float()
    amax = w.abs().amax(dim=1)
    scale = torch.where(amax > 0, amax / 127.0, torch.ones_like(amax))
    wq = torch.round(w / scale[:, None]).clamp_(-127, 127).to(torch.int8)
    return wq.contiguous(), scale.contiguous()


class LinearBase(nn.Module):
    def __init__(self, input_size: int, output_size: int, tp_dim: int | None = None):
        super().__init__()
        self.input_size = input_size
        self.output_size = output_size
        self.tp_dim = tp_dim
        self.tp_rank = 0
        self.tp_size = 1
        self.qweight = None        # int8 [out, in] row-major (None again once packed)
        self.qpacked = None        # ops.PackedW8: the same weight in the GEMM kernels' tile order
        self.qscale = None

    def _make_params(self, out_features: int, in_features: int, bias: bool):
        self.weight = nn.Parameter(torch.empty(out_features, in_features))
        self.weight.weight_loader = self.weight_loader
        if bias:
            self.bias = nn.Parameter(torch.empty(out_features))
            self.bias.weight_loader = self.weight_loader
        else:
            self.register_parameter("bias", None)

    def quantize_(self):
        """Replace the bf16 weight by int8 + scale (frees the bf16 copy).  Nothing to do for a layer
        whose int8 weight came from a quantised checkpoint."""
        if self.is_quantized:
            return self
        self.qweight, self.qscale = quantize_per_channel(self.weight.data)
        self.weight.data = torch.empty(0, dtype=self.weight.dtype, device=self.weight.device)
        return self

    @property
    def is_quantized(self) -> bool:
        return self.qweight is not None or self.qpacked is not None

    def pack_(self):
        """Row-major int8 weight -> tile order, on the GPU, once; the row-major copy is dropped."""
        if self.qpacked is None and self.qweight is not None:
            self.qpacked = ops.pack_w8(self.qweight)
            self.qweight = None
        return self

    def load_quantized(self, qweight: torch.Tensor, qscale: torch.Tensor):
        self.qweight, self.qscale = qweight.contiguous(), qscale.contiguous()
        self.weight.data = torch.empty(0, dtype=self.weight.dtype, device=qweight.device)

    def shard_rows(self, shard_id=None):
        """(first output row, row count) of a checkpoint tensor inside this layer's weight."""
        return 0, self.weight.shape[0] if self.weight.numel() else self.qweight.shape[0]

    def load_quantized_shard(self, kind: str, tensor: torch.Tensor, shard_id=None):
        """One ``.qweight`` (int8 ``[rows, in]``) or ``.qscale`` (fp32 ``[rows]``) tensor of a quantised
        checkpoint into rows ``shard_rows(shard_id)``.  Per-output-channel scales make the rows of a packed
        projection independent, so q/k/v (gate/up) are quantised one by one offline and packed here."""
        if self.qweight is None:
            out_f, in_f = self.weight.shape
            dev = self.weight.device
            self.qweight = torch.zeros(out_f, in_f, dtype=torch.int8, device=dev)
            self.qscale = torch.ones(out_f, dtype=torch.float32, device=dev)
            self.weight.data = torch.empty(0, dtype=self.weight.dtype, device=dev)
            self.pending_quantized = True
        first, rows = self.shard_rows(shard_id)
        dst = self.qweight if kind == "qweight" else self.qscale
        assert tensor.shape[0] == rows and tensor.dtype == dst.dtype, (kind, tensor.shape, tensor.dtype)
        dst[first:first + rows].copy_(tensor)

    def finish_quantized_load(self):
        """Called once after every shard is in."""
        self.pending_quantized = False

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        if self.is_quantized:
            y = ops.w8a16_linear(x, self.pack_().qpacked, self.qscale)
        else:
            y = ops.bf16_linear(x, self.weight.data)
        if self.bias is not None:
            y = y + self.bias
        return y


class ReplicatedLinear(LinearBase):
    def __init__(self, input_size: int, output_size: int, bias: bool = False):
        super().__init__(input_size, output_size)
        self._make_params(output_size, input_size, bias)

    def weight_loader(self, param: nn.Parameter, loaded_weight: torch.Tensor):
        param.data.copy_(loaded_weight)


class ColumnParallelLinear(LinearBase):
    def __init__(self, input_size: int, output_size: int, bias: bool = False):
        super().__init__(input_size, output_size, 0)
        self.input_size_per_partition = input_size
        self.output_size_per_partition = output_size // self.tp_size
        self._make_params(self.output_size_per_partition, input_size, bias)

    def weight_loader(self, param: nn.Parameter, loaded_weight: torch.Tensor):
        n = param.data.size(self.tp_dim)
        param.data.copy_(loaded_weight.narrow(self.tp_dim, self.tp_rank * n, n))


class MergedColumnParallelLinear(ColumnParallelLinear):
    """Several projections stacked along the output dim (gate_up_proj)."""

    def __init__(self, input_size: int, output_sizes: list[int], bias: bool = False):
        self.output_sizes = output_sizes
        super().__init__(input_size, sum(output_sizes), bias=bias)

    def quantize_(self):
        """int8 + scale; a gate/up pair is also re-ordered for the fused projection + SiLU-and-mul
        kernel (``ops.gate_up_interleave_index``), which ``forward_silu_mul`` then uses."""
        if not self.is_quantized:
            super().quantize_()
            self.interleave_()
        return self

    def interleave_(self):
        """Rows into the order the fused projection + SiLU-and-mul kernels read (int8 weight and scale, or the bf16
        weight): once, after loading."""
        if not getattr(self, "interleaved", False) and len(self.output_sizes) == 2 \
                and self.output_sizes[0] == self.output_sizes[1] \
                and sum(self.output_sizes) % 16 == 0 and self.bias is None:
            if self.is_quantized:
                if self.qweight is None:
                    return                   # already packed without the interleave: leave it alone
                idx = ops.gate_up_interleave_index(sum(self.output_sizes), self.qweight.device)
                self.qweight = self.qweight[idx].contiguous()
                self.qscale = self.qscale[idx].contiguous()
            else:
                idx = ops.gate_up_interleave_index(sum(self.output_sizes), self.weight.device)
                self.weight.data = self.weight.data[idx].contiguous()
            self.interleaved = True

    def natural_weight(self) -> torch.Tensor:
        """The bf16 weight in checkpoint order ([gate; up]) whatever order it is held in."""
        w = self.weight.data
        if getattr(self, "interleaved", False) and w.numel():
            idx = ops.gate_up_interleave_index(sum(self.output_sizes), w.device)
            inv = torch.empty_like(idx)
            inv[idx] = torch.arange(idx.numel(), device=idx.device)
            w = w[inv]
        return w

    def shard_rows(self, shard_id=None):
        return sum(self.output_sizes[:shard_id]) // self.tp_size, self.output_sizes[shard_id] // self.tp_size

    def finish_quantized_load(self):
        super().finish_quantized_load()
        self.interleave_()

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        if getattr(self, "interleaved", False):
            raise RuntimeError("this gate_up weight is interleaved for the fused kernel: call forward_silu_mul")
        return super().forward(x)

    def forward_silu_mul(self, x: torch.Tensor) -> torch.Tensor:
        """``SiluAndMul()(self(x))`` (activation.py:11-14 after linear.py:82-83), one kernel once the rows are interleaved."""
        if getattr(self, "interleaved", False):
            if self.is_quantized:
                return ops.w8a16_linear_silu_mul(x, self.pack_().qpacked, self.qscale)
            return ops.bf16_linear_silu_mul(x, self.weight)
        return ops.silu_and_mul(super().forward(x))

    def weight_loader(self, param: nn.Parameter, loaded_weight: torch.Tensor, loaded_shard_id: int):
        if getattr(self, "interleaved", False):
            raise RuntimeError("this gate_up weight was re-ordered for the fused kernel: load weights before pack_linears_()")
        offset = sum(self.output_sizes[:loaded_shard_id]) // self.tp_size
        size = self.output_sizes[loaded_shard_id] // self.tp_size
        dst = param.data.narrow(self.tp_dim, offset, size)
        dst.copy_(loaded_weight.chunk(self.tp_size, self.tp_dim)[self.tp_rank])


class QKVParallelLinear(ColumnParallelLinear):
    """q, k and v projections stacked as [q | k | v] along the output dim."""

    def __init__(self, hidden_size: int, head_size: int, total_num_heads: int,
                 total_num_kv_heads: int | None = None, bias: bool = False):
        self.head_size = head_size
        self.total_num_heads = total_num_heads
        self.total_num_kv_heads = total_num_kv_heads or total_num_heads
        self.num_heads = self.total_num_heads
        self.num_kv_heads = self.total_num_kv_heads
        super().__init__(hidden_size, (self.num_heads + 2 * self.num_kv_heads) * head_size, bias)

    def forward_qknorm_rope_store(self, x: torch.Tensor, q_norm, k_norm, positions, cos_sin, k_cache, v_cache,
                                  slot_mapping, k_scale, v_scale, want_kv: bool):
        """``ops.qknorm_rope_store(self(x), ...)`` (models/qwen3.py:78-94 + layers/attention.py:94-95) behind
        one call; ``q_norm`` / ``k_norm`` are the RMSNorm modules.  Returns ``(q, k, v)``."""
        tail = (q_norm.weight.data, k_norm.weight.data, q_norm.eps, positions, cos_sin, self.num_heads,
                self.num_kv_heads, self.head_size, k_cache, v_cache, slot_mapping, k_scale, v_scale)
        if self.bias is not None:
            return ops.qknorm_rope_store(self.forward(x), *tail, want_kv=want_kv)
        if self.is_quantized:
            return ops.linear_qknorm_rope_store(x, self.pack_().qpacked, self.qscale, *tail, want_kv=want_kv)
        return ops.linear_qknorm_rope_store(x, self.weight.data, None, *tail, want_kv=want_kv)

    def shard_rows(self, shard_id=None):
        assert shard_id in ("q", "k", "v")
        q_size, kv_size = self.num_heads * self.head_size, self.num_kv_heads * self.head_size
        return {"q": (0, q_size), "k": (q_size, kv_size), "v": (q_size + kv_size, kv_size)}[shard_id]

    def weight_loader(self, param: nn.Parameter, loaded_weight: torch.Tensor, loaded_shard_id: str):
        offset, size = self.shard_rows(loaded_shard_id)
        dst = param.data.narrow(self.tp_dim, offset, size)
        dst.copy_(loaded_weight.chunk(self.tp_size, self.tp_dim)[self.tp_rank])


class RowParallelLinear(LinearBase):
    def __init__(self, input_size: int, output_size: int, bias: bool = False):
        super().__init__(input_size, output_size, 1)
        self.input_size_per_partition = input_size // self.tp_size
        self._make_params(output_size, self.input_size_per_partition, bias)

    def forward_add_rmsnorm(self, x: torch.Tensor, residual: torch.Tensor, norm):
        """``norm(self(x), residual)`` (layernorm.py:33-45 after linear.py:181-183) behind one call;
        ``norm`` is the ``RMSNorm`` module that follows this projection.  Returns ``(normed, residual)``."""
        if self.bias is not None:
            return norm(self.forward(x), residual)
        if self.is_quantized:
            return ops.linear_add_rms_norm(x, self.pack_().qpacked, self.qscale, residual, norm.weight.data, norm.eps)
        return ops.linear_add_rms_norm(x, self.weight.data, None, residual, norm.weight.data, norm.eps)

    def weight_loader(self, param: nn.Parameter, loaded_weight: torch.Tensor):
        n = param.data.size(self.tp_dim)
        param.data.copy_(loaded_weight.narrow(self.tp_dim, self.tp_rank * n, n))
