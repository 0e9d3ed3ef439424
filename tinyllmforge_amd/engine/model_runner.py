"""Host -> GPU boundary of one engine step (reference: tinyvllm/engine/model_runner.py:15-308).

One process, one GPU: no process group, no shared-memory RPC.  Per step the runner builds the
integer inputs on the host (``engine/inputs.py``), stages them in one pinned buffer, copies them
to the device and runs the model either eagerly (prefill) or by replaying a captured hipGraph
(decode; ``torch.cuda.CUDAGraph`` is the hipGraph wrapper on ROCm).  Graph padding rows carry
slot -1 and context length 0, so they neither write the KV cache nor read it.
"""
from __future__ import annotations

import numpy as np
import torch

from .. import _lib, ops
from ..config import Config
from ..layers.sampler import Sampler
from ..models.qwen3 import Qwen3ForCausalLM
from ..utils.context import get_context, reset_context, set_context
from ..utils.loader import load_model, random_init_
from . import inputs as I
from .sequence import Sequence


class ModelRunner:
    def __init__(self, config: Config, rank: int = 0, event=None, state_dict: dict | None = None):
        assert rank == 0
        if not torch.cuda.is_available():
            raise RuntimeError("ModelRunner needs a GPU: the HIP hot path has no CPU fallback")
        self.config = config
        hf = config.hf_config
        self.block_size = config.kvcache_block_size
        Sequence.block_size = self.block_size
        self.enforce_eager = config.enforce_eager
        self.device = torch.device("cuda", torch.cuda.current_device())
        self.kv_dtype = torch.bfloat16 if config.kv_cache_dtype == "bf16" else torch.float8_e4m3fn

        default_dtype = torch.get_default_dtype()
        torch.set_default_dtype(hf.torch_dtype)
        try:
            with torch.device(self.device):
                self.model = Qwen3ForCausalLM(hf)
            # the RoPE table is built on the host (same bits as a CPU restatement), then moved
            self.model.to(self.device)
            if state_dict is not None:
                from ..utils.loader import load_state_dict
                load_state_dict(self.model, state_dict)
            elif isinstance(config.model, str) and __import__("os").path.isdir(config.model):
                load_model(self.model, config.model)
            else:
                big = hf.hidden_size >= 2048
                random_init_(self.model, seed=config.seed, device_fill=big)
            if config.quantization == "w8a16":
                self.model.quantize_linears_()
            self.model.pack_linears_()        # int8 weights (quantised here or loaded) into tile order
        finally:
            torch.set_default_dtype(default_dtype)
        self.model.eval()
        self.sampler = Sampler(seed=config.seed)
        self.fused_greedy = True      # all-greedy batches: LM head and argmax in one call
        self.graphs = {}
        self.graph_bs = []
        self._stage = None            # pinned staging buffer of the eager steps' integer inputs (grow-only)
        with torch.inference_mode():
            self.warmup_model()
            self.allocate_kv_cache()
            if not self.enforce_eager:
                self.capture_graphs()

    def exit(self):
        """Release the graphs, the KV pool and the weights (whoever still holds this object holds no memory)."""
        torch.cuda.synchronize()
        self.graphs.clear()
        self.graph_vars = self.graph_ring = self.graph_pack_dev = None
        if getattr(self, "model", None) is not None:
            for module in self.model.modules():
                if hasattr(module, "k_cache") and hasattr(module, "v_cache"):
                    module.k_cache = module.v_cache = torch.tensor([])
        self.kv_cache = None
        self.model = None
        import gc
        gc.collect()
        torch.cuda.empty_cache()

    def call(self, method_name, *args):
        return getattr(self, method_name)(*args)

    # ------------------------------------------------------------------ set-up
    def warmup_model(self):
        """One worst-case prefill before the cache exists, to learn the activation peak
        (model_runner.py:108-116); it also allocates the kernels' workspaces."""
        torch.cuda.empty_cache()
        torch.cuda.reset_peak_memory_stats()
        cfg = self.config
        num_seqs = max(1, min(cfg.max_num_batched_tokens // cfg.max_model_len, cfg.max_num_seqs))
        seqs = [Sequence([0] * cfg.max_model_len) for _ in range(num_seqs)]
        self.run(seqs, True)
        torch.cuda.empty_cache()

    def kv_block_bytes(self) -> int:
        hf = self.config.hf_config
        itemsize = 2 if self.kv_dtype == torch.bfloat16 else 1
        return 2 * hf.num_hidden_layers * self.block_size * hf.num_key_value_heads * hf.head_dim * itemsize

    def allocate_kv_cache(self):
        """One tensor ``[2, L, nblk, block, Hkv, Dh]``; layer l gets views ``kv[0, l]`` / ``kv[1, l]``
        (model_runner.py:118-139).  ``num_kvcache_blocks`` may be fixed in the config."""
        cfg, hf = self.config, self.config.hf_config
        if cfg.num_kvcache_blocks <= 0:
            free, total = torch.cuda.mem_get_info()
            used = total - free
            stats = torch.cuda.memory_stats()
            peak, current = stats["allocated_bytes.all.peak"], stats["allocated_bytes.all.current"]
            cfg.num_kvcache_blocks = int(total * cfg.gpu_memory_utilization - used - (peak - current)) // self.kv_block_bytes()
        assert cfg.num_kvcache_blocks > 0
        self.kv_cache = torch.zeros(2, hf.num_hidden_layers, cfg.num_kvcache_blocks, self.block_size,
                                    hf.num_key_value_heads, hf.head_dim, dtype=self.kv_dtype, device=self.device)
        layer_id = 0
        for module in self.model.modules():
            if hasattr(module, "k_cache") and hasattr(module, "v_cache"):
                module.k_cache = self.kv_cache[0, layer_id]
                module.v_cache = self.kv_cache[1, layer_id]
                if self.kv_dtype != torch.bfloat16:
                    # build-defined static per-head scales of the e4m3 cache (Config.kv_k_scale / kv_v_scale):
                    # |x| above 448 * scale saturates
                    module.k_scale = self._kv_scale(cfg.kv_k_scale, layer_id)
                    module.v_scale = self._kv_scale(cfg.kv_v_scale, layer_id)
                layer_id += 1

    @torch.inference_mode()
    def kv_saturation(self, block_ids=None) -> dict:
        """How many entries of an e4m3 KV cache sit at the format's largest magnitude (|code| = 0x7e, i.e.
        +-448 x scale): the store clamps there, so a scale too small for a layer's keys or values shows up as
        saturated entries, not as an error.  Counted over ``block_ids`` (default: every block; unwritten rows
        are zeros and count as entries).  Returns totals and the worst (layer, KV head) for K and for V; a bf16
        cache has nothing to saturate and returns zeros."""
        out = dict(entries=0, k_saturated=0, v_saturated=0, k_worst=None, v_worst=None)
        if self.kv_cache is None or self.kv_dtype == torch.bfloat16:
            return out
        kv = self.kv_cache.view(torch.uint8)                       # [2, L, nblk, block, Hkv, Dh]
        if block_ids is not None:
            kv = kv[:, :, torch.as_tensor(sorted(set(block_ids)), dtype=torch.long, device=kv.device)]
        out["entries"] = int(kv[0].numel())
        for which, name in ((0, "k"), (1, "v")):
            per = torch.zeros(kv.shape[1], kv.shape[4], dtype=torch.int64, device=kv.device)
            for layer in range(kv.shape[1]):                        # one layer at a time: the mask is a byte per entry
                per[layer] = ((kv[which, layer] & 0x7f) == 0x7e).sum(dim=(0, 1, 3))
            out[name + "_saturated"] = int(per.sum())
            if out[name + "_saturated"]:
                layer, head = divmod(int(per.argmax()), kv.shape[4])
                out[name + "_worst"] = dict(layer=layer, kv_head=head, saturated=int(per[layer, head]))
        return out

    def _kv_scale(self, spec, layer_id: int) -> torch.Tensor:
        """fp32 ``[Hkv]`` from a float (every head), ``[Hkv]`` values (every layer) or ``[L][Hkv]`` values."""
        hkv = self.config.hf_config.num_key_value_heads
        t = torch.as_tensor(spec, dtype=torch.float32)
        if t.dim() == 2:
            t = t[layer_id]
        t = t.expand(hkv).contiguous() if t.dim() == 0 else t.contiguous()
        assert t.shape == (hkv,) and bool((t > 0).all()), "KV scales: a positive float, [Hkv] or [L][Hkv]"
        return t.to(self.device)

    # ------------------------------------------------------------------ per-step inputs
    def _upload(self, arrays: dict) -> dict:
        """All integer inputs of a step go through ONE pinned staging buffer and ONE H2D copy."""
        names = [k for k, v in arrays.items() if isinstance(v, np.ndarray)]
        offs, total = {}, 0
        for k in names:
            total = (total + 15) // 16 * 16
            offs[k] = total
            total += arrays[k].nbytes
        total = max(total, 16)
        if self._stage is not None:
            # the copy out of the buffer must be over before it is rewritten (normally it is: every
            # step ends in the device -> host copy of its token ids)
            self._stage_copied.synchronize()
        if self._stage is None or self._stage.numel() < total:
            self._stage = torch.empty(max(total, 1 << 20), dtype=torch.uint8, pin_memory=True)
            self._stage_copied = torch.cuda.Event()
        stage = self._stage[:total]
        sv = stage.numpy()
        for k in names:
            sv[offs[k]:offs[k] + arrays[k].nbytes] = arrays[k].reshape(-1).view(np.uint8)
        dev = stage.to(self.device, non_blocking=True)
        self._stage_copied.record()
        out = dict(arrays)
        for k in names:
            a = arrays[k]
            dt = {np.dtype("int64"): torch.int64, np.dtype("int32"): torch.int32, np.dtype("float32"): torch.float32}[a.dtype]
            out[k] = dev[offs[k]:offs[k] + a.nbytes].view(dt).view(*a.shape)
        return out

    def prepare_block_tables(self, seqs):
        return torch.from_numpy(I.block_tables_array(seqs)).to(self.device)

    def _temperatures_of(self, seqs) -> np.ndarray | None:
        """fp32 temperatures of the step, or None for an all-greedy batch (the greedy kernel reads none)."""
        t = np.asarray([s.temperature for s in seqs], dtype=np.float32)
        self._all_greedy = bool((t == 0).all())
        return None if self._all_greedy else t

    def prepare_prefill(self, seqs):
        arrays = I.prefill_inputs(seqs, self.block_size)
        arrays["temperatures"] = self._temperatures_of(seqs)       # rides in the step's one staging copy
        d = self._upload(arrays)
        self._temperatures = d["temperatures"]
        set_context(True, d["cu_seqlens_q"], d["cu_seqlens_k"], d["max_seqlen_q"], d["max_seqlen_k"],
                    d["slot_mapping"], None, d["block_tables"])
        return d["input_ids"], d["positions"]

    def prepare_decode(self, seqs):
        arrays = I.decode_inputs(seqs, self.block_size, self.config.decode_position_quirk)
        arrays["temperatures"] = self._temperatures_of(seqs)
        d = self._upload(arrays)
        self._temperatures = d["temperatures"]
        set_context(False, slot_mapping=d["slot_mapping"], context_lens=d["context_lens"], block_tables=d["block_tables"])
        return d["input_ids"], d["positions"]

    def prepare_sample(self, seqs):
        """Temperatures of the step on the device (model_runner.py:230-236), None when all are 0: what the
        step's ``prepare_prefill`` / ``prepare_decode`` / graph upload already carried over."""
        return self._temperatures

    # ------------------------------------------------------------------ forward
    @torch.inference_mode()
    def run_hidden(self, input_ids, positions, is_prefill):
        """Final hidden states of the step's tokens (eager, or a graph replay with device-side inputs)."""
        bs = input_ids.size(0)
        ctx = get_context()
        if (is_prefill or self.enforce_eager or not self.graph_bs or bs > self.graph_bs[-1]
                or ctx.block_tables is None or ctx.block_tables.size(1) > self.graph_max_blocks):
            if not is_prefill:
                self.plan_decode()
            return self.model(input_ids, positions)      # a table wider than the graphs' static one runs eagerly
        gbs = next(x for x in self.graph_bs if x >= bs)
        gv = self.graph_vars
        if gbs != bs:      # padding rows: slot -1 (no cache write), length 0 (no cache read)
            gv["slot_mapping"][bs:gbs].fill_(-1)
            gv["context_lens"][bs:gbs].zero_()
            gv["input_ids"][bs:gbs].zero_()
            gv["positions"][bs:gbs].zero_()
        gv["input_ids"][:bs] = input_ids
        gv["positions"][:bs] = positions
        gv["slot_mapping"][:bs] = ctx.slot_mapping
        gv["context_lens"][:bs] = ctx.context_lens
        w = ctx.block_tables.size(1)
        gv["block_tables"][:bs, :w] = ctx.block_tables
        self.graphs[gbs].replay()
        return gv["outputs"][:bs]

    def plan_decode(self):
        """The attention kernel's work split of this decode step, made once for all layers (they share the
        lengths and the block tables) into one buffer that every step and every captured graph re-uses."""
        ctx = get_context()
        if (not self.config.decode_plan or ctx.context_lens is None or ctx.block_tables is None
                or ctx.context_lens.numel() > 1024):
            return      # switched off, or more sequences than a plan holds: every layer scans for itself
        ctx.decode_plan = self.decode_plan_buf = ops.paged_decode_plan(ctx.context_lens, ctx.block_tables, self.block_size,
                                                                       out=getattr(self, "decode_plan_buf", None))

    @torch.inference_mode()
    def run_model(self, input_ids, positions, is_prefill):
        return self.model.compute_logits(self.run_hidden(input_ids, positions, is_prefill))

    RING = 4   # pinned mirrors of the graphs' static inputs (two steps in flight + the one being filled + slack)

    def graph_ready(self, seqs) -> bool:
        """Whether a decode step over ``seqs`` fits the captured graphs (batch bucket, block-table width)."""
        return bool(not self.enforce_eager and self.graph_bs and len(seqs) <= self.graph_bs[-1]
                    and max(len(s.block_table) for s in seqs) <= self.graph_max_blocks)

    @torch.inference_mode()
    def launch_decode_graph(self, seqs, feed=None):
        """Decode step through a captured graph: the integer inputs (I.decode_inputs, the same function the
        eager path uploads) are written straight into a pinned mirror of the graph's static buffers,
        padding rows get slot -1 (no cache write) and length 0 (no cache read), one H2D copy, replay.
        ``feed = (token ids of the step before on the device, row of each of this step's sequences in that
        step)`` takes the input ids from there instead of from the host (whose sequences do not know them
        yet).  Returns the final hidden states (the graphs' static output buffer)."""
        bs = len(seqs)
        gbs = next(x for x in self.graph_bs if x >= bs)
        d = I.decode_inputs(seqs, self.block_size, self.config.decode_position_quirk)
        slot = self.graph_ring[self.graph_ring_at]
        self.graph_ring_at = (self.graph_ring_at + 1) % self.RING
        if slot["copied"] is not None:
            slot["copied"].synchronize()      # the copy out of this mirror, four steps ago, has long run
        h = slot["views"]
        h["input_ids"][:bs] = d["input_ids"]
        h["positions"][:bs] = d["positions"]
        h["slot_mapping"][:bs] = d["slot_mapping"]
        h["context_lens"][:bs] = d["context_lens"]
        w = d["block_tables"].shape[1]
        h["block_tables"][:bs, :w] = d["block_tables"]
        if feed is not None:
            h["feed_index"][:bs] = feed[1]
        if gbs != bs:
            h["input_ids"][bs:gbs] = 0
            h["positions"][bs:gbs] = 0
            h["slot_mapping"][bs:gbs] = -1
            h["context_lens"][bs:gbs] = 0
        t = self._temperatures_of(seqs)
        self._temperatures = None
        if t is not None:
            h["temperatures"][:bs] = t
            self._temperatures = self.graph_vars["temperatures"][:bs]
        self.graph_pack_dev.copy_(slot["pack"], non_blocking=True)
        if slot["copied"] is None:
            slot["copied"] = torch.cuda.Event()
        slot["copied"].record()
        if feed is not None:
            torch.index_select(feed[0], 0, self.graph_vars["feed_index"][:bs], out=self.graph_vars["input_ids"][:bs])
        set_context(False)
        self.graphs[gbs].replay()
        return self.graph_vars["outputs"][:bs], slot

    def run_decode_graph(self, seqs):
        return self.launch_decode_graph(seqs)[0]

    @torch.inference_mode()
    def run_ahead(self, seqs, feed=None):
        """One graph decode step whose token ids stay on the device: returns them with the pinned buffer their
        copy lands in and the event that says when.  Nothing here waits for the GPU."""
        hidden, slot = self.launch_decode_graph(seqs, feed)
        if self._all_greedy and self.fused_greedy:
            tokens = self.model.compute_greedy_ids(hidden)
        else:
            tokens = self.sampler(self.model.compute_logits(hidden), self._temperatures, self._all_greedy)
        reset_context()
        landing = slot["tokens"][:len(seqs)]
        landing.copy_(tokens, non_blocking=True)
        arrived = torch.cuda.Event()
        arrived.record()
        return tokens, landing, arrived

    @torch.inference_mode()
    def sample(self, hidden, temperatures):
        """Token ids from the final hidden states.  An all-greedy batch goes through the fused LM head +
        argmax (no logits in memory); otherwise logits, then the sampler.  The ``tolist`` is the step's one
        device sync."""
        if self._all_greedy and self.fused_greedy:
            return self.model.compute_greedy_ids(hidden).tolist()
        return self.sampler(self.model.compute_logits(hidden), temperatures, self._all_greedy).tolist()

    def run(self, seqs, is_prefill):
        use_graph = not is_prefill and self.graph_ready(seqs)
        if use_graph:
            hidden = self.run_decode_graph(seqs)
            token_ids = self.sample(hidden, self.prepare_sample(seqs))
            reset_context()
            return token_ids
        input_ids, positions = self.prepare_prefill(seqs) if is_prefill else self.prepare_decode(seqs)
        temperatures = self.prepare_sample(seqs)
        token_ids = self.sample(self.run_hidden(input_ids, positions, is_prefill), temperatures)
        reset_context()
        return token_ids

    # ------------------------------------------------------------------ hipGraph capture
    @torch.inference_mode()
    def capture_graphs(self):
        """Capture ``model(input_ids, positions)`` for batch buckets 1, 2, 4, 8, 16, 32, ... (model_runner.py:272-308).
        Every kernel of the hot path takes its geometry from the static shapes only, so a replay
        is valid for any lengths and block tables written into the static buffers."""
        cfg, hf = self.config, self.config.hf_config
        max_bs = min(cfg.max_num_seqs, 512)
        max_blocks = (cfg.max_model_len + self.block_size - 1) // self.block_size
        dev = self.device
        # The static integer inputs of the graphs live in ONE device allocation mirrored by ONE pinned
        # host buffer of the same layout: a decode step writes the host mirror in place (padding
        # rows included) and issues a single H2D copy - no per-step staging allocation, no
        # device-side copies or fills between the replays.
        layout, off = {}, 0
        for name, dt, shape in (("input_ids", torch.int64, (max_bs,)), ("positions", torch.int64, (max_bs,)),
                                ("feed_index", torch.int64, (max_bs,)),
                                ("slot_mapping", torch.int32, (max_bs,)), ("context_lens", torch.int32, (max_bs,)),
                                ("temperatures", torch.float32, (max_bs,)),
                                ("block_tables", torch.int32, (max_bs, max_blocks))):
            nbytes = int(np.prod(shape)) * torch.empty(0, dtype=dt).element_size()
            layout[name] = (off, nbytes, dt, shape)
            off += (nbytes + 15) // 16 * 16
        self.graph_pack_dev = torch.zeros(off, dtype=torch.uint8, device=dev)
        # A ring of pinned mirrors: a step that runs ahead fills the next mirror while the copy out of the
        # previous one may still be queued behind the graph before it; an event per mirror says when its
        # copy has run.  The token ids of a step come back through a ring of pinned buffers of their own.
        np_dt = {torch.int64: np.int64, torch.int32: np.int32, torch.float32: np.float32}
        self.graph_ring = []
        for _ in range(self.RING):
            pack = torch.zeros(off, dtype=torch.uint8, pin_memory=True)
            host_np = pack.numpy()
            views = {name: host_np[o:o + nbytes].view(np_dt[dt]).reshape(shape) for name, (o, nbytes, dt, shape) in layout.items()}
            views["slot_mapping"][:] = -1
            self.graph_ring.append(dict(pack=pack, views=views, copied=None,
                                        tokens=torch.zeros(max_bs, dtype=torch.int64, pin_memory=True)))
        self.graph_ring_at = 0
        gv = {}
        for name, (o, nbytes, dt, shape) in layout.items():
            gv[name] = self.graph_pack_dev[o:o + nbytes].view(dt).view(*shape)
        self.graph_pack_dev.copy_(self.graph_ring[0]["pack"])
        gv["outputs"] = torch.zeros(max_bs, hf.hidden_size, dtype=hf.torch_dtype, device=dev)
        self.graph_max_blocks = max_blocks
        self.graph_bs = [b for b in (1, 2, 4, 8) if b <= max_bs] + list(range(16, max_bs + 1, 16))
        pool = None
        lib = _lib.load()
        self.graph_kernels = {}      # batch bucket -> kernels in its graph
        for bs in reversed(self.graph_bs):
            graph = torch.cuda.CUDAGraph()
            set_context(False, slot_mapping=gv["slot_mapping"][:bs], context_lens=gv["context_lens"][:bs],
                        block_tables=gv["block_tables"][:bs, :])
            self.plan_decode()
            gv["outputs"][:bs] = self.model(gv["input_ids"][:bs], gv["positions"][:bs])    # warm-up
            launched = lib.tlf_kernel_launches()
            with torch.cuda.graph(graph, pool):
                self.plan_decode()       # first node of the graph: the attention work split of the step
                gv["outputs"][:bs] = self.model(gv["input_ids"][:bs], gv["positions"][:bs])
            self.graph_kernels[bs] = lib.tlf_kernel_launches() - launched + 1    # + the copy into the static output
            if pool is None:
                pool = graph.pool()
            self.graphs[bs] = graph
            torch.cuda.synchronize()
            reset_context()
        self.graph_vars = gv
