"""The package under the reference's import name (``tinyvllm``), on the CPU.

The reference's scripts do ``from tinyvllm import LLM, SamplingParams`` (bench.py:31, example.py:2,
tinyvllm/__init__.py:1-2) and its model / runner reach the layers as ``tinyvllm.layers.*`` and
``tinyvllm.utils.context``.  After ``tinyllmforge_amd.dropin.install()`` each of those imports must resolve to
this package's module OBJECTS (not to second copies of the files), and every class a caller of the hot path
constructs or calls must take the reference's parameter names in the reference's order.  The table below is
transcribed from the reference's ``def`` lines (file:line beside each row); parameters this build adds must
come after them and have defaults, so that a call written against the reference binds the same way.
"""
import importlib
import inspect

import pytest

MODULES = [
    "layers.attention", "layers.layernorm", "layers.rotary_embedding", "layers.activation", "layers.linear",
    "layers.sampler", "layers.embed_head", "utils.context", "utils.loader", "engine.scheduler",
    "engine.block_manager", "engine.sequence", "engine.model_runner", "engine.llm_engine", "models.qwen3",
    "config", "sampling_params", "llm",
]

# (module, object, method or None for a function, the reference's parameters after self)
SIGNATURES = [
    ("layers.attention", "Attention", "__init__", ["num_heads", "head_dim", "scale", "num_kv_heads"]),       # attention.py:73-79
    ("layers.attention", "Attention", "forward", ["q", "k", "v"]),                                             # attention.py:86
    ("layers.attention", "store_kvcache", None, ["key", "value", "k_cache", "v_cache", "slot_mapping"]),      # attention.py:33-39
    ("layers.layernorm", "RMSNorm", "__init__", ["hidden_size", "eps"]),                                       # layernorm.py:10-14
    ("layers.layernorm", "RMSNorm", "forward", ["x", "residual"]),                                             # layernorm.py:47-50
    ("layers.rotary_embedding", "RotaryEmbedding", "__init__",
     ["head_size", "rotary_dim", "max_position_embedding", "base"]),                                           # rotary_embedding.py:21-27
    ("layers.rotary_embedding", "RotaryEmbedding", "forward", ["positions", "query", "key"]),                  # rotary_embedding.py:42-46
    ("layers.rotary_embedding", "get_rope", None,
     ["head_size", "rotary_dim", "max_position", "base", "rope_scaling"]),                                     # rotary_embedding.py:61-67
    ("layers.activation", "SiluAndMul", "forward", ["x"]),                                                     # activation.py:12
    ("layers.linear", "ReplicatedLinear", "__init__", ["input_size", "output_size", "bias"]),                  # linear.py:29-34
    ("layers.linear", "ColumnParallelLinear", "__init__", ["input_size", "output_size", "bias"]),              # linear.py:54-59
    ("layers.linear", "MergedColumnParallelLinear", "__init__", ["input_size", "output_sizes", "bias"]),       # linear.py:87-91
    ("layers.linear", "QKVParallelLinear", "__init__",
     ["hidden_size", "head_size", "total_num_heads", "total_num_kv_heads", "bias"]),                           # linear.py:114-121
    ("layers.linear", "RowParallelLinear", "__init__", ["input_size", "output_size", "bias"]),                 # linear.py:155-159
    ("layers.linear", "RowParallelLinear", "forward", ["x"]),                                                  # linear.py:180
    ("layers.sampler", "Sampler", "forward", ["logits", "temperatures"]),                                      # sampler.py:8-12
    ("layers.embed_head", "VocabParallelEmbedding", "__init__", ["num_embeddings", "embedding_dim"]),          # embed_head.py:10
    ("layers.embed_head", "VocabParallelEmbedding", "forward", ["x"]),                                         # embed_head.py:34
    ("layers.embed_head", "ParallelLMHead", "forward", ["x"]),                                                 # embed_head.py:58
    ("utils.context", "set_context", None,
     ["is_prefill", "cu_seqlens_q", "cu_seqlens_k", "max_seqlen_q", "max_seqlen_k", "slot_mapping",
      "context_lens", "block_tables"]),                                                                        # context.py:21
    ("utils.context", "get_context", None, []),                                                                # context.py:18
    ("utils.context", "reset_context", None, []),                                                              # context.py:25
    ("engine.scheduler", "Scheduler", "__init__", ["config"]),                                                 # scheduler.py:9
    ("engine.scheduler", "Scheduler", "add", ["seq"]),                                                         # scheduler.py:19
    ("engine.scheduler", "Scheduler", "schedule", []),                                                         # scheduler.py:22
    ("engine.scheduler", "Scheduler", "preempt", ["seq"]),                                                     # scheduler.py:59
    ("engine.scheduler", "Scheduler", "postprocess", ["seqs", "token_ids"]),                                   # scheduler.py:64
    ("engine.block_manager", "BlockManager", "__init__", ["num_blocks", "block_size"]),                        # block_manager.py:26
    ("engine.block_manager", "BlockManager", "can_allocate", ["seq"]),                                         # block_manager.py:62
    ("engine.block_manager", "BlockManager", "allocate", ["seq"]),                                             # block_manager.py:66
    ("engine.block_manager", "BlockManager", "deallocate", ["seq"]),                                           # block_manager.py:100
    ("engine.block_manager", "BlockManager", "can_append", ["seq"]),                                           # block_manager.py:110
    ("engine.block_manager", "BlockManager", "may_append", ["seq"]),                                           # block_manager.py:117
    ("engine.sequence", "Sequence", "__init__", ["token_ids", "sampling_params"]),                             # sequence.py:15
    ("engine.sequence", "Sequence", "append_token", ["token_id"]),                                             # sequence.py:68
    ("engine.sequence", "Sequence", "block", ["i"]),                                                           # sequence.py:64
    ("engine.model_runner", "ModelRunner", "__init__", ["config", "rank", "event"]),                           # model_runner.py:17
    ("engine.model_runner", "ModelRunner", "prepare_block_tables", ["seqs"]),                                  # model_runner.py:155
    ("engine.model_runner", "ModelRunner", "prepare_prefill", ["seqs"]),                                       # model_runner.py:164
    ("engine.model_runner", "ModelRunner", "prepare_decode", ["seqs"]),                                        # model_runner.py:210
    ("engine.model_runner", "ModelRunner", "prepare_sample", ["seqs"]),                                        # model_runner.py:231
    ("engine.model_runner", "ModelRunner", "run_model", ["input_ids", "positions", "is_prefill"]),             # model_runner.py:244
    ("engine.model_runner", "ModelRunner", "run", ["seqs", "is_prefill"]),                                     # model_runner.py:264
    ("engine.model_runner", "ModelRunner", "call", ["method_name"]),                                           # model_runner.py:101
    ("engine.llm_engine", "LLMEngine", "__init__", ["model"]),                                                 # llm_engine.py:17
    ("engine.llm_engine", "LLMEngine", "add_request", ["prompt", "sampling_params"]),                          # llm_engine.py:43
    ("engine.llm_engine", "LLMEngine", "generate", ["prompts", "sampling_params", "use_tqdm"]),                # llm_engine.py:64-68
    ("models.qwen3", "Qwen3ForCausalLM", "forward", ["input_ids", "positions"]),                               # qwen3.py:221-225
    ("models.qwen3", "Qwen3ForCausalLM", "compute_logits", ["hidden_states"]),                                 # qwen3.py:229
    ("sampling_params", "SamplingParams", "__init__", ["temperature", "max_tokens", "ignore_eos"]),            # sampling_params.py:5-11
]

# the reference's Config fields (config.py:7-17), which LLM(model, **kwargs) accepts by name (llm_engine.py:18-20)
CONFIG_FIELDS = ["model", "max_num_batched_tokens", "max_num_seqs", "max_model_len", "gpu_memory_utilization",
                 "tensor_parallel_size", "enforce_eager", "hf_config", "eos", "kvcache_block_size", "num_kvcache_blocks"]
CONFIG_DEFAULTS = dict(max_num_batched_tokens=16384, max_num_seqs=512, max_model_len=4096, gpu_memory_utilization=0.9,
                       tensor_parallel_size=1, enforce_eager=False, eos=-1, kvcache_block_size=256, num_kvcache_blocks=-1)
# the Context fields (context.py:7-14)
CONTEXT_FIELDS = ["is_prefill", "cu_seqlens_q", "cu_seqlens_k", "max_seqlen_q", "max_seqlen_k", "slot_mapping",
                  "context_lens", "block_tables"]


@pytest.fixture()
def tinyvllm():
    from tinyllmforge_amd import dropin
    dropin.install()
    yield importlib.import_module("tinyvllm")
    dropin.uninstall()


def test_the_reference_import_lines_resolve_to_this_package(tinyvllm):
    import tinyllmforge_amd
    assert tinyvllm is tinyllmforge_amd
    from tinyvllm import LLM, SamplingParams                 # bench.py:31, example.py:2
    assert LLM is tinyllmforge_amd.LLM and SamplingParams is tinyllmforge_amd.SamplingParams
    for name in MODULES:
        alias = importlib.import_module("tinyvllm." + name)
        real = importlib.import_module("tinyllmforge_amd." + name)
        assert alias is real, name                            # one module object, one set of globals
    # the statements the reference's own files use to reach the seam (qwen3.py:5-11, model_runner.py:8-13)
    from tinyvllm.layers.attention import Attention           # noqa: F401
    from tinyvllm.layers.layernorm import RMSNorm             # noqa: F401
    from tinyvllm.layers.rotary_embedding import get_rope     # noqa: F401
    from tinyvllm.layers.activation import SiluAndMul         # noqa: F401
    from tinyvllm.layers.linear import QKVParallelLinear, MergedColumnParallelLinear, RowParallelLinear  # noqa: F401
    from tinyvllm.layers.embed_head import VocabParallelEmbedding, ParallelLMHead                        # noqa: F401
    from tinyvllm.layers.sampler import Sampler               # noqa: F401
    from tinyvllm.utils.context import set_context, get_context, reset_context
    from tinyvllm.utils.loader import load_model              # noqa: F401
    from tinyvllm.engine.sequence import Sequence, SequenceStatus                                        # noqa: F401
    from tinyvllm.engine.block_manager import BlockManager    # noqa: F401
    from tinyvllm.engine.scheduler import Scheduler           # noqa: F401
    from tinyvllm.engine.model_runner import ModelRunner      # noqa: F401
    from tinyvllm.models.qwen3 import Qwen3ForCausalLM        # noqa: F401
    # one Context for both names: what the runner publishes under one name the layers read under the other
    from tinyllmforge_amd.utils.context import get_context as real_get
    set_context(False, context_lens="lens")
    assert real_get().context_lens == "lens" and get_context() is real_get()
    reset_context()
    assert real_get().context_lens is None
    with pytest.raises(ModuleNotFoundError):
        importlib.import_module("tinyvllm.no_such_module")


@pytest.mark.parametrize("module,obj,method,want", SIGNATURES, ids=[f"{m}.{o}.{f or ''}" for m, o, f, _ in SIGNATURES])
def test_parameter_names_are_the_references(tinyvllm, module, obj, method, want):
    target = getattr(importlib.import_module("tinyvllm." + module), obj)
    if method is not None:
        target = getattr(target, method)
    params = [p for p in inspect.signature(target).parameters.values() if p.name != "self"]
    named = [p for p in params if p.kind in (p.POSITIONAL_ONLY, p.POSITIONAL_OR_KEYWORD)]
    got = [p.name for p in named[:len(want)]]
    assert got == want, f"{module}.{obj}.{method}: {got} != {want}"
    for extra in named[len(want):]:                            # what this build adds must be optional
        assert extra.default is not inspect.Parameter.empty, extra.name


def test_config_context_and_sampling_params_fields(tinyvllm):
    from dataclasses import fields
    from tinyvllm.config import Config
    from tinyvllm.sampling_params import SamplingParams
    from tinyvllm.utils.context import Context
    names = [f.name for f in fields(Config)]
    assert names[:len(CONFIG_FIELDS)] == CONFIG_FIELDS
    defaults = {f.name: f.default for f in fields(Config)}
    for k, v in CONFIG_DEFAULTS.items():
        assert defaults[k] == v, k
    assert [f.name for f in fields(SamplingParams)] == ["temperature", "max_tokens", "ignore_eos"]
    sp = SamplingParams()
    assert (sp.temperature, sp.max_tokens, sp.ignore_eos) == (1.0, 64, False)      # sampling_params.py:5-7
    ctx = Context()
    assert [n for n in CONTEXT_FIELDS if hasattr(ctx, n)] == CONTEXT_FIELDS
    assert ctx.is_prefill is False and ctx.max_seqlen_q == 0 and ctx.block_tables is None


def test_attention_module_state_the_runner_binds(tinyvllm):
    """model_runner.py:135-139 finds the attention modules by their ``k_cache`` / ``v_cache`` attributes and
    attention.py:94 tests ``numel()`` on them: both exist, empty, on a fresh module."""
    from tinyvllm.layers.attention import Attention
    a = Attention(16, 128, 128 ** -0.5, 8)
    assert hasattr(a, "k_cache") and hasattr(a, "v_cache")
    assert a.k_cache.numel() == 0 and a.v_cache.numel() == 0
    assert (a.num_heads, a.head_dim, a.num_kv_heads) == (16, 128, 8)


def test_packed_modules_mapping_is_the_references(tinyvllm):
    from tinyvllm.models.qwen3 import Qwen3ForCausalLM
    assert Qwen3ForCausalLM.packed_modules_mapping == {             # qwen3.py:200-206
        "q_proj": ("qkv_proj", "q"), "k_proj": ("qkv_proj", "k"), "v_proj": ("qkv_proj", "v"),
        "gate_proj": ("gate_up_proj", 0), "up_proj": ("gate_up_proj", 1)}
