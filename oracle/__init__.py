"""CPU restatement of the reference's per-token hot path.

THIS PACKAGE IS TEST INFRASTRUCTURE, NOT PRODUCT CODE.  Only ``tests/``,
``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` may
import it, and only as the checker.  Nothing under ``tinyllmforge_amd/`` imports
it: the product path fails loudly when its HIP library is missing and has no
CPU fallback.

Every function restates, in eager PyTorch on the CPU (fp32 math with the
reference's bf16 rounding points) or in numpy for the pure integer / byte work,
what the reference's layer does, and cites the reference file:line it follows.
The reference has no tests, golden vectors or fixtures of its own, so each
function is pinned in ``tests/test_oracle_*.py`` against closed forms,
invariants, library routines and brute force on tiny inputs.

Parity status of each function (a function with no independent pin would say
"parity unpinned" here):

* ``store_kvcache``            pinned: python-loop brute force + permutation invariants
* ``rms_norm``/``add_rms_norm`` pinned: closed form in fp64, unit-RMS invariant, residual=0 reduction
* ``rope_table``/``rope``       pinned: pos=0 identity, norm preservation, composition of rotations, fp64 closed form
* ``silu_and_mul``             pinned: ``F.silu`` library routine, fp64 closed form
* ``greedy_sample``            pinned: ``torch.argmax``, tie vectors
* ``linear``                   pinned: fp64 matmul
* ``w8a16_linear``             build-defined semantics (the reference has no int8 path); pinned: exact integer arithmetic on integer-valued activations, fp64 matmul
* ``paged_decode_attention``   pinned: ``F.scaled_dot_product_attention``, ctx=1 returns the V row, pool-permutation invariance, brute-force loops
* ``varlen_prefill_attention`` pinned: ``F.scaled_dot_product_attention`` with causal / bottom-right masks, paged == dense after gather
* ``fp8`` KV-cache variants    build-defined semantics (the reference has no fp8 cache); pinned: e4m3 round trip of representable values, saturation, scale linearity
* flash-attn's internal P->bf16 rounding and inductor's fused roundings are
  not restated (they need the CUDA stack): the oracle follows the eager text;
  the attention tolerance (2e-2 max-abs) absorbs the former.
"""
