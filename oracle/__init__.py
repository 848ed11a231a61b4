"""CPU oracle for the KV-cache decode path.

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package (``ohara_amd``) imports
this directory.  The only callers are ``tests/``, ``__graft_entry__.smoke()`` and the
``cpu_baseline`` leg of ``bench.py`` - and there only as the checker / the reported
host baseline, never as the thing measured or shipped.

Every function restates, in plain PyTorch on the CPU (integer parts in numpy/torch
integer arithmetic), the algorithm of the reference file:line it cites.  The
restatement is functional (a flat ``dict`` of tensors keyed by the reference's
state-dict names) rather than an ``nn.Module`` tree.

Pinning status (what independently fixes each function; see tests/test_oracle.py):

  rms_norm            closed form, unit-RMS invariant, fp64 brute force
  rope_table          closed form cos/sin(t * theta^(-2i/D)) in fp64
  apply_rope          complex multiply (torch.view_as_complex), norm preservation,
                      identity at position 0
  KVCacheRef          copy semantics + the reference's error substrings
  attention           fp64 brute-force loops on tiny inputs; cached == uncached
                      (the uncached path reduces to F.scaled_dot_product_attention
                      with is_causal=True, a library routine)
  attention in bf16   (_attention_reduced, fexp_u20) the library's bf16 routine on six shapes
                      and a V = identity probe of the exponential (tests/test_oracle_bf16.py);
                      the reference's per-module operands of a mid-size GQA model
                      (tests/golden/llama_bf16_mid_gqa.pt)
  swiglu / linear     F.silu / matmul library routines
  llama_forward       composition: golden fixtures tests/golden/llama_tiny_*.pt (fp32) and
                      tests/golden/llama_bf16_*.pt (the reference model cast to bfloat16:
                      tiny models bit-identical; d12 widths and d12 itself within the
                      distance between the reference's own runs, which the fixtures hold)
  moe_route/dispatch  per-token hand loop, k distinct experts, weights sum to 1,
                      golden fixture tests/golden/llama_tiny_moe.pt
  sample_*            the reference tests' known answers; exhaustive small-V
                      restatement in fp64; inverse-CDF identities
  bitlinear_*         torch.int32 matmul (library routine), closed forms
                      (W = c*T reproduces T, equal activations -> +-127)
  generate loops      the reference tests' literal outputs ("1 2 3 5 5 5",
                      call lengths [3,1,1], positions [0,3,4])

  Phi (phi_ref.py)    rope_partial: the reference RoPE module's vectors (tests/golden/phi_rope.pt)
                      + fp64 closed form; new_gelu / layer_norm / linear_bias: library routines;
                      attention: fp64 brute force; phi_forward as a composition is PARITY
                      UNPINNED by golden logits (ohara/models/phi.py is not importable here: it
                      needs the absent `lightning` package) - held by the reference test's
                      cached == uncached invariant and an fp64 hand-written block
                      (tests/test_oracle_phi.py)

bf16 GEMM accumulation order is "parity unpinned": the library's own kernels differ
from each other in it (each bf16 fixture holds the reference run with all threads, with
one thread and with the library's other matrix kernels); the oracle defines a Linear as
an fp32-accumulated product of the dtype-rounded operands, rounded once to the model
dtype, which reproduces >= 99.98 % of the reference's per-operator outputs bit for bit.
"""
