"""CPU restatement of the reference algorithms on the per-layer training
compute path.

THIS PACKAGE IS TEST INFRASTRUCTURE.  It is the checker the HIP kernels are
compared against; nothing in ``flextrain_amd`` imports it, and only ``tests/``,
``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` may.
Every function runs on the CPU in fp32 (or exact integers) with plain PyTorch /
NumPy and cites the reference file:line it restates.

How each function is pinned (tests/test_oracle_*.py, all CPU-only):

  rmsnorm      fwd: closed form on constant rows, scale invariance, per-head ==
               reshaped full-row, the reference-held ``_rmsnorm`` formula
               (flextrain/bench/parity.py:112-115) written independently in the
               test through torch.nn.functional.rms_norm; bwd: torch.autograd of
               that forward, and the identity sum_d dx*x = dot*eps/(var+eps).
  rope         ``_rope_pair_interleave`` (flextrain/bench/parity.py:118-139);
               complex multiplication by exp(i*angle) (torch.polar), norm of
               every pair preserved, pos = 0 identity, bwd o fwd = identity.
  glu          torch.nn.functional.silu / gelu(approximate="tanh") and
               torch.autograd of those (tests/test_gelu_tanh_gated_kernel.py:57-89);
               silu_bwd: torch.autograd of F.silu; embedding_bwd: torch.autograd
               through F.embedding and a per-token Python loop on a tiny case.
  adamw        torch.optim.AdamW run for several steps
               (flextrain/bench/parity.py:546-577) and the step-1 closed form.
  linear_ce    torch.softmax / argmax, F.cross_entropy (none / sum, ignore_index),
               torch.autograd through rms_norm -> matmul -> cross-entropy.
  moe          stable sort / bincount / indexing identities, torch.autograd through
               the eager expert formula (tests/moe/test_moe_backend_parity.py:45-107).
  ffn_dense    torch.autograd through the textbook gated-FFN formula in fp32 (both
               activations), weight gradients accumulated onto given tensors.
  attention_proj  torch.autograd through an independent fp32 formulation of the attention
               block (projections with biases, F.rms_norm per head, RoPE as complex
               multiplication, dense causal grouped-query attention as the core, output
               projection plus residual): each half is fed autograd's own tensors at the
               core's boundary and must return autograd's gradients.
  dp_solver    golden vectors from the compiled reference solver (oracle/_ref, built
               by oracle/Makefile from the reference's own C file), the README known
               answer, exhaustive enumeration of all option vectors on small problems.
"""
