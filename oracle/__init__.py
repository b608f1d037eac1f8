"""CPU oracle for the fused RoPE-attention hot path.

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package imports this
directory; it exists so that tests, the smoke entry and the benchmark's CPU
baseline leg can check the HIP kernels against an eager-PyTorch restatement
of the reference algorithm (fused-rope/rope_attn_pytorch.py and
corope-exp/corope_attn_gqa_pytorch.py of the reference repository).

Pin status of every function (what, other than its own formula, fixes it):

  precompute_freqs_cis   closed form in fp64, row-0 / unit-norm / duplicate-half invariants
  apply_rotary_emb       complex-number restatement, norm preservation, inverse round trip
  rope_attn_forward      torch SDPA (identity rotation and rotated inputs), fp64 brute-force
                         C program (oracle/brute_force.c), row-0 / convexity / logsumexp invariants
  rope_attn_backward     torch.autograd through the forward, gradcheck on fp64, delta identity
  corope_gqa_forward     fp64 brute-force C program, zero-leader reduction to RoPE attention,
                         G=1 bookkeeping, delta invariants
  corope_gqa_backward    torch.autograd through the forward (fp64)

No function here is "parity unpinned".
"""
