"""CPU oracle for the Vision-RWKV WKV operators.  TEST INFRASTRUCTURE ONLY.

Nothing in this directory is part of the shipped operator path: it is imported
by the test-suite, by the smoke check and by the CPU-baseline leg of the
benchmark, always as the checker and never as the thing being measured or
shipped.  The HIP operators never call into it and never fall back to it.

Contents
--------
biwkv.py       Bi-WKV forward in float64: O(T^2) closed form, two-pass
               stabilised recurrence, and gradients by autograd through the
               closed form.
wkv6.py        bidirectional RWKV-6 scan in float64: sequential recurrence,
               O(T^2) cumulative-log-decay closed form, autograd gradients.
qshift.py      q_shift / q_shift_multihead as explicit index loops.
blocks.py      the element-wise block steps around the operators (row epilogues,
               VRWKV6 token mixes, GroupNorm x gate), row by row in float64.
chunk_carry.py float64 model of the reference kernel's 32-way token split (what a
               literal CUDA run would return; tests/test_reference_chunk_carry.py).
torch_eager.py the same recurrences as PyTorch CPU-eager fp32 loops over T
               (what the benchmark times as its CPU baseline).
c/             plain-C restatement of the recurrences (double accumulators),
               used for full-size parity where NumPy would take minutes.

Pinning status (what each function is checked against, see tests/test_oracle_*):
  biwkv_closed / biwkv_scan : mutual agreement (independent restatements),
      softmax reduction (w=u=0), T=1, u->inf, w->inf 3-term mean, constant-v,
      convexity, k-shift invariance, reversal symmetry, channel independence.
  wkv6_scan / wkv6_closed   : mutual agreement, d==1 linear-attention einsum,
      d==0 three-token form, T=1, head independence, reversal symmetry.
  q_shift loops             : zero-border / pass-through invariants, a
      tensor-slicing restatement with channel-group bounds stated by hand
      (equal quarters and the unequal groups of C % 4 != 0).
  blocks                    : hand-computed rows, torch LayerNorm / GroupNorm
      in float64, step-order checks.
  C backward routines       : autograd through the closed forms, finite
      differences and the sum identities (tests/test_oracle_c.py).
The reference ships no golden vectors or tests for these operators, so the
fixtures under tests/golden/ are produced from the float64 closed forms here.
"""
