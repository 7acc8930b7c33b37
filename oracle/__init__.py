"""CPU restatement of the Pi0 / Pi05 single-observation forward pass.

TEST INFRASTRUCTURE ONLY.  This package is the checker for the HIP path: it may be
imported by tests/, by __graft_entry__.smoke() and by the cpu_baseline leg of bench.py,
never by the product package.  It is plain PyTorch CPU eager: bf16-valued weights and
activations, fp32 arithmetic inside every dot product, reduction and transcendental,
and a round-to-bf16 at each place the reference writes a bf16 buffer.

Parity status: the reference ships no golden vectors, known-answer tests or fixtures
for this path (its test.py only prints a comparison against a JAX policy that needs
network-hosted assets).  Each function below is therefore pinned by tests/test_oracle_*.py
against an independent statement of the same mathematics (torch.nn.functional routines,
brute-force loops on small sizes, closed forms and invariants), not against reference
outputs.  What cannot be pinned at all - the reference's bit-level rounding inside its
bf16 LayerNorm and softmax kernels and inside torch.compile'd attention - is
"parity unpinned" at the bit level; the tolerance model (action MAE <= 1e-2,
per-layer relative L2 <= 2e-2) is what the GPU parity tests assert.
"""
