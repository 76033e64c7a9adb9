"""CPU oracle for the FP8 hot path. TEST INFRASTRUCTURE ONLY.

Plain PyTorch-on-CPU / numpy restatements of the reference's arithmetic, one
function per reference kernel, each citing the reference file:line it follows.
Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import
this package, and only as the checker. The product (viola_amd) never imports
it and has no CPU fallback.

Pinning status (what fixes each function besides its own formula):
  fp8 casts        : independent bit-level encoder (oracle.fp8) vs torch's CPU cast, all
                     256 codes round-trip, tie and saturation cases        -> pinned
  grouped quantize : closed form + invariants (group max maps to +-limit, exact
                     round trip of representable inputs)                     -> pinned
  grouped GEMM     : textbook fp64 matmul of the dequantized operands        -> pinned
  Philox4x32-10    : Random123 known-answer vectors held by the reference
                     (checks/quantization.py:77-81)                          -> pinned
  stochastic round : adjacency + probability properties (checks/quantization.py:114-153)
  momentum/weight/adam/comm codec : closed forms held by the reference's checks
  Newton-Schulz    : golden vectors written by tests/golden/make_ns_golden.py from the
                     reference's own optim/_orthogonalize.py + invariants   -> pinned
  per-tensor scaling (oracle.tensor) : the reference's own CPU definitions (checks/linear.py:17-20,
                     viola/nn/linear.py:298-312) + textbook matmul           -> pinned; an Inf inside the
                     tensor (infinite scale, Inf / Inf)                       -> parity unpinned
  Hadamard-64 rotation (oracle.rotation) : the matrix the reference defines it by (rotate_cpu,
                     _rotation_kernels.py:126-130): exact on integers, one-hot rows, involution  -> pinned
  MLP composition (oracle.linear.mlp) : float autograd of down(act(gate x) * up x) + an exact recomposition
                     from linear / gated_forward / gated_backward called by hand           -> pinned
  variable-group (MoE) linear : NOT in the reference (no fixture or check of its own there); brute force over
                     groups of sizes 0, 1, 37, 3, 0 through the Linear restatement         -> pinned by that only
  FP16-accumulator model (grouped.gemm_half, tensor.gemm_half) : hand cases that fix where the roundings
                     fall (2048 + 1 -> 2048 across steps, exact within a step, cleared per period). Where an
                     NVIDIA mma rounds inside a 32-k step is not in the reference's text   -> the model's own
                     arithmetic is pinned, its agreement with the reference's hardware is parity unpinned
  NaN/Inf inside a quantize group: the reference's GPU and CPU branches disagree
                     (GPU reduce_absmax ignores NaN); the GPU behaviour is restated
                                                                   -> parity unpinned
"""
