"""CPU oracle: a plain-PyTorch restatement of the reference's arithmetic for the training-step
kernels (attention, fp8 fused MLP, RMSNorm / residual blocks, loss head, AdamW, the 12-layer
model that strings them together).

THIS PACKAGE IS TEST INFRASTRUCTURE. Only tests/, __graft_entry__.smoke() and bench.py's
cpu_baseline leg may import it, and only as the checker / the timed CPU baseline. Nothing under
trainium_frontier_them_bones_amd/ imports it and the HIP path never routes through it.

Every function cites the reference lines it restates (paths relative to the reference repo:
R1 = round1/source/train.py, R2 = round2/source/train.py, K/ = round2/source/kernels/).
The reference ships no golden vectors or test files for this path, so each function is pinned
against a PyTorch library routine, a closed form, an invariant or a brute-force loop in
tests/test_oracle_*.py; the header of each module says what pins it.
"""
