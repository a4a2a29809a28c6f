"""CPU oracle for the block-sparse attention forward.  TEST INFRASTRUCTURE ONLY.

Nothing in the product (the package directory, the C ABI, the Python module) imports,
links or executes anything from here; only tests/, __graft_entry__.smoke() and the
cpu_baseline leg of bench.py do, and only as the checker.

Two independent restatements of the reference's semantics:

  dense_oracle.py   fp32 dense attention + logsumexp over a dense bool mask, following
                    naive_attention_with_dense_mask (omni-attn-mma/omni_attn_torch.py:348-387)
                    with the kernels' empty-row convention (omni-attn-mma/mma/attn_naive.cu:177-183).
  block_walk.c      scalar C walk over the block metadata, following the reference's scalar
                    kernel omni_attn_simple_kernel_impl (omni-attn-mma/mma/attn_naive.cu:21-302).

How each is pinned (tests/test_oracle_pinning.py):
  * dense attention: library scaled_dot_product_attention, a brute-force triple loop on
    tiny inputs, closed forms (uniform scores -> mean of V; one allowed key -> that V row;
    logsumexp of equal scores = score + log n), torch.logsumexp.
  * block semantics (global-index CAUSAL, stored-bit PARTIAL, FULL): the block patterns
    and dense-mask sparsities the reference's generators printed
    (omni-attn-mma/logs/printed_mask.md:3-57, :59-76, :123-139, :153-176), held as data in
    tests/golden/printed_masks.json.
  * the two restatements against each other on random metadata.
  * gradients (dense_oracle.attention_dense_grads: autograd through the dense oracle, for the
    backward kernels, which have no counterpart in the reference): torch.autograd.gradcheck in
    fp64 on tiny inputs, the textbook closed form written without autograd, and the special
    case of one allowed key per row (dV = scatter of dO, dQ = dK = 0).
The reference's own golden tensors (*.pt) are absent from its tree, and its CUDA sources
cannot be compiled here (mma.sync / cp.async PTX), so there is no oracle/_ref build.
"""
