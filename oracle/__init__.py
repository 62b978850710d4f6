"""CPU oracle for the tree-mask packed-prefill attention path and the Gated DeltaNet scan.

TEST INFRASTRUCTURE ONLY.  Nothing under this directory is part of the shipped product: it may be imported by
``tests/``, by ``__graft_entry__.smoke()`` and by the ``cpu_baseline`` leg of ``bench.py`` as the checker, never
by the package itself.  Every function restates, in plain numpy, the algorithm of the reference file:line it
cites; the product's HIP kernels are compared against these results.

How each function is pinned (none relies on re-typing its own formula in a test):

  layout.pack_stream        the literal known answers of the reference's tests/test_packer.py:11-39,191-206, the
                            golden fixtures under tests/golden/ (written from the reference packer), the
                            "each read row sees exactly its prompt" invariant (tests/test_packer.py:209-239)
  mask.dense_tree_mask      brute force on tiny trees (ancestor walk along ``prev``), golden fixtures
  mask.block_classes        cover-the-dense-mask invariant and the two literal answers of
                            tests/test_packer.py:182-188,251-259
  attention.tree_attention  reductions to torch's own scaled_dot_product_attention (a trunk alone == causal;
                            B branches == B independent causal runs of trunk||branch; sliding == banded causal)
  gdn.recurrent             closed forms: g=0, beta=0 leaves the state unchanged; beta=1, g=0 is the plain delta
                            rule (after one token the state maps k_t to v_t exactly when |k_t|=1); linearity in v
  gdn.chunked               equals gdn.recurrent in float64 (two different algorithms for the same function)
  gdn.tree_scan             branch from the trunk's state == one sequence trunk||branch (docs/QWEN.md:51-52)
  gdn_layer.prologue/gate   torch's conv1d (one path = a depthwise causal convolution), silu, sigmoid, softplus, rms_norm
  lm_head.logprobs          torch.tanh / torch.log_softmax
  xdecode.x_attention       torch's scaled_dot_product_attention over the concatenated visible keys (the mask rebuilt key by
                            key in the test), and attention.tree_attention: a decoding step is the last row of causal
                            attention over prefix || own template || own generated tokens
  plan.tree_plan            the toy integer recurrence of the reference's tests/test_qwen_plan.py:27-94 and the
                            literal of tests/test_stacks.py:67-75

Third-party arithmetic that is absent from /root/reference (torch.nn.attention.flex_attention, pinned torch==2.14.0;
flash-linear-attention==0.5.2) has no golden vectors in the reference's tests: its published algorithm (masked softmax
attention; the gated delta rule) is restated here and pinned by the mathematical checks above.
"""
