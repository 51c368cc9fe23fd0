"""CPU oracle for the LeanFFN hot path.  TEST INFRASTRUCTURE ONLY.

A from-scratch restatement, in stock PyTorch / numpy on the CPU, of what the reference's LeanFFN path computes
(lean_transformer/ffn.py, lean_transformer/blocksparse/{linear,native_backend,layout}.py, lean_transformer/utils.py).
It exists to check the HIP kernels and to be timed as the CPU baseline.  Nothing in the product package
``lean_transformer_amd`` imports it; only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg do.

Pin status of each function (what, other than re-reading the formula, fixes its result):

  gelu_fused / gelu_fused_grad      |F.gelu| bound 5e-4 (reference tests/test_utils.py:25-29); grad vs autograd of the closed form
  plain_ffn                         composition of library routines (F.layer_norm, F.linear, dropout-by-mask); op order and
                                    GeGLU half order are the ones reference tests/test_ffn.py:121-147 restates
  LeanFFNFunction (manual backward) equals autograd of plain_ffn (what reference tests/test_ffn.py:58-86,212-241 assert of the
                                    reference) + torch.autograd.gradcheck in fp64
  butterfly_mask / pixelfly_layout  golden layouts written by the reference (tests/golden/blocksparse_golden.npz) + densities
  / hypercube_layout                of reference tests/test_layout.py:10-13 + brute-force butterfly factor products
  indices_from_layout               golden forward/backward indices from the reference; invariant of tests/test_butterfly.py:33
  blocksparse_matmul (+ backward)   golden y / dx / dw from the reference on seeded inputs; backward == autograd of forward
                                    (reference tests/test_butterfly.py:141-142); brute-force triple loop on tiny shapes
  full LeanGPT step                 parity unpinned by fixture (reference tests/gpt_test_data.pth is absent from the checkout);
                                    not part of this oracle
"""
