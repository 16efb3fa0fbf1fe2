"""CPU oracle for the fused fp8 LM-head + tanh-softcap + cross-entropy path.

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package imports this
directory; only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg
may, and only as the checker.

Contents
--------
eager.py        the reference's eager head restated with stock torch ops
                (quantise -> fp32 matmul -> cap*tanh(u/cap) -> F.cross_entropy ->
                autograd), row-chunked so N x V never has to exist at once.
closed_form.py  numpy float64 forward/backward written from the explicit
                formulas (no autograd), for small shapes.
fp8.py          numpy tables for OCP e4m3fn / e5m2 decode and RNE encode.

How each function is pinned (see tests/test_oracle_*.py)
--------------------------------------------------------
fp8.encode_e4m3 / decode_e4m3   against torch's Tensor.to(float8_e4m3fn) on
                                all 256 codes, every midpoint between adjacent
                                codes, the 448/464/465 overflow edge, subnormals.
eager.quantize_e4m3             is the library cast itself; checked against fp8.py.
eager.softcapped_ce             against closed_form (independent derivation),
                                cap -> inf limit == F.cross_entropy on raw
                                logits, W = 0 => loss == ln V, chunked == unchunked,
                                row-permutation equivariance, fp8 bytes invariant
                                under a joint power-of-two rescale of X and x_s.
closed_form.backward            central finite differences of closed_form.forward
                                in float64, sum_v dz == 0, ignored rows => zero
                                dX row, autograd (torch float64) on the same inputs.
eager.softcapped_ce_mtp         n_predict=1 == plain path bit for bit;
                                weights [1,0,0] == [1]; against closed_form MTP.
eager.rms_norm                  bit-identical to F.rms_norm (fp32 and bf16 input,
                                default and explicit eps).
eager.rms_norm_backward         against torch's autograd through F.rms_norm in
                                float64.
eager.norm_softcapped_ce        is the composition of the two above with
                                softcapped_ce.

The reference holds no golden vectors, tests or fixtures for this path, and its
fused CUDA kernel cannot be imported on this toolchain, so the reference's own
numerics (bf16-rounded tanh, e5m2 dlogits, fast-math exp) are "parity unpinned";
the contract is the eager path named above.
"""
