"""CPU oracle for the FP8 skinny-GEMM / residual-RMSNorm / SwiGLU path.

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package imports this directory: it is the checker that
`tests/`, `__graft_entry__.smoke()` and the `cpu_baseline` leg of `bench.py` compare the HIP kernels against.
It restates, on the CPU, what the reference computes for this path (the torch functions its own tests use),
with FP8 taken as OCP e4m3fn -- the format gfx950 implements -- instead of the e4m3fnuz the reference was
written for.

Modules (each function cites the reference lines it follows):
  fp8.py          e4m3fn decode table, round-to-nearest-even encoder, `fp8_quantize`
  skinny_gemm.py  `reference_skinny_gemm` (dequantise -> fp32 matmul -> scale -> 16-bit) and the exact variant
  residual_rms.py `reference_residual_rms`, `precise_residual_rms`
  swiglu.py       `reference_swiglu`
  llama_mlp.py    the four-op chain
  weight_format.py packed tile layout (pack / unpack / element offset) and e4m3fnuz -> e4m3fn re-encoding
  c/hfrk_oracle.c plain-C restatement (integer-exact GEMM, scalar RMSNorm/SwiGLU) used to pin the above

How each function is pinned (see tests/test_oracle_*.py):
  fp8 decode      closed form over all 256 codes == torch's uint8->float8_e4m3fn->float view (library routine)
  fp8 encode      own RNE encoder == torch's cast on a dense sweep incl. every midpoint; idempotence,
                  monotonicity, saturation, odd symmetry
  skinny GEMM     exact int64 dot products in C == fp64 matmul == pure-Python integers on tiny shapes; closed
                  forms (zero, scaled identity, one-hot, powers of two); fp32 path within 1 bf16 ulp of exact
  residual RMS    16-bit add == numpy IEEE add; fp32 path vs fp64 textbook formula; C scalar restatement
  SwiGLU          x*sigmoid(x) closed form == torch.nn.functional.silu; special values; C restatement
  weight format   fnuz decode table == torch's float8_e4m3fnuz view for all 256 codes and == fn/2 on the same
                  bits; re-encode table == torch's fnuz -> float -> fn casts for all 256 codes; layout: reshape
                  implementation == element-offset formula written from the MFMA operand definition, round trip
  llama MLP       composition of the pinned parts; the reference holds no test or fixture for the chain, so
                  the composition itself (which buffer feeds which op) is "parity unpinned" beyond that
"""
