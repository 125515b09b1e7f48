"""CPU oracle for the compress / decompress hot path — TEST INFRASTRUCTURE ONLY.

A restatement, in plain torch-CPU / numpy op chains (and a small C file for the
scalar arithmetic), of what the reference computes on this path, one op per
line in the reference's order so that dtype promotion and rounding happen
where the reference has them.  Every function cites the reference file:line it
follows (paths relative to src/compressed_tensors/ of neuralmagic/compressed-tensors).

Nothing in the product imports this package.  Its only users are tests/,
__graft_entry__.smoke() and the cpu_baseline leg of bench.py, and there it is
the checker / the timed CPU baseline, never the thing shipped.

How each part is pinned (see tests/test_oracle_*.py):
  pack_to_int32 / unpack_from_int32   reference known answers (tests/golden/pack_int32.json)
  quantize / dequantize / qparams     reference QDQ matrices (tests/golden/static_lifecycle.json),
                                      C restatement of the scalar chain, closed forms
  fp8 e4m3 cast                       C restatement over all 65 536 bf16 inputs + fp32 sweeps
  fp4 cast / pack                     reference sign-of-zero vector, 16-entry code table
  bitmasks                            numpy.packbits itself; round trips; brute force
  2:4 masks                           torch.topk itself (the reference calls it); C restatement
  Hadamard                            reference seed-42 sign vector; H Hᵀ = nI; textbook FWHT
"""
