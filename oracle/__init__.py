"""CPU oracle for the KV-cache compression path — TEST INFRASTRUCTURE, not product code.

Each function restates, on the CPU with torch/numpy, what the reference computes at the
file:line it cites (paths relative to the reference root).  Only the tests, the smoke check
and the CPU-baseline leg of the benchmark may import this package; nothing under
``fastcache_amd`` does.

Pinning status (what independent check fixes each restatement; see tests/test_oracle_*.py):
  paged.extract_kv / write_back      closed form dense[s] = pool[table[s // bs], s % bs], brute force
  presses.knorm_score                float64 brute force of -sqrt(sum k^2)
  presses.topk_lowest_index          pure-Python sorted() on rows with injected exact ties
  presses.gather_tokens              integer-patterned payloads, brute-force loops
  presses.adapter_compress_layer     index arithmetic by hand for streaming_llm / uniform stride
  presses.snapkv_score               float64 loops on tiny shapes for the composition
                                     matmul -> softmax -> slice -> reduce -> avg_pool1d -> group reduce;
                                     the residual choices made by the third-party kvpress package
                                     (causal mask inside the window, mean vs sum, window inside the
                                     budget) cannot be checked offline: PARITY UNPINNED for those
  ccm.*                              float64 loops for Linear/ReLU chain, reshape by hand
  autocompress.linear_act / mlp_nobias   float64 loops with the rounding points made explicit
  autocompress.quantize / dequantize      numpy float16 arithmetic step by step, hand-worked rows
  presses.expected_attention_*        float64 loops over tokens / keys for the statistics and the score, closed
                                     forms (zero covariance, identity rotation); the kvpress package itself is
                                     unavailable offline: PARITY UNPINNED beyond the published formula
  presses.think_* / simlayer_*        loops over heads, tokens, queries with the causal rule written out, hand-worked
                                     rows; kvpress itself is unavailable offline: PARITY UNPINNED beyond the
                                     published description of ThinK and SimLayerKV
  presses.fake_quantize               numpy float16 arithmetic step by step, hand-worked rows, idempotence
  autocompress.quantize_fp8 / quantize_int8_asymmetric
                                      the float8 cast against a brute-force nearest-code search (ties, both formats),
                                      hand-worked rows, numpy float16 arithmetic step by step
  blocks.*                           invariants of the free deque / ref counts, hand-worked cases
  attention.decode_attention         float64 loops; flash-attn itself is unavailable offline:
                                     PARITY UNPINNED beyond the mathematical definition
"""
