"""CPU oracle of crit's paged-KV hot path. TEST INFRASTRUCTURE ONLY.

This package restates, on the CPU, the arithmetic of the reference's KV append, paged attention and log-sum-exp merge
so that the HIP kernels can be checked against it. Nothing here is part of the product: only tests/, the smoke check
and the CPU-baseline leg of the benchmark may import it, and only as the checker (never as the thing measured against
the roofline, never as a fallback for a missing HIP library).

Modules and the reference code each follows (paths relative to the reference checkout):

  e4m3.py    E4M3FN codec with integer arithmetic        kernels/core/python/crit_kcore/formats.py:49-79,
                                                         tests/e4m3_vectors.py:17-22
  append.py  slot math and the append encodings          inference/attention-state/code/pages.py:439-453, 721-722,
                                                         872-895
  attend.py  float64 attention over stored values,       kernels/techniques/attention/paged-kv-attention/tests/
             gather + SDPA CPU path, dense FP32 windows, test_paged_kv_attention.py:71-81,
             online-softmax steps, LSE merge             inference/attention-state/code/pages.py:455-493,
                                                         inference/attention-state/code/device_attention.py:1148-1166,
                                                         1301-1335, kernels/core/python/crit_kcore/
                                                         attention_softmax.py:37-101,
                                                         inference/partitioned-attention/plugin.py:52-64,
                                                         inference/partitioned-attention/code/implementation.py:22-138

What pins each function (so a plausible mistake fails a check in tests/test_oracle.py):

  e4m3.encode / decode       the 24 reference-held vectors tests/inference/e4m3_scale_vectors.txt (committed as
                             tests/golden/e4m3_scale_vectors.txt), the closed-form decoder, exhaustive agreement with
                             torch's float8_e4m3fn cast on every 97th FP32 bit pattern in [-448, 448], and
                             decode(encode(v)) == v on all 254 finite codes
  append.*                   torch-CPU's own casts (library routine), the integer encoder above (independent
                             algorithm), IEEE-division counter-example (reciprocal multiply differs), untouched
                             bytes stay zero
  attend.reference           brute-force Python floats on tiny inputs; uniform-score closed form (mean of values)
  attend.sdpa_rows           against attend.reference to FP32 rounding
  attend.merge               worked example of inference/partitioned-attention/README.md:48-62 (merged output 5.0),
                             edge cases of inference/partitioned-attention/tests/test_device.py:70-77, independence
                             of the cut
  attend.fold / finish / lse folding any cut of a score vector equals the one-pass softmax

No function here is "parity unpinned".
"""
