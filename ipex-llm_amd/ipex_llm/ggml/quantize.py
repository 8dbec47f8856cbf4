"""qtype name -> integer table (python/llm/src/ipex_llm/ggml/quantize.py:28-57).

The integers are part of the on-disk and C ABI contract, so the whole table is
kept even though only five entries have kernels behind them in this build.
"""

ggml_tensor_qtype = {"sym_int4": 2,   # ggml Q4_0
                     "asym_int4": 3,  # ggml Q4_1
                     "sym_int5": 6,
                     "asym_int5": 7,
                     "sym_int8": 8,   # ggml Q8_0
                     "nf4": 10,
                     "nf3": 11,
                     "fp16": 12,
                     "fp8_e4m3": 15,
                     "fp4": 16,
                     "mixed_fp4": 17,
                     "mixed_fp8": 18,
                     "fp8_e5m2": 19,
                     "fp8": 19,
                     "bf16": 20,
                     "gguf_iq2_xxs": 21,
                     "gguf_iq2_xs": 22,
                     "q2_k": 23,
                     "gguf_iq1_s": 24,
                     "gguf_iq1_m": 25,
                     "q6_k": 26,
                     "q4_k": 27,
                     "q5_k": 28,
                     "fp6": 29,
                     "fp6_k": 30,
                     "sym_int4_rtn": 31,
                     "sym_int8_rtn": 32,
                     "asym_int4_rtn": 33,
                     "woq_int4": 34,
                     }

# qtypes that have MI355X kernels in this build
SUPPORTED_QTYPES = {k: ggml_tensor_qtype[k] for k in
                    ("sym_int4", "asym_int4", "sym_int8", "nf4", "fp8_e4m3")}
