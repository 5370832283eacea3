"""CPU oracle for the quantized-linear hot path — TEST INFRASTRUCTURE ONLY.

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import
this package; the product (latentq_llm_amd) never does.

`c_oracle`  : ctypes front end to lq_oracle.c (numpy in / numpy out).
`torch_ref` : op-for-op torch-CPU restatement of the reference's Python path
              (the "reference CPU dequant path" timed as the CPU baseline).
"""
