"""CPU oracle for the logprob and sampling operators.

TEST INFRASTRUCTURE ONLY.  Nothing under kernel-align_amd/ imports, links or
runs this package; only tests/, __graft_entry__.smoke() and the cpu_baseline leg
of bench.py do, and only as the checker of the HIP kernels' results.

Modules:
  logprob_ref   torch/numpy restatement of the reference's logprob math
                (rl_engine/kernels/sampling.py:108-110,
                benchmarks/benchmark_grpo_op.py:52-54).
  sampling_ref  torch restatement of the reference's filter
                (benchmarks/benchmark_sampling.py:12-37) plus the inverse-CDF draw.
  exact         ctypes binding of ka_oracle.c, the exactly specified fixed-point
                restatement of the sampling operator (plain C, built by build.py).
"""
