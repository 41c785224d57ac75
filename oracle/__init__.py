"""Oracle package: CPU restatements of the reference algorithms, used only as the checker.

  torch_ref.py   floating-point operators, PyTorch ATen on the host (what the reference's own
                 --ref cpu tests compute)
  kv_oracle.c    byte/integer work in plain C: the paged-cache scatter, the page walk and the
                 stream-K partition
  cref.py        ctypes binding of the C oracle

TEST INFRASTRUCTURE: only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may
import this package.
"""
