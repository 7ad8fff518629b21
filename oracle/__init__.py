"""Oracle: CPU restatements of the reference's algorithms for the hot path.

TEST INFRASTRUCTURE ONLY — imported by tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg,
never by the product under triton-distributed_amd/.

  golden.py  torch / numpy restatement of the reference's golden computations
  c/         scalar C restatement (built by `make -C oracle`), loaded through cref.py
"""
