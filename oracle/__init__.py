"""CPU oracle of OpenRLHF's token-level RL numerics. TEST INFRASTRUCTURE ONLY.

This package restates, on CPU torch, the algorithms of the reference functions the HIP library
replaces, keeping the reference's op sequence (fp32 up-cast, gather minus chunked logsumexp,
eager elementwise chains, Python reverse-time loops), so that it doubles as the timed CPU
baseline. Every function cites the reference lines it follows. Running the same code on
float64 inputs gives the high-precision oracle the tolerances are checked against.

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import it. Nothing in
openrlhf_amd/ imports it; the product path has no CPU route.

The reference is Python and is not imported anywhere: each function below is pinned instead by
tests/test_oracle_*.py against closed forms, brute-force scalar loops, library routines and the
identities the reference's own tests/test_loss_aggregation.py asserts, and against the
hand-computed vectors in tests/golden/. The flash-attn Triton cross-entropy the reference
prefers when installed (openrlhf/models/utils.py:147-150, flash-attn 2.8.3, not vendored) is
third-party code that is absent here; it is defined to return the same x[label] - logsumexp(x)
as the in-tree fallback this oracle follows, and that equality is "parity unpinned".
"""
