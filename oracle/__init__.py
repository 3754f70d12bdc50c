"""CPU oracle: a NumPy restatement of rai's Cpu evaluation path.

TEST INFRASTRUCTURE ONLY.  Nothing under rai_amd/ imports this package; it is
used by tests/, by __graft_entry__.smoke() and by the cpu_baseline leg of
bench.py as the checker / the timed CPU comparator, never as a fallback for the
HIP path.

The reference (cksac/rai 0.11.0) delegates all arithmetic to the third-party
crate candle-core 0.6 (Cargo.toml:31), whose sources are not part of the rai
tree and cannot be built here (no Rust toolchain).  Each function below restates
the rai-side composition it cites (file:line relative to the rai tree) on top of
the published semantics of the candle op it calls.

Pinning status (see tests/test_oracle_*.py):
  * index_select, argmax, broadcast arithmetic, casts, matmul, softmax,
    LayerNorm, RMSNorm, RoPE, activations, Linear: pinned against the known
    answers readable from the reference's own tests (rai-core/tests/ops.rs,
    tests/eval.rs), brute force on tiny inputs, closed forms and independent
    library routines (torch CPU, scipy).
  * Parity unpinned (only compiling candle could pin them): candle's exact f32
    summation order, its argmax NaN rule, its bf16 reduction accumulator width,
    and whether candle's Cpu backend runs bf16 matmul at all.  The oracle uses
    f32 accumulation with one rounding to bf16 per primitive.
"""
