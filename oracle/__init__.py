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
  * gather, index_add, scatter_add: pinned against torch's routines (integer
    dtypes and exactly representable floats, so the order of additions cannot
    matter), the shapes of rai-core/tests/ops.rs:156-161 and
    tests/check_grad.rs:117-169, and the adjoint identities their vjp rules
    rely on.
  * the example loop's token choice (oracle/sampling.py): pinned against a
    pure-Python max_by over Rust's documented f32::total_cmp and hand-computed
    penalty rows.
  * the model files (phi2, qwen2/gemma, phi3): pinned against Hugging Face
    transformers models built locally from in-memory configs with the oracle's
    seeded weights.
  * Parity unpinned (only compiling candle could pin them): candle's exact f32
    summation order, its argmax NaN rule, its bf16 reduction accumulator width,
    whether candle's Cpu backend runs bf16 matmul at all, and that its
    index_add / scatter_add loops add source rows in index order in the element
    type (one rounding per addition), which is what the oracle does.  The oracle uses
    f32 accumulation with one rounding to bf16 per primitive.
"""
