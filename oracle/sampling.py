"""Token choice of the reference's example loop, restated (TEST INFRASTRUCTURE ONLY, like the rest
of this package).

Follows examples/phi2/src/main.rs: sample_argmax :29-37, apply_repeat_penalty :39-50, the loop
:72-95 (examples/qwen2 and examples/gemma hold the same three pieces).  The example works on the
logits row as a Vec<f32> (main.rs:78 `as_vec(dtype)` with dtype F32); a bf16 model's row is widened
to f32 first, which is exact.

Pinned by tests/test_oracle_sampling.py: sample_argmax against a pure-Python max_by over Rust's
documented f32::total_cmp bit trick (ties, signed zeros, infinities, NaNs of both signs),
apply_repeat_penalty against hand-computed rows and against a per-element loop.
"""
import numpy as np


def total_order_key(x):
    """u32 key whose unsigned order is f32::total_cmp's order: negative values have all their bits
    flipped, the others get the sign bit set."""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    return np.where(u & np.uint32(0x80000000), ~u, u | np.uint32(0x80000000))


def sample_argmax(logits):
    """main.rs:29-37: `iter().enumerate().max_by(total_cmp)` returns the LAST of several equal maxima."""
    key = total_order_key(np.asarray(logits, dtype=np.float32).reshape(-1))
    return np.uint32(len(key) - 1 - int(np.argmax(key[::-1])))


def apply_repeat_penalty(logits, penalty, context):
    """main.rs:39-50: every token id present in `context` (a set: once per id) has its logit divided
    by the penalty when it is >= 0 and multiplied otherwise; f32 arithmetic.  Returns a new row."""
    out = np.array(logits, dtype=np.float32, copy=True).reshape(-1)
    p = np.float32(penalty)
    ids = np.unique(np.asarray(context, dtype=np.uint32))
    ids = ids[ids < out.shape[0]]
    v = out[ids]
    with np.errstate(all="ignore"):
        out[ids] = np.where(v >= 0, v / p, v * p).astype(np.float32)
    return out


def choose(logits_row, tokens_so_far, repeat_penalty, repeat_last_n):
    """main.rs:78-82 for one sequence: the penalty is skipped when it is below 1."""
    row = np.asarray(logits_row, dtype=np.float32)
    if repeat_penalty >= 1.0:
        start = max(0, len(tokens_so_far) - repeat_last_n)
        row = apply_repeat_penalty(row, repeat_penalty, tokens_so_far[start:])
    return sample_argmax(row), row


def sampled_decode(model, prompt, n_new, repeat_penalty=1.10, repeat_last_n=64, eos_token=None):
    """main.rs:72-95 for every row of prompt [B, S] independently: the whole prompt first, then one
    token per step.  Runs n_new steps regardless of eos; returns tokens [B, n_new] u32, n_generated [B]
    (where the example's loop would have stopped: after the first eos_token) and, per step, the
    penalised f32 rows [B, vocab] the choice was made from."""
    prompt = np.asarray(prompt, dtype=np.uint32)
    model.clear_kv_cache()
    b = prompt.shape[0]
    seqs = [list(prompt[i]) for i in range(b)]
    tokens, rows_all = [], []
    ctx = prompt
    for _ in range(n_new):
        logits = np.asarray(model.fwd(ctx), dtype=np.float32)
        nxt, rows = np.empty((b,), np.uint32), []
        for i in range(b):
            nxt[i], row = choose(logits[i], seqs[i], repeat_penalty, repeat_last_n)
            seqs[i].append(nxt[i])
            rows.append(row)
        tokens.append(nxt)
        rows_all.append(np.stack(rows))
        ctx = nxt.reshape(-1, 1)
    tokens = np.stack(tokens, axis=1)
    n_gen = np.full((b,), n_new, np.int32)
    if eos_token is not None:
        for i in range(b):
            hit = np.nonzero(tokens[i] == np.uint32(eos_token))[0]
            if hit.size:
                n_gen[i] = hit[0] + 1
    return tokens, n_gen, rows_all
