"""Host handle of the decoder-only model drivers in librai_hip.so.

Mirrors the public surface of rai-models' LLMs (rai-models/src/llm/phi2.rs:316-353:
`Model::new(cfg, dtype, device)`, `fwd`, `clear_kv_cache`) and the greedy loop
of examples/phi2/src/main.rs:75-95.  All compute happens in the HIP library.
"""
from __future__ import annotations

import ctypes as C

import numpy as np

from . import _lib
from ._lib import ARCH, DTYPE_BY_NAME, UNARY, DecoderConfig, call

_ACT = {"gelu_new": "new_gelu", "new_gelu": "new_gelu", "gelu": "gelu", "silu": "silu", "relu": "relu"}


class Decoder:
    def __init__(self, arch, dtype, *, vocab_size, hidden_size, intermediate_size, num_hidden_layers,
                 num_attention_heads, num_key_value_heads=None, head_dim=None, rotary_dim=None,
                 max_position_embeddings=2048, hidden_act="gelu_new", tie_word_embeddings=False, rope_theta=10000.0,
                 norm_eps=1e-5, max_batch=1, max_context=None, rope_tables_f32=False, qk_layernorm=False,
                 dev=0):
        head_dim = head_dim or hidden_size // num_attention_heads
        cfg = DecoderConfig()
        cfg.arch = ARCH[arch]
        cfg.dtype = DTYPE_BY_NAME[dtype]
        cfg.vocab_size = vocab_size
        cfg.hidden_size = hidden_size
        cfg.intermediate_size = intermediate_size
        cfg.num_hidden_layers = num_hidden_layers
        cfg.num_attention_heads = num_attention_heads
        cfg.num_key_value_heads = num_key_value_heads or num_attention_heads
        cfg.head_dim = head_dim
        cfg.rotary_dim = rotary_dim or head_dim
        cfg.max_position_embeddings = max_position_embeddings
        cfg.hidden_act = UNARY[_ACT[hidden_act]]
        cfg.tie_word_embeddings = int(tie_word_embeddings)
        cfg.max_batch = max_batch
        cfg.max_context = max_context or max_position_embeddings
        cfg.rope_tables_f32 = int(rope_tables_f32)
        cfg.qk_layernorm = int(qk_layernorm)
        cfg.rope_theta = rope_theta
        cfg.norm_eps = norm_eps
        self.cfg, self.dtype, self.dev = cfg, dtype, dev
        self._h = C.c_void_p()
        call("rai_hip_init", dev)
        call("rai_hip_decoder_create", dev, C.byref(cfg), C.byref(self._h))

    def close(self):
        if self._h:
            _lib.load().rai_hip_decoder_destroy(self._h)
            self._h = C.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def param_names(self):
        n = C.c_int32(0)
        call("rai_hip_decoder_param_count", self._h, C.byref(n))
        out = {}
        buf = C.create_string_buffer(256)
        for i in range(n.value):
            numel = C.c_int64(0)
            call("rai_hip_decoder_param_name", self._h, i, buf, 256, C.byref(numel))
            out[buf.value.decode()] = numel.value
        return out

    def load_param(self, name, storage):
        """`storage`: host array in the model dtype's storage form (bf16 = uint16 bits)."""
        a = np.ascontiguousarray(storage)
        call("rai_hip_decoder_load_param", self._h, name.encode(), a.ctypes.data_as(C.c_void_p), a.nbytes)

    def load_safetensors(self, paths):
        """Module::update_by_safetensors (rai-core/src/nn.rs:39-55): every parameter by name from the given files."""
        paths = [paths] if isinstance(paths, (str, bytes)) or hasattr(paths, "__fspath__") else list(paths)
        arr = (C.c_char_p * len(paths))(*[str(p).encode() for p in paths])
        call("rai_hip_decoder_load_safetensors", self._h, arr, len(paths))

    def forward(self, ids, want_logits=True):
        """Model::fwd: ids [B, S] u32 -> (logits [B, vocab] f32, greedy tokens [B] u32)."""
        ids = np.ascontiguousarray(ids, dtype=np.uint32)
        b, s = ids.shape
        logits = np.empty((b, self.cfg.vocab_size), np.float32) if want_logits else None
        toks = np.empty((b,), np.uint32)
        call("rai_hip_decoder_forward", self._h, ids.ctypes.data_as(C.POINTER(C.c_uint32)), b, s,
             logits.ctypes.data_as(C.POINTER(C.c_float)) if want_logits else None,
             toks.ctypes.data_as(C.POINTER(C.c_uint32)))
        return logits, toks

    def forward_hidden(self, ids=None, hidden_in=None, want_logits=False):
        """Model::fwd with the layer stack's ends open: ids [B, S] u32, or hidden_in [B, S, hidden] in the model
        dtype's storage form in place of the embedding lookup -> (residual stream after the last layer [B, S, hidden]
        f32, logits [B, vocab] f32 or None, greedy tokens [B] u32)."""
        if ids is not None:
            ids = np.ascontiguousarray(ids, dtype=np.uint32)
            b, s = ids.shape
            ids_p, hid_p = ids.ctypes.data_as(C.POINTER(C.c_uint32)), None
        else:
            hidden_in = np.ascontiguousarray(hidden_in)
            b, s, h = hidden_in.shape
            assert h == self.cfg.hidden_size
            ids_p, hid_p = None, hidden_in.ctypes.data_as(C.c_void_p)
        hidden = np.empty((b, s, self.cfg.hidden_size), np.float32)
        logits = np.empty((b, self.cfg.vocab_size), np.float32) if want_logits else None
        toks = np.empty((b,), np.uint32)
        call("rai_hip_decoder_forward_hidden", self._h, ids_p, hid_p, b, s, hidden.ctypes.data_as(C.POINTER(C.c_float)),
             logits.ctypes.data_as(C.POINTER(C.c_float)) if want_logits else None,
             toks.ctypes.data_as(C.POINTER(C.c_uint32)))
        return hidden, logits, toks

    def generate(self, prompt, n_new):
        """Greedy decode: returns (tokens [B, n_new], prefill_ms, decode_ms)."""
        prompt = np.ascontiguousarray(prompt, dtype=np.uint32)
        b, s = prompt.shape
        toks = np.empty((b, n_new), np.uint32)
        pm, dm = C.c_float(0), C.c_float(0)
        call("rai_hip_decoder_generate", self._h, prompt.ctypes.data_as(C.POINTER(C.c_uint32)), b, s, n_new,
             toks.ctypes.data_as(C.POINTER(C.c_uint32)), C.byref(pm), C.byref(dm))
        return toks, pm.value, dm.value

    def generate_sampled(self, prompt, n_new, repeat_penalty=1.10, repeat_last_n=64, eos_token=None):
        """The example loop (examples/phi2/src/main.rs:72-95) with its repeat penalty and last-maximum
        argmax: returns (tokens [B, n_new], n_generated [B], prefill_ms, decode_ms)."""
        prompt = np.ascontiguousarray(prompt, dtype=np.uint32)
        b, s = prompt.shape
        toks = np.empty((b, n_new), np.uint32)
        ngen = np.empty((b,), np.int32)
        pm, dm = C.c_float(0), C.c_float(0)
        call("rai_hip_decoder_generate_sampled", self._h, prompt.ctypes.data_as(C.POINTER(C.c_uint32)), b, s, n_new,
             float(repeat_penalty), int(repeat_last_n), -1 if eos_token is None else int(eos_token),
             toks.ctypes.data_as(C.POINTER(C.c_uint32)), ngen.ctypes.data_as(C.POINTER(C.c_int32)), C.byref(pm),
             C.byref(dm))
        return toks, ngen, pm.value, dm.value

    def clear_kv_cache(self):
        call("rai_hip_decoder_clear_kv_cache", self._h)

    def context_len(self):
        n = C.c_int32(0)
        call("rai_hip_decoder_context_len", self._h, C.byref(n))
        return n.value

    def time_decode_step(self, sweeps=20):
        """Mean launch time (us) and algorithmic bytes of the persistent per-token decode kernel."""
        us, by = C.c_float(0), C.c_double(0)
        call("rai_hip_decoder_time_decode_step", self._h, int(sweeps), C.byref(us), C.byref(by))
        return us.value, by.value

    def time_decode_linear(self, sweeps=20):
        """Mean launch time (us) and algorithmic bytes of the decode weight-streaming kernel."""
        us, by = C.c_float(0), C.c_double(0)
        call("rai_hip_decoder_time_decode_linear", self._h, int(sweeps), C.byref(us), C.byref(by))
        return us.value, by.value


def safetensors_index_files(index_json_path):
    """The shard files a model.safetensors.index.json names (rai/src/lib.rs:17-42, without the hub download)."""
    buf = C.create_string_buffer(1 << 16)
    n = C.c_int32(0)
    call("rai_hip_safetensors_index_files", str(index_json_path).encode(), buf, len(buf), C.byref(n))
    files = buf.value.decode().split("\n") if n.value else []
    assert len(files) == n.value
    return files
