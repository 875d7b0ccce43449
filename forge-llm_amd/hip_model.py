"""HipModel — host-side mirror of the reference's GPU model object.

Same surface as `MetalModel` in the reference (crates/forgellm-codegen-metal/src/lib.rs:
`new(weights: &[u8])` :4209, `forward(token_id) -> Vec<f32>` :5070,
`forward_prefill_batch(tokens)` :5568, `reset()` :5981), plus the CPU backend's
`forward_prefill` signature that returns the last token's logits
(crates/forgellm-codegen-cpu/src/emit.rs:4553).  Errors that panic in the reference raise
ForgeHipError here.
"""
import ctypes as C

import numpy as np


class HipModel:
    def __init__(self, config: dict, weights, proj_dtypes=None):
        """config: dict with the forge_hip_config fields; weights: the weights.bin bytes
        (numpy uint8 array, bytes or memoryview).  The blob is copied to the GPU.
        proj_dtypes: the GGML type ids of (q, k, v, o, gate, up, down) for a model with a storage format per
        projection (ProjectionDTypes, crates/forgellm-frontend/src/ir.rs:410-421); None: all in config["wdtype"]."""
        from . import Config, check, lib
        self._lib = lib()
        self._check = check
        self.config = dict(config)
        self._cfg = Config(**config)
        w = np.frombuffer(weights, dtype=np.uint8) if not isinstance(weights, np.ndarray) else weights
        w = np.ascontiguousarray(w, dtype=np.uint8)
        h = C.c_void_p()
        if proj_dtypes is None:
            check(self._lib.forge_hip_model_create(C.byref(self._cfg), w.ctypes.data_as(C.c_void_p), w.size, C.byref(h)))
        else:
            pd = np.ascontiguousarray(proj_dtypes, dtype=np.uint32)
            if pd.size != 7:
                raise ValueError("proj_dtypes: seven GGML type ids (q, k, v, o, gate, up, down)")
            check(self._lib.forge_hip_model_create_mixed(C.byref(self._cfg), pd.ctypes.data_as(C.c_void_p),
                                                         w.ctypes.data_as(C.c_void_p), w.size, C.byref(h)))
        self._h = h
        self.vocab = int(config["vocab"])

    @classmethod
    def from_gguf(cls, path: str, max_seq: int = 0, flags: int = 0):
        """Model straight from a GGUF file: what the reference does with `forge export-weights` + `Model::new`
        (crates/forgellm-cli/src/main.rs:2585-2757).  max_seq = 0 takes the file's context length."""
        from . import check, lib
        from .gguf import GgufFile, _declare
        L = lib()
        _declare(L)
        g = GgufFile(path)
        cfg, pd, _ = g.config_mixed(max_seq, flags)
        if all(d == cfg["wdtype"] for d in pd) and cfg["lm_head_dtype"] in (8, 2):
            cfg, pd = g.config(max_seq, flags), None       # every projection in one format: the uniform rules
        g.close()
        self = cls.__new__(cls)
        self._lib, self._check = L, check
        self.config = cfg
        self.proj_dtypes = pd
        h = C.c_void_p()
        check(L.forge_hip_model_create_from_gguf(path.encode(), max_seq, flags, C.byref(h)))
        self._h = h
        self.vocab = int(cfg["vocab"])
        return self

    # -- MetalModel::forward / model::forward
    def forward(self, token_id: int) -> np.ndarray:
        out = np.empty(self.vocab, np.float32)
        self._check(self._lib.forge_hip_forward(self._h, int(token_id), out.ctypes.data_as(C.c_void_p)))
        return out

    def forward_greedy(self, token_id: int) -> int:
        """forward + argmax (last index among ties) on the device."""
        nxt = C.c_uint32()
        self._check(self._lib.forge_hip_forward_greedy(self._h, int(token_id), C.byref(nxt)))
        return int(nxt.value)

    # -- MetalModel::forward_prefill_batch: fills the cache, no logits
    def forward_prefill_batch(self, tokens) -> None:
        t = np.ascontiguousarray(tokens, dtype=np.uint32)
        self._check(self._lib.forge_hip_prefill_batch(self._h, t.ctypes.data_as(C.c_void_p), t.size, None))

    # -- model::forward_prefill: returns the last token's logits
    def forward_prefill(self, tokens) -> np.ndarray:
        t = np.ascontiguousarray(tokens, dtype=np.uint32)
        out = np.empty(self.vocab, np.float32)
        self._check(self._lib.forge_hip_prefill_batch(self._h, t.ctypes.data_as(C.c_void_p), t.size,
                                                      out.ctypes.data_as(C.c_void_p)))
        return out

    # -- MetalModel::forward_profile: per-stage device time of one eager decode step
    STAGES = ("embedding", "rms_norm", "qkv_matmul", "rope_kv_store", "attention", "quantize_act", "o_matmul",
              "gate_up_matmul", "silu_mul", "down_matmul", "lm_head_matmul", "argmax")

    def forward_profile(self, token_id: int) -> dict:
        """{stage: (milliseconds, launches)} for one decode step launched eagerly with events around each kernel."""
        ms = (C.c_float * len(self.STAGES))()
        n = (C.c_uint32 * len(self.STAGES))()
        self._check(self._lib.forge_hip_forward_profile(self._h, int(token_id), ms, n))
        return {s: (float(ms[i]), int(n[i])) for i, s in enumerate(self.STAGES)}

    def prefill_profile(self, tokens) -> dict:
        t = np.ascontiguousarray(tokens, dtype=np.uint32)
        ms = (C.c_float * len(self.STAGES))()
        n = (C.c_uint32 * len(self.STAGES))()
        self._check(self._lib.forge_hip_prefill_profile(self._h, t.ctypes.data_as(C.c_void_p), t.size, ms, n))
        return {s: (float(ms[i]), int(n[i])) for i, s in enumerate(self.STAGES)}

    def reset(self) -> None:
        self._check(self._lib.forge_hip_reset(self._h))

    @property
    def decode_launches(self) -> int:
        """Kernel launches per decode step: 1 when the step runs as one resident kernel."""
        return int(self._lib.forge_hip_model_decode_launches(self._h))

    @property
    def pos(self) -> int:
        return int(self._lib.forge_hip_model_pos(self._h))

    def read_kv(self, layer: int, which: int) -> np.ndarray:
        """Cached K (which=0) or V (1) rows [0, pos) of a layer as fp16 bit patterns."""
        kv = self.config["kv_heads"] * self.config["head_dim"]
        out = np.empty((self.pos, kv), np.uint16)
        self._check(self._lib.forge_hip_model_read_kv(self._h, layer, which, out.ctypes.data_as(C.c_void_p)))
        return out

    def set_kv_pages(self, page_rows: int, page_table=None) -> None:
        """Paged KV cache: position t lives in row t % page_rows of pool page page_table[t // page_rows] (a permutation of
        range(max_seq // page_rows); page_rows a power of two >= 64).  page_rows = 0: the flat cache.  Only while the cache
        is empty; same results bit for bit under either layout."""
        if not page_rows:
            self._check(self._lib.forge_hip_model_set_kv_pages(self._h, 0, None, 0))
            return
        t = np.ascontiguousarray(page_table, dtype=np.uint32)
        self._check(self._lib.forge_hip_model_set_kv_pages(self._h, int(page_rows), t.ctypes.data_as(C.c_void_p), t.size))

    def generate_greedy(self, prompt, n_tokens: int):
        """The reference's greedy loop (crates/forgellm-codegen-cpu/src/project.rs:714-751 with
        temperature 0 and repeat penalty 1.0): prefill, argmax, then feed tokens back."""
        from .ops import argmax_host
        logits = self.forward_prefill(prompt)
        nxt = argmax_host(logits)
        out = [nxt]
        for _ in range(n_tokens - 1):
            nxt = self.forward_greedy(nxt)
            out.append(nxt)
        return out

    def set_poll_limit(self, polls: int) -> None:
        """Polls a workgroup of the resident decode kernel spends on one hand-over before the step gives up (0: default).
        A step that gives up raises ForgeHipError(ERR_HIP) and leaves position, token counts and context as they were."""
        self._check(self._lib.forge_hip_model_set_poll_limit(self._h, int(polls)))

    def set_repeat_penalty(self, penalty: float) -> None:
        """With a penalty > 1, forward_greedy takes the argmax of the logits after apply_repeat_penalty over every token
        fed since the last reset (project.rs:505-513, 742-744), on the device."""
        self._check(self._lib.forge_hip_model_set_repeat_penalty(self._h, float(penalty)))

    def generate(self, prompt, max_tokens: int = 128, temperature: float = 0.0, top_k: int = 0, top_p: float = 0.9,
                 repeat_penalty: float = 1.1, seed: int = 0xdeadbeef12345678, eos=()):
        """The generation loop of the generated main.rs with its defaults (project.rs:607-612, 714-751): prefill, sample
        (no penalty on the first token), then per token: stop on EOS, feed it, penalise every token fed so far, sample.
        Greedy decoding (temperature <= 0) stays on the device; with a temperature the logits come back and the
        host-side sampler runs."""
        from .ops import apply_repeat_penalty, sample
        rng = seed
        logits = self.forward_prefill(prompt)
        nxt, rng = sample(logits, temperature, top_k, top_p, rng)
        recent = [int(t) for t in prompt]
        out = []
        self.set_repeat_penalty(repeat_penalty)
        for _ in range(max_tokens):
            if nxt in eos:
                break
            out.append(nxt)
            recent.append(nxt)
            if temperature <= 0.0:
                nxt = self.forward_greedy(nxt)
            else:
                logits = self.forward(nxt)
                apply_repeat_penalty(logits, recent, repeat_penalty)
                nxt, rng = sample(logits, temperature, top_k, top_p, rng)
        return out

    def close(self):
        if getattr(self, "_h", None):
            self._lib.forge_hip_model_destroy(self._h)
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


def weights_nbytes(config: dict) -> int:
    from . import Config, lib
    c = Config(**config)
    return int(lib().forge_hip_weights_nbytes(C.byref(c)))


def weights_nbytes_mixed(config: dict, proj_dtypes) -> int:
    """Byte length of a weights.bin whose projections (q, k, v, o, gate, up, down) are stored in proj_dtypes."""
    from . import Config, lib
    c = Config(**config)
    pd = np.ascontiguousarray(proj_dtypes, dtype=np.uint32)
    if pd.size != 7:
        raise ValueError("proj_dtypes: seven GGML type ids (q, k, v, o, gate, up, down)")
    return int(lib().forge_hip_weights_nbytes_mixed(C.byref(c), pd.ctypes.data_as(C.c_void_p)))
