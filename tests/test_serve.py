"""The OpenAI-compatible serve loop (forge-llm_amd/serve.py) against what the generated binary of the reference does
(crates/forgellm-codegen-metal/src/lib.rs:8564-8900): request parsing and status codes, ChatML formatting, prefill split,
greedy loop with the hard-wired end-of-sequence id 2, JSON and event-stream bodies.  The host logic runs against a
scripted model on the CPU; the GPU test holds the served text to the model's own greedy generation."""
import json
import threading
import urllib.error
import urllib.request

import numpy as np
import pytest


class ScriptedModel:
    """Answers forward_greedy from a script and records what it was fed."""

    def __init__(self, script):
        self.script = list(script)
        self.calls = []
        self.i = 0

    def reset(self):
        self.calls.append(("reset",))
        self.i = 0

    def set_repeat_penalty(self, p):
        self.calls.append(("penalty", p))

    def forward_prefill_batch(self, tokens):
        self.calls.append(("prefill_batch", [int(t) for t in tokens]))

    def forward_greedy(self, token):
        self.calls.append(("forward", int(token)))
        out = self.script[self.i]
        self.i += 1
        return out


class Enc:
    def __init__(self, ids):
        self.ids = ids


class CharTokenizer:
    """One token per character: id = ord(c) + 3 (0..2 stay special)."""

    def encode(self, text, add_special_tokens=True):
        assert add_special_tokens is True
        return Enc([ord(c) + 3 for c in text])

    def decode(self, ids, skip_special_tokens=False):
        assert skip_special_tokens is False
        if ids[0] == 7:
            raise ValueError("undecodable")
        return "".join(chr(i - 3) for i in ids)


def tok(c):
    return ord(c) + 3


MSGS = [{"role": "system", "content": "be brief"}, {"role": "user", "content": "hi"}]
PROMPT = "<|im_start|>system\nbe brief<|im_end|>\n<|im_start|>user\nhi<|im_end|>\n<|im_start|>assistant\n"


def post(server, payload):
    body = payload if isinstance(payload, bytes) else json.dumps(payload).encode()
    return server.handle("POST", "/v1/chat/completions", body)


def test_chatml_prompt(fh):
    assert fh.serve.format_chat_messages(MSGS) == PROMPT
    assert fh.serve.format_chat_messages([]) == "<|im_start|>assistant\n"


def test_completion_json_and_model_calls(fh):
    m = ScriptedModel([tok("o"), tok("k"), 2, tok("x")])
    s = fh.serve.ChatServer(m, CharTokenizer())
    status, headers, body = post(s, {"messages": MSGS, "temperature": 0.7, "model": "whatever"})
    assert status == 200 and headers["Content-Type"] == "application/json"
    r = json.loads(body)
    assert r["id"] == "chatcmpl-1" and r["object"] == "chat.completion"
    assert r["choices"] == [{"index": 0, "message": {"role": "assistant", "content": "ok"}, "finish_reason": "stop"}]
    u = r["usage"]
    assert u["prefill_tokens"] == len(PROMPT) and u["generation_tokens"] == 2
    assert isinstance(u["prefill_time_ms"], int) and isinstance(u["generation_time_ms"], int) and u["tokens_per_sec"] > 0
    ids = [ord(c) + 3 for c in PROMPT]
    # reset, all tokens but the last as one batch, the last through the decode step, then the fed-back tokens
    assert m.calls == [("reset",), ("penalty", 1.0), ("prefill_batch", ids[:-1]), ("forward", ids[-1]),
                       ("forward", tok("o")), ("forward", tok("k"))]


def test_completion_stops_at_max_tokens_and_resets_per_request(fh):
    m = ScriptedModel([tok("a")] * 600)
    s = fh.serve.ChatServer(m, CharTokenizer())
    _, _, body = post(s, {"messages": MSGS, "max_tokens": 5})
    assert json.loads(body)["choices"][0]["message"]["content"] == "aaaaa"
    _, _, body = post(s, {"messages": MSGS})                      # default of the reference: 256
    r = json.loads(body)
    assert r["choices"][0]["message"]["content"] == "a" * 256 and r["usage"]["generation_tokens"] == 256
    assert [c for c in m.calls if c == ("reset",)] == [("reset",)] * 2
    _, _, body = post(s, {"messages": MSGS, "max_tokens": 0})
    assert json.loads(body)["choices"][0]["message"]["content"] == ""


def test_first_token_eos_and_undecodable_token(fh):
    s = fh.serve.ChatServer(ScriptedModel([2]), CharTokenizer())
    r = json.loads(post(s, {"messages": MSGS})[2])
    assert r["choices"][0]["message"]["content"] == "" and r["usage"]["generation_tokens"] == 0
    # a token the tokenizer cannot decode is skipped in the text and still counted
    s = fh.serve.ChatServer(ScriptedModel([tok("a"), 7, tok("b"), 2]), CharTokenizer())
    r = json.loads(post(s, {"messages": MSGS})[2])
    assert r["choices"][0]["message"]["content"] == "ab" and r["usage"]["generation_tokens"] == 3


def test_event_stream_body(fh):
    m = ScriptedModel([tok("h"), tok('"'), tok("\n"), tok("é"), 2])
    s = fh.serve.ChatServer(m, CharTokenizer())
    status, headers, body = post(s, {"messages": MSGS, "stream": True})
    assert status == 200 and headers == {"Content-Type": "text/event-stream", "Cache-Control": "no-cache"}
    text = body.decode("utf-8")
    assert text.endswith("\n\ndata: [DONE]\n\n")
    events = text.split("\n\n")[:-1]
    assert events[-1] == "data: [DONE]"
    chunks = [json.loads(e[len("data: "):]) for e in events[:-1]]
    assert all(e.startswith("data: ") for e in events)
    assert [c["choices"][0]["delta"].get("content") for c in chunks] == ["h", '"', "\n", "é", None]
    for c in chunks[:-1]:
        assert c["id"] == "chatcmpl-1" and c["object"] == "chat.completion.chunk" and c["choices"][0]["finish_reason"] is None
    last = chunks[-1]
    assert last["choices"] == [{"index": 0, "delta": {}, "finish_reason": "stop"}]
    assert set(last["usage"]) == {"prefill_tokens", "prefill_time_ms", "generation_tokens", "generation_time_ms", "tokens_per_sec"}
    assert last["usage"]["generation_tokens"] == 4 and last["usage"]["prefill_tokens"] == len(PROMPT)
    # the first chunk byte for byte as the reference writes it
    assert events[0] == 'data: {"id":"chatcmpl-1","object":"chat.completion.chunk","choices":[{"index":0,"delta":{"content":"h"},"finish_reason":null}]}'
    assert "é" in text                                            # serde_json leaves non-ASCII text as it is


@pytest.mark.parametrize("payload", [b"{not json", b"[1, 2]", b'{"stream": true}', b'{"messages": "hi"}',
                                     b'{"messages": [{"role": "user"}]}', b'{"messages": [{"role": 1, "content": "x"}]}',
                                     b'{"messages": [], "max_tokens": -1}', b'{"messages": [], "stream": "yes"}',
                                     b'\xff\xfe'])
def test_bad_requests_are_400(fh, payload):
    m = ScriptedModel([2])
    status, _, body = post(fh.serve.ChatServer(m, CharTokenizer()), payload)
    assert status == 400 and json.loads(body)["error"].startswith("Invalid JSON: ")
    assert m.calls == []                                          # nothing reached the model


def test_tokenizer_failure_is_500(fh):
    class Broken(CharTokenizer):
        def encode(self, text, add_special_tokens=True):
            raise RuntimeError("no vocabulary")
    status, _, body = post(fh.serve.ChatServer(ScriptedModel([2]), Broken()), {"messages": MSGS})
    assert status == 500 and json.loads(body)["error"] == "Tokenization failed: no vocabulary"


class LimitedModel(ScriptedModel):
    """A scripted model with a cache of `max_seq` rows that raises, like HipModel, when a token is fed past its end."""

    def __init__(self, script, max_seq):
        super().__init__(script)
        self.config = {"max_seq": max_seq}
        self.pos = 0

    def reset(self):
        super().reset()
        self.pos = 0

    def forward_prefill_batch(self, tokens):
        if self.pos + len(tokens) > self.config["max_seq"]:
            raise RuntimeError("prompt does not fit the KV cache")
        super().forward_prefill_batch(tokens)
        self.pos += len(tokens)

    def forward_greedy(self, token):
        if self.pos >= self.config["max_seq"]:
            raise RuntimeError("KV cache is full (pos == max_seq)")
        self.pos += 1
        return super().forward_greedy(token)


def test_context_limit_is_an_answer_not_an_exception(fh):
    """The cache's end: a prompt that fills it is a 400, a generation that reaches it ends with finish_reason "length"
    after exactly the tokens that fit, and a model call that fails all the same comes back as a 500 body."""
    n = len(PROMPT)
    s = fh.serve.ChatServer(LimitedModel([tok("a")] * 64, n), CharTokenizer())
    status, _, body = post(s, {"messages": MSGS})
    assert status == 400 and "Prompt too long" in json.loads(body)["error"]
    # room for 3 more rows: the prompt's n tokens, then the tokens "a", "a", "a" can still be fed; the 4th pick is the last
    m = LimitedModel([tok("a")] * 64, n + 3)
    s = fh.serve.ChatServer(m, CharTokenizer())
    status, _, body = post(s, {"messages": MSGS, "max_tokens": 50})
    resp = json.loads(body)
    assert status == 200 and resp["choices"][0]["finish_reason"] == "length"
    assert resp["choices"][0]["message"]["content"] == "aaaa" and resp["usage"]["generation_tokens"] == 4
    assert m.pos == n + 3
    status, _, body = post(s, {"messages": MSGS, "max_tokens": 50, "stream": True})
    assert status == 200 and b'"finish_reason":"length"' in body
    # max_tokens below the room: an ordinary stop
    status, _, body = post(s, {"messages": MSGS, "max_tokens": 2})
    assert json.loads(body)["choices"][0]["finish_reason"] == "stop"

    class Broken(ScriptedModel):
        def forward_greedy(self, token):
            raise RuntimeError("device lost")
    status, _, body = post(fh.serve.ChatServer(Broken([]), CharTokenizer()), {"messages": MSGS})
    assert status == 500 and "device lost" in json.loads(body)["error"]


def test_other_routes(fh):
    s = fh.serve.ChatServer(ScriptedModel([2]), CharTokenizer())
    status, headers, body = s.handle("GET", "/v1/models")
    assert status == 200 and headers["Content-Type"] == "application/json"
    assert json.loads(body) == {"object": "list", "data": [{"id": "forgellm-hip", "object": "model", "owned_by": "forgellm"}]}
    assert s.handle("GET", "/health") == (200, {}, b'{"status":"ok"}')
    for method, url in (("GET", "/"), ("GET", "/v1/chat/completions"), ("POST", "/health"), ("PUT", "/v1/models")):
        assert s.handle(method, url) == (404, {}, b"Not Found")


def _serve_in_thread(fh, model, tokenizer):
    httpd = fh.serve.make_http_server(model, tokenizer, 0, host="127.0.0.1")
    t = threading.Thread(target=httpd.serve_forever, daemon=True)
    t.start()
    return httpd, t, "http://127.0.0.1:%d" % httpd.server_address[1]


def test_over_http(fh):
    httpd, t, base = _serve_in_thread(fh, ScriptedModel([tok("y"), tok("o"), 2] * 4), CharTokenizer())
    try:
        assert urllib.request.urlopen(base + "/health", timeout=10).read() == b'{"status":"ok"}'
        req = urllib.request.Request(base + "/v1/chat/completions", data=json.dumps({"messages": MSGS}).encode(), method="POST")
        with urllib.request.urlopen(req, timeout=10) as r:
            assert r.status == 200 and r.headers["Content-Type"] == "application/json"
            assert json.loads(r.read())["choices"][0]["message"]["content"] == "yo"
        req = urllib.request.Request(base + "/v1/chat/completions", data=json.dumps({"messages": MSGS, "stream": True}).encode(), method="POST")
        with urllib.request.urlopen(req, timeout=10) as r:
            assert r.headers["Content-Type"] == "text/event-stream" and r.headers["Cache-Control"] == "no-cache"
            assert r.read().decode().endswith("data: [DONE]\n\n")
        with pytest.raises(urllib.error.HTTPError) as e:
            urllib.request.urlopen(urllib.request.Request(base + "/v1/chat/completions", data=b"{", method="POST"), timeout=10)
        assert e.value.code == 400
        with pytest.raises(urllib.error.HTTPError) as e:
            urllib.request.urlopen(base + "/nothing", timeout=10)
        assert e.value.code == 404 and e.value.read() == b"Not Found"
    finally:
        httpd.shutdown()
        httpd.server_close()
        t.join(timeout=10)


def _word_tokenizer(vocab_size):
    """A `tokenizers` word-level tokenizer built in memory: token i is the word w<i>; ids 0..2 are special."""
    tokenizers = pytest.importorskip("tokenizers")
    vocab = {"<unk>": 0, "<s>": 1, "</s>": 2}
    for i in range(3, vocab_size):
        vocab["w%d" % i] = i
    tk = tokenizers.Tokenizer(tokenizers.models.WordLevel(vocab, unk_token="<unk>"))
    tk.pre_tokenizer = tokenizers.pre_tokenizers.WhitespaceSplit()
    return tk


def test_word_tokenizer_round_trip():
    tk = _word_tokenizer(64)
    assert tk.encode("w5 w63 nope", add_special_tokens=True).ids == [5, 63, 0]
    assert tk.decode([17], skip_special_tokens=False) == "w17"


@pytest.mark.gpu
def test_served_text_is_the_models_greedy_generation(fh):
    """Over HTTP, with a real model on the GPU and a real `tokenizers` tokenizer: the text of both response forms is the
    decoding of the model's own greedy continuation of the ChatML prompt, cut at token 2 or at max_tokens."""
    cfg = fh.synth.tiny(max_seq=1024, vocab=512)
    blob = fh.synth.make_weights_blob(cfg, seed=11)
    model = fh.HipModel(cfg, blob)
    tk = _word_tokenizer(cfg["vocab"])
    msgs = [{"role": "user", "content": "w40 w41 w42 w43 w44 w45 w46"}]
    prompt_ids = tk.encode(fh.serve.format_chat_messages(msgs), add_special_tokens=True).ids
    assert len(prompt_ids) > 8
    want = model.generate_greedy(prompt_ids, 24)
    model.reset()
    cut = want.index(2) if 2 in want else len(want)
    want_text = "".join(tk.decode([t], skip_special_tokens=False) for t in want[:cut])
    httpd, t, base = _serve_in_thread(fh, model, tk)
    try:
        for stream in (False, True, False):
            req = urllib.request.Request(base + "/v1/chat/completions",
                                         data=json.dumps({"messages": msgs, "max_tokens": 24, "stream": stream}).encode(), method="POST")
            with urllib.request.urlopen(req, timeout=60) as r:
                body = r.read().decode()
            if stream:
                chunks = [json.loads(e[6:]) for e in body.split("\n\n") if e.startswith("data: {")]
                got = "".join(c["choices"][0]["delta"].get("content", "") for c in chunks)
                usage = chunks[-1]["usage"]
            else:
                r = json.loads(body)
                got, usage = r["choices"][0]["message"]["content"], r["usage"]
            assert got == want_text
            assert usage["prefill_tokens"] == len(prompt_ids) and usage["generation_tokens"] == cut
    finally:
        httpd.shutdown()
        httpd.server_close()
        t.join(timeout=10)
        model.close()
