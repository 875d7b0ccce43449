"""OpenAI-compatible serve loop over a HipModel — the `serve` function of the binary the reference generates
(crates/forgellm-codegen-metal/src/lib.rs:8564-8900), behaviour for behaviour:

  POST /v1/chat/completions   ChatRequest {messages, stream?, max_tokens? = 256, temperature?, model?}
  GET  /v1/models             one model entry
  GET  /health                {"status":"ok"}
  anything else               404 "Not Found"

One request at a time (the reference walks `server.incoming_requests()` in a loop).  Every request resets the KV
cache, formats the messages as ChatML (lib.rs:8594-8603), tokenises with special tokens, prefills all tokens but the
last as a batch and feeds the last one through `forward` (lib.rs:8607-8622), then decodes greedily — the request's
temperature is parsed and ignored, as in the reference (lib.rs:8730) — until `max_tokens` tokens were produced or the
next token is 2, the reference's hard-wired end-of-sequence id (lib.rs:8757, 8816).  A streaming request gets the
whole event stream as one body, again like the reference, which builds `sse_body` before it responds.

The greedy loop itself runs on the GPU (`forward_greedy`: the last maximum among equal logits, which is what the
reference's `max_by(partial_cmp)` returns).
"""
import json
import time
from http.server import BaseHTTPRequestHandler, HTTPServer

EOS_TOKEN = 2            # lib.rs:8757
DEFAULT_MAX_TOKENS = 256  # lib.rs:8729
MAX_BODY_BYTES = 16 << 20  # a larger request body is refused with 413 before it is read (the reference reads any length)
MODEL_ID = "forgellm-hip"


def format_chat_messages(messages) -> str:
    """ChatML, ending with the opened assistant turn (lib.rs:8594-8603)."""
    prompt = ""
    for m in messages:
        prompt += "<|im_start|>%s\n%s<|im_end|>\n" % (m["role"], m["content"])
    return prompt + "<|im_start|>assistant\n"


class BadRequest(Exception):
    pass


def parse_chat_request(body: bytes) -> dict:
    """The fields serde would accept for ChatRequest (lib.rs:8574-8592); anything else is the reference's 400."""
    try:
        req = json.loads(body.decode("utf-8"))
    except (ValueError, UnicodeDecodeError) as e:
        raise BadRequest(str(e))
    if not isinstance(req, dict):
        raise BadRequest("invalid type: expected struct ChatRequest")
    if "messages" not in req:
        raise BadRequest("missing field `messages`")
    msgs = req["messages"]
    if not isinstance(msgs, list):
        raise BadRequest("invalid type for `messages`: expected a sequence")
    for m in msgs:
        if not isinstance(m, dict):
            raise BadRequest("invalid type: expected struct ChatMessage")
        for k in ("role", "content"):
            if k not in m:
                raise BadRequest("missing field `%s`" % k)
            if not isinstance(m[k], str):
                raise BadRequest("invalid type for `%s`: expected a string" % k)
    stream = req.get("stream")
    if stream is not None and not isinstance(stream, bool):
        raise BadRequest("invalid type for `stream`: expected a boolean")
    max_tokens = req.get("max_tokens")
    if max_tokens is not None and (isinstance(max_tokens, bool) or not isinstance(max_tokens, int) or max_tokens < 0):
        raise BadRequest("invalid type for `max_tokens`: expected usize")
    temperature = req.get("temperature")
    if temperature is not None and (isinstance(temperature, bool) or not isinstance(temperature, (int, float))):
        raise BadRequest("invalid type for `temperature`: expected f32")
    model = req.get("model")
    if model is not None and not isinstance(model, str):
        raise BadRequest("invalid type for `model`: expected a string")
    return {"messages": msgs, "stream": bool(stream) if stream is not None else False,
            "max_tokens": DEFAULT_MAX_TOKENS if max_tokens is None else max_tokens}


def _token_ids(encoding):
    ids = getattr(encoding, "ids", encoding)
    return [int(t) for t in ids]


class ChatServer:
    """The request handling without the socket: `handle(method, url, body)` returns (status, headers, body bytes)."""

    def __init__(self, model, tokenizer):
        self.model = model
        self.tokenizer = tokenizer

    def _prefill(self, tokens) -> int:
        """`prefill` of lib.rs:8607-8622 followed by the argmax of its logits: all tokens but the last as a batch, the
        last one through the decode step."""
        if len(tokens) > 1:
            self.model.forward_prefill_batch(tokens[:-1])
        return self.model.forward_greedy(tokens[-1])

    def _decode_one(self, token):
        try:
            return self.tokenizer.decode([token], skip_special_tokens=False)
        except Exception:
            return None              # `if let Ok(text)`: a token that does not decode is skipped, and still counted

    def chat_completion(self, body: bytes):
        try:
            req = parse_chat_request(body)
        except BadRequest as e:
            return 400, {}, json.dumps({"error": "Invalid JSON: %s" % e}).encode()
        prompt = format_chat_messages(req["messages"])
        try:
            tokens = _token_ids(self.tokenizer.encode(prompt, add_special_tokens=True))
            if not tokens:
                raise ValueError("empty prompt")     # the reference indexes tokens[len - 1] and would panic here
        except Exception as e:
            return 500, {}, json.dumps({"error": "Tokenization failed: %s" % e}).encode()
        model = self.model
        # The cache holds max_seq positions and every token fed takes one: a prompt that fills it is refused up front, and
        # the decode loop stops at the last free position with finish_reason "length".  (The reference has neither check:
        # its generated binary panics on the slice index; here the model call would raise in the middle of the request.)
        max_seq = int(getattr(model, "config", {}).get("max_seq", 0) or 0)
        if max_seq and len(tokens) >= max_seq:
            return 400, {}, json.dumps({"error": "Prompt too long: %d tokens, the model's context holds %d"
                                                 % (len(tokens), max_seq)}).encode()
        room = max_seq - len(tokens) if max_seq else req["max_tokens"]      # decode steps the cache still has rows for
        finish = "stop"
        try:
            model.reset()
            if hasattr(model, "set_repeat_penalty"):
                model.set_repeat_penalty(1.0)                # the serve loop is a plain argmax
            t0 = time.perf_counter()
            next_token = self._prefill(tokens)
            prefill_s = time.perf_counter() - t0
            t0 = time.perf_counter()
            pieces, generated = [], 0
            for _ in range(req["max_tokens"]):
                if next_token == EOS_TOKEN:
                    break
                text = self._decode_one(next_token)
                if text is not None:
                    pieces.append(text)
                generated += 1
                if generated > room:                         # feeding this token would need a row past the cache's end
                    finish = "length"
                    break
                next_token = model.forward_greedy(next_token)
            gen_s = time.perf_counter() - t0
        except Exception as e:                               # a failed model call is an answer, not a dropped connection
            return 500, {}, json.dumps({"error": "Generation failed: %s" % e}).encode()
        tok_s = generated / gen_s if gen_s > 0.0 else 0.0
        if req["stream"]:
            out = []
            for text in pieces:
                chunk = {"id": "chatcmpl-1", "object": "chat.completion.chunk",
                         "choices": [{"index": 0, "delta": {"content": text}, "finish_reason": None}]}
                out.append("data: %s\n\n" % json.dumps(chunk, separators=(",", ":"), ensure_ascii=False))
            usage = ('{"prefill_tokens":%d,"prefill_time_ms":%.1f,"generation_tokens":%d,"generation_time_ms":%.1f,'
                     '"tokens_per_sec":%.1f}' % (len(tokens), prefill_s * 1e3, generated, gen_s * 1e3, tok_s))
            out.append('data: {"id":"chatcmpl-1","object":"chat.completion.chunk","choices":[{"index":0,"delta":{},'
                       '"finish_reason":"%s"}],"usage":%s}\n\ndata: [DONE]\n\n' % (finish, usage))
            return 200, {"Content-Type": "text/event-stream", "Cache-Control": "no-cache"}, "".join(out).encode("utf-8")
        resp = {"id": "chatcmpl-1", "object": "chat.completion",
                "choices": [{"index": 0, "message": {"role": "assistant", "content": "".join(pieces)}, "finish_reason": finish}],
                "usage": {"prefill_tokens": len(tokens), "prefill_time_ms": int(prefill_s * 1e3),
                          "generation_tokens": generated, "generation_time_ms": int(gen_s * 1e3), "tokens_per_sec": tok_s}}
        return 200, {"Content-Type": "application/json"}, json.dumps(resp, ensure_ascii=False).encode("utf-8")

    def handle(self, method: str, url: str, body: bytes = b""):
        if method == "POST" and url == "/v1/chat/completions":
            return self.chat_completion(body)
        if method == "GET" and url == "/v1/models":
            listing = {"object": "list", "data": [{"id": MODEL_ID, "object": "model", "owned_by": "forgellm"}]}
            return 200, {"Content-Type": "application/json"}, json.dumps(listing).encode()
        if method == "GET" and url == "/health":
            return 200, {}, b'{"status":"ok"}'
        return 404, {}, b"Not Found"


def make_http_server(model, tokenizer, port: int, host: str = "0.0.0.0") -> HTTPServer:
    """A single-threaded HTTP server around ChatServer; `serve_forever()` on it is the reference's request loop."""
    chat = ChatServer(model, tokenizer)

    class Handler(BaseHTTPRequestHandler):
        protocol_version = "HTTP/1.1"

        def _respond(self, method):
            try:
                n = int(self.headers.get("Content-Length") or 0)
            except ValueError:
                n = -1
            if n < 0 or n > MAX_BODY_BYTES:
                status, headers, payload = 413, {}, json.dumps({"error": "Request body too large"}).encode()
                self.close_connection = True                 # the unread body must not be taken for the next request
            else:
                body = self.rfile.read(n) if n > 0 else b""
                status, headers, payload = chat.handle(method, self.path, body)
            self.send_response(status)
            for k, v in headers.items():
                self.send_header(k, v)
            self.send_header("Content-Length", str(len(payload)))
            self.end_headers()
            self.wfile.write(payload)

        def do_GET(self):
            self._respond("GET")

        def do_POST(self):
            self._respond("POST")

        def do_PUT(self):
            self._respond("PUT")

        def do_DELETE(self):
            self._respond("DELETE")

        def log_message(self, fmt, *args):
            pass

    return HTTPServer((host, port), Handler)


def serve(model, tokenizer, port: int, host: str = "0.0.0.0") -> None:
    """`serve(model, tokenizer, port)` of the generated binary (lib.rs:8627-8684)."""
    import sys
    httpd = make_http_server(model, tokenizer, port, host)
    print("ForgeLLM HIP server listening on http://%s:%d" % (host, httpd.server_address[1]), file=sys.stderr)
    print("Endpoints:\n  POST /v1/chat/completions\n  GET  /v1/models\n  GET  /health", file=sys.stderr)
    try:
        httpd.serve_forever()
    finally:
        httpd.server_close()
