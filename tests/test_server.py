"""OpenAI API server on the CPU engine: the reference smoke test's contract
(llm-d-test.yaml:32-78: GET /v1/models contains the model id; POST /v1/completions with
{"model", "prompt"} and no max_tokens), plus chat, streaming, errors and /metrics."""
import json

import pytest
from fastapi.testclient import TestClient

from aws_k8s_ansible_provisioner_amd.engine.config import EngineConfig
from aws_k8s_ansible_provisioner_amd.server.api_server import build_app

MODEL = "Qwen/Qwen3-0.6B"


@pytest.fixture(scope="module")
def client():
    ecfg = EngineConfig(model="tiny-qwen3", served_model_name=MODEL, device="cpu",
                        max_model_len=256, max_num_seqs=8, max_num_batched_tokens=64,
                        block_size=32, num_gpu_blocks=128, chat_template="default")
    app, ae = build_app(ecfg)
    with TestClient(app) as c:
        yield c


def test_models_lists_served_model(client):
    r = client.get("/v1/models")
    assert r.status_code == 200
    assert MODEL in r.text
    assert r.json()["data"][0]["id"] == MODEL


def test_reference_smoke_completion(client):
    r = client.post("/v1/completions", json={"model": MODEL, "prompt": "Who are you?"})
    assert r.status_code == 200, r.text
    j = r.json()
    assert j["object"] == "text_completion" and j["model"] == MODEL
    assert j["usage"]["completion_tokens"] <= 16 and j["usage"]["prompt_tokens"] == 12
    assert j["choices"][0]["finish_reason"] in ("length", "stop")


def test_batch_prompts_token_ids_and_n(client):
    r = client.post("/v1/completions", json={"prompt": [[5, 6, 7], [8, 9]], "max_tokens": 4,
                                             "temperature": 0, "n": 2, "ignore_eos": True})
    j = r.json()
    assert len(j["choices"]) == 4
    assert all(c["finish_reason"] == "length" for c in j["choices"])
    assert j["usage"]["completion_tokens"] == 16
    # greedy: both samples of a prompt agree
    assert j["choices"][0]["text"] == j["choices"][1]["text"]


def test_streaming_completion_sse(client):
    with client.stream("POST", "/v1/completions",
                       json={"prompt": "abc", "max_tokens": 5, "temperature": 0, "stream": True,
                             "ignore_eos": True,
                             "stream_options": {"include_usage": True}}) as r:
        lines = [l for l in r.iter_lines() if l.startswith("data: ")]
    assert lines[-1] == "data: [DONE]"
    chunks = [json.loads(l[6:]) for l in lines[:-1]]
    assert chunks[-1]["usage"]["completion_tokens"] == 5
    fins = [c["choices"][0]["finish_reason"] for c in chunks if c["choices"]]
    assert fins[-1] == "length" and fins.count("length") == 1


def test_streaming_multiple_prompts_and_n(client):
    """stream with two prompts x n=2: four choice indices interleave in one SSE stream, each
    ends once, their texts equal the non-streaming response, usage sums every choice."""
    body = {"prompt": [[5, 6, 7], [8, 9]], "max_tokens": 4, "temperature": 0, "n": 2,
            "ignore_eos": True}
    ref = client.post("/v1/completions", json=body).json()["choices"]
    with client.stream("POST", "/v1/completions",
                       json=dict(body, stream=True,
                                 stream_options={"include_usage": True})) as r:
        lines = [l for l in r.iter_lines() if l.startswith("data: ")]
    assert lines[-1] == "data: [DONE]"
    chunks = [json.loads(l[6:]) for l in lines[:-1]]
    text, fins = {}, {}
    for c in chunks:
        for ch in c["choices"]:
            text[ch["index"]] = text.get(ch["index"], "") + ch["text"]
            if ch["finish_reason"]:
                fins[ch["index"]] = fins.get(ch["index"], 0) + 1
    assert sorted(text) == [0, 1, 2, 3] and fins == {0: 1, 1: 1, 2: 1, 3: 1}
    assert [text[k] for k in range(4)] == [c["text"] for c in ref]
    assert chunks[-1]["usage"]["completion_tokens"] == 16
    assert chunks[-1]["usage"]["prompt_tokens"] == 5
    msgs = [{"role": "user", "content": "hi"}]
    with client.stream("POST", "/v1/chat/completions",
                       json={"messages": msgs, "max_tokens": 3, "stream": True, "n": 3,
                             "temperature": 0, "ignore_eos": True}) as r:
        lines = [l for l in r.iter_lines() if l.startswith("data: ")]
    idx = {ch["index"] for l in lines[:-1] for ch in json.loads(l[6:])["choices"]}
    assert idx == {0, 1, 2}


def test_chat_completion_and_stream(client):
    msgs = [{"role": "system", "content": "be brief"}, {"role": "user", "content": "hi"}]
    r = client.post("/v1/chat/completions", json={"model": MODEL, "messages": msgs,
                                                  "max_tokens": 6, "temperature": 0})
    j = r.json()
    assert j["object"] == "chat.completion"
    assert j["choices"][0]["message"]["role"] == "assistant"
    with client.stream("POST", "/v1/chat/completions",
                       json={"messages": msgs, "max_tokens": 3, "stream": True,
                             "temperature": 0, "ignore_eos": True}) as r:
        lines = [l for l in r.iter_lines() if l.startswith("data: ")]
    first = json.loads(lines[0][6:])
    assert first["choices"][0]["delta"]["role"] == "assistant"
    assert lines[-1] == "data: [DONE]"


def test_chat_template_override_and_tokenize(client):
    msgs = [{"role": "user", "content": "Hi"}]
    r = client.post("/tokenize", json={"messages": msgs})
    assert r.json()["count"] == len("User: Hi\n\nAssistant:")
    r = client.post("/v1/chat/completions", json={"messages": msgs, "chat_template": "phi",
                                                  "max_tokens": 2})
    assert r.status_code == 200


def test_errors(client):
    assert client.post("/v1/completions", json={"model": "nope", "prompt": "x"}).status_code == 404
    assert client.post("/v1/completions", json={"prompt": {"bad": 1}}).status_code == 400
    assert client.post("/v1/chat/completions", json={"messages": []}).status_code == 400
    too_long = list(range(5, 400))
    assert client.post("/v1/completions", json={"prompt": too_long}).status_code == 400


def test_health_and_metrics(client):
    assert client.get("/health").json()["status"] == "ok"
    m = client.get("/metrics").text
    for name in ["vllm:num_requests_running", "vllm:prompt_tokens_total",
                 "vllm:generation_tokens_total", "vllm:time_to_first_token_seconds_bucket",
                 "vllm:gpu_cache_usage_perc", "vllm_request_total", "vllm_active_requests",
                 "vllm_request_duration_seconds_bucket"]:
        assert name in m, name


def test_logprobs_and_penalties_in_api(client):
    r = client.post("/v1/completions", json={"model": MODEL, "prompt": "hello there",
                                             "max_tokens": 5, "logprobs": 1, "ignore_eos": True,
                                             "temperature": 0})
    assert r.status_code == 200, r.text
    lp = r.json()["choices"][0]["logprobs"]
    assert len(lp["tokens"]) == len(lp["token_logprobs"]) == 5
    assert all(x <= 1e-6 for x in lp["token_logprobs"])
    r = client.post("/v1/chat/completions", json={
        "messages": [{"role": "user", "content": "hi"}], "max_tokens": 4, "logprobs": True,
        "ignore_eos": True, "presence_penalty": 1.5, "frequency_penalty": 0.5,
        "repetition_penalty": 1.2})
    assert r.status_code == 200, r.text
    content = r.json()["choices"][0]["logprobs"]["content"]
    assert len(content) == 4 and all("logprob" in c for c in content)
    # top-N alternatives (completions: logprobs=N, chat: top_logprobs=N)
    r = client.post("/v1/completions", json={"model": MODEL, "prompt": "hello there",
                                             "max_tokens": 3, "logprobs": 3, "ignore_eos": True,
                                             "temperature": 0})
    tops = r.json()["choices"][0]["logprobs"]["top_logprobs"]
    assert len(tops) == 3 and all(1 <= len(t) <= 3 for t in tops)
    r = client.post("/v1/chat/completions", json={
        "messages": [{"role": "user", "content": "hi"}], "max_tokens": 2, "logprobs": True,
        "top_logprobs": 5, "ignore_eos": True, "temperature": 0})
    content = r.json()["choices"][0]["logprobs"]["content"]
    assert all(len(c["top_logprobs"]) == 5 for c in content)
    assert all(c["top_logprobs"][0]["logprob"] >= c["top_logprobs"][-1]["logprob"]
               for c in content)


def test_prefix_cache_and_queue_time_metrics_are_live():
    """vllm:prefix_cache_{hits,queries}_total (tokens) and vllm:request_queue_time_seconds
    are fed by the engine (they read 0 forever in round 1)."""
    from fastapi.testclient import TestClient

    from aws_k8s_ansible_provisioner_amd.engine.config import EngineConfig
    from aws_k8s_ansible_provisioner_amd.server.api_server import build_app

    app, ae = build_app(EngineConfig(model="tiny-qwen3", served_model_name="m", device="cpu",
                                     max_model_len=256, max_num_seqs=4,
                                     max_num_batched_tokens=64, block_size=32,
                                     num_gpu_blocks=64))
    prompt = list(range(10, 110))
    with TestClient(app) as c:
        for _ in range(2):
            r = c.post("/v1/completions", json={"prompt": prompt, "max_tokens": 2})
            assert r.status_code == 200
        text = c.get("/metrics").text
    vals = {}
    for ln in text.splitlines():
        if ln and not ln.startswith("#"):
            k, v = ln.rsplit(" ", 1)
            vals[k.split("{")[0]] = vals.get(k.split("{")[0], 0.0) + float(v)
    assert vals["vllm:prefix_cache_queries_total"] >= 2 * 99
    assert vals["vllm:prefix_cache_hits_total"] >= 96  # 3 full 32-token blocks reused
    assert vals["vllm:request_queue_time_seconds_count"] == 2


def test_bidetar_served_with_prefix_cache_and_sampling():
    """The layered fp32-stream design behind the same OpenAI endpoints: greedy completions are
    reproducible, a repeated prompt reuses its cached pages (every layer run keeps its K / V
    under the same page ids) and returns the same tokens, sampled requests run too."""
    from fastapi.testclient import TestClient

    from aws_k8s_ansible_provisioner_amd.engine.config import EngineConfig
    from aws_k8s_ansible_provisioner_amd.server.api_server import build_app

    app, ae = build_app(EngineConfig(model="tiny-bidetar", served_model_name="b", device="cpu",
                                     dtype="float32", max_model_len=256, max_num_seqs=4,
                                     max_num_batched_tokens=48, block_size=32,
                                     num_gpu_blocks=64))
    prompt = list(range(10, 110))
    with TestClient(app) as c:
        outs = []
        for _ in range(2):
            r = c.post("/v1/completions", json={"prompt": prompt, "max_tokens": 6,
                                                "temperature": 0.0})
            assert r.status_code == 200, r.text
            outs.append(r.json()["choices"][0]["text"])
        assert outs[0] == outs[1]
        r = c.post("/v1/completions", json={"prompt": prompt[:50], "max_tokens": 5,
                                            "temperature": 0.8, "top_p": 0.9, "seed": 3})
        assert r.status_code == 200 and r.json()["usage"]["completion_tokens"] == 5
        text = c.get("/metrics").text
    hits = sum(float(ln.rsplit(" ", 1)[1]) for ln in text.splitlines()
               if ln.startswith("vllm:prefix_cache_hits_total"))
    assert hits >= 96  # the second request reused 3 full pages of the first


def test_puputar_served_with_sampling_and_no_prefix_cache():
    """The latent-attention design with per-sequence shift state behind the same OpenAI
    endpoints: greedy completions are reproducible although the repeated prompt may NOT reuse
    cached pages (a cached prefix does not hold the shift state at its end, so the engine
    turns prefix caching off for this model), concurrent prompts share the slot pool, sampled
    requests run too."""
    from aws_k8s_ansible_provisioner_amd.engine.config import EngineConfig
    from aws_k8s_ansible_provisioner_amd.server.api_server import build_app

    app, ae = build_app(EngineConfig(model="tiny-puputar", served_model_name="p", device="cpu",
                                     dtype="float32", max_model_len=256, max_num_seqs=2,
                                     max_num_batched_tokens=48, block_size=32,
                                     num_gpu_blocks=64, enable_prefix_caching=True))
    prompt = list(range(10, 110))
    with TestClient(app) as c:
        outs = []
        for _ in range(2):
            r = c.post("/v1/completions", json={"prompt": prompt, "max_tokens": 6,
                                                "temperature": 0.0})
            assert r.status_code == 200, r.text
            outs.append(r.json()["choices"][0]["text"])
        assert outs[0] == outs[1]
        # more prompts than sequence slots in one request: slots are handed on
        r = c.post("/v1/completions", json={"prompt": [prompt[:20], prompt[:33], prompt[:7]],
                                            "max_tokens": 4, "temperature": 0.0})
        assert r.status_code == 200 and len(r.json()["choices"]) == 3
        r = c.post("/v1/completions", json={"prompt": prompt[:50], "max_tokens": 5,
                                            "temperature": 0.8, "top_p": 0.9, "seed": 3})
        assert r.status_code == 200 and r.json()["usage"]["completion_tokens"] == 5
        text = c.get("/metrics").text
    hits = sum(float(ln.rsplit(" ", 1)[1]) for ln in text.splitlines()
               if ln.startswith("vllm:prefix_cache_hits_total"))
    assert hits == 0


def test_sazepel_served_with_sampling_and_no_prefix_cache():
    """The retention design behind the same OpenAI endpoints: its recurrent states live in the
    scheduler's sequence slots, so a repeated prompt must give the same greedy completion
    WITHOUT reusing cached pages (a cached prefix holds keys, not the retention state at its
    end), more prompts than slots are served by handing slots on (each new owner starts from a
    zero state), and sampled requests run."""
    from aws_k8s_ansible_provisioner_amd.engine.config import EngineConfig
    from aws_k8s_ansible_provisioner_amd.server.api_server import build_app

    app, ae = build_app(EngineConfig(model="tiny-sazepel", served_model_name="s", device="cpu",
                                     dtype="float32", max_model_len=256, max_num_seqs=2,
                                     max_num_batched_tokens=48, block_size=32,
                                     num_gpu_blocks=64, enable_prefix_caching=True))
    prompt = list(range(10, 110))
    with TestClient(app) as c:
        outs = []
        for _ in range(2):
            r = c.post("/v1/completions", json={"prompt": prompt, "max_tokens": 6,
                                                "temperature": 0.0})
            assert r.status_code == 200, r.text
            outs.append(r.json()["choices"][0]["text"])
        assert outs[0] == outs[1]
        r = c.post("/v1/completions", json={"prompt": [prompt[:20], prompt[:33], prompt[:7]],
                                            "max_tokens": 4, "temperature": 0.0})
        assert r.status_code == 200 and len(r.json()["choices"]) == 3
        # the same three alone give the same text: a handed-on slot carries nothing over
        alone = [c.post("/v1/completions", json={"prompt": p, "max_tokens": 4,
                                                 "temperature": 0.0}).json()["choices"][0]["text"]
                 for p in (prompt[:20], prompt[:33], prompt[:7])]
        assert [ch["text"] for ch in sorted(r.json()["choices"], key=lambda ch: ch["index"])] == alone
        r = c.post("/v1/completions", json={"prompt": prompt[:50], "max_tokens": 5,
                                            "temperature": 0.8, "top_p": 0.9, "seed": 3})
        assert r.status_code == 200 and r.json()["usage"]["completion_tokens"] == 5
        text = c.get("/metrics").text
    hits = sum(float(ln.rsplit(" ", 1)[1]) for ln in text.splitlines()
               if ln.startswith("vllm:prefix_cache_hits_total"))
    assert hits == 0


def test_mudepel_served_with_sampling_and_no_prefix_cache():
    """The multi-stream design behind the same OpenAI endpoints: convolution inputs and
    state-space states live in the scheduler's sequence slots, so a repeated prompt must give
    the same greedy completion WITHOUT reusing cached pages, more prompts than slots are served
    by handing slots on (each new owner starts from zeros), and sampled requests run."""
    from aws_k8s_ansible_provisioner_amd.engine.config import EngineConfig
    from aws_k8s_ansible_provisioner_amd.server.api_server import build_app

    app, ae = build_app(EngineConfig(model="tiny-mudepel", served_model_name="m", device="cpu",
                                     dtype="float32", max_model_len=256, max_num_seqs=2,
                                     max_num_batched_tokens=48, block_size=32,
                                     num_gpu_blocks=64, enable_prefix_caching=True))
    prompt = list(range(10, 110))
    with TestClient(app) as c:
        outs = []
        for _ in range(2):
            r = c.post("/v1/completions", json={"prompt": prompt, "max_tokens": 6,
                                                "temperature": 0.0})
            assert r.status_code == 200, r.text
            outs.append(r.json()["choices"][0]["text"])
        assert outs[0] == outs[1]
        r = c.post("/v1/completions", json={"prompt": [prompt[:20], prompt[:33], prompt[:7]],
                                            "max_tokens": 4, "temperature": 0.0})
        assert r.status_code == 200 and len(r.json()["choices"]) == 3
        alone = [c.post("/v1/completions", json={"prompt": p, "max_tokens": 4,
                                                 "temperature": 0.0}).json()["choices"][0]["text"]
                 for p in (prompt[:20], prompt[:33], prompt[:7])]
        assert [ch["text"] for ch in sorted(r.json()["choices"], key=lambda ch: ch["index"])] == alone
        r = c.post("/v1/completions", json={"prompt": prompt[:50], "max_tokens": 5,
                                            "temperature": 0.8, "top_p": 0.9, "seed": 3})
        assert r.status_code == 200 and r.json()["usage"]["completion_tokens"] == 5
        text = c.get("/metrics").text
    hits = sum(float(ln.rsplit(" ", 1)[1]) for ln in text.splitlines()
               if ln.startswith("vllm:prefix_cache_hits_total"))
    assert hits == 0
