"""The provider's decode callbacks (volvoxai_amd/provider/decoder_route.inc) driven through the
test double of the runtime side of the SPI (tests/provider_host/mock_host.c): a decoder package
written with the reference's operator names, one prefill and N steps with the key/value cache on
the device, the host feeding the ids back -- against the CPU restatement of the decoder
(tests/_decoder_ref.py) token for token.  Without a GPU: the graph reader's verdicts."""
import ctypes as C
import json
from pathlib import Path

import numpy as np
import pytest

from test_provider import MOCK, PROVIDER, ModelSource, write_safetensors

pytestmark = pytest.mark.skipif(not (PROVIDER.exists() and MOCK.exists()),
                                reason="provider and mock host are built where the reference's headers are present")


class MockDecode(C.Structure):
    _fields_ = [("graph_path", C.c_char_p), ("weight_path", C.c_char_p), ("input_name", C.c_char_p),
                ("ids_name", C.c_char_p), ("logits_name", C.c_char_p), ("slots", C.c_int32), ("capacity", C.c_int32),
                ("vocab", C.c_int32), ("prompt_len", C.c_int32), ("steps", C.c_int32), ("token_ids", C.c_void_p),
                ("generated", C.c_void_p), ("first_logits", C.c_void_p),
                ("status", C.c_int32), ("failed_stage", C.c_int32), ("writes", C.c_int32), ("sink_mismatch", C.c_int32),
                ("wrong_step_refused", C.c_int32), ("reset_repeats", C.c_int32), ("attested", C.c_int32),
                ("message", C.c_char * 256), ("compile_route", C.c_char * 512), ("execute_route", C.c_char * 512),
                ("replayed_steps", C.c_int32), ("step_seconds", C.c_double)]


def decoder_package(tmp, cfg, weights, slots, capacity, with_logits=True, mutate=None):
    """graph.json + model.safetensors of the decoder: one node per operator, q/k/v and gate/up as
    the separate PackedLinear nodes an importer writes (rows of the fused random weights)."""
    from volvoxai_amd.decoder import pack_w8_words, rope_tables
    import dataclasses
    cos, sin = rope_tables(dataclasses.replace(cfg, max_seq=capacity))
    tensors = {"embed.weight": weights["embedding"], "rope.cos": cos, "rope.sin": sin, "norm_f.weight": weights["norm_f"]}
    nodes = []
    lead = [slots, capacity]

    def out(name, last, dtype="float32"):
        return {"out": {"tensor": name, "shape": lead + [last], "dtype": dtype}}

    def linear(node_id, lin, rows, fed, out_name):
        tensors[node_id + ".weight#as_i32"] = pack_w8_words(lin["w"][rows])
        tensors[node_id + ".scale"] = lin["scales"][rows]
        nodes.append({"id": node_id, "opType": "PackedLinear",
                      "inputs": {"input": fed, "weight": node_id + ".weight", "scale": node_id + ".scale"},
                      "outputs": out(out_name, int(lin["w"][rows].shape[0])),
                      "params": {"group_size": cfg.group, "weight_bits": 8}})

    nodes.append({"id": "embed", "opType": "Embedding", "inputs": {"input": "token_ids", "weight": "embed.weight"},
                  "outputs": out("h0", cfg.hidden), "params": {}})
    stream = "h0"
    q, kv = cfg.q_dim, cfg.kv_dim
    for i, L in enumerate(weights["layers"]):
        p = f"l{i}."
        tensors[p + "norm1.weight"], tensors[p + "norm2.weight"] = L["norm1"], L["norm2"]
        nodes.append({"id": p + "norm1", "opType": "RMSNorm", "inputs": {"input": stream, "weight": p + "norm1.weight"},
                      "outputs": out(p + "n1", cfg.hidden), "params": {"eps": cfg.eps}})
        linear(p + "q", L["qkv"], slice(0, q), p + "n1", p + "q_out")
        linear(p + "k", L["qkv"], slice(q, q + kv), p + "n1", p + "k_out")
        linear(p + "v", L["qkv"], slice(q + kv, q + 2 * kv), p + "n1", p + "v_out")
        for which, width in (("q", q), ("k", kv)):
            nodes.append({"id": p + "rope_" + which, "opType": "RoPE",
                          "inputs": {"input": p + which + "_out", "cos": "rope.cos", "sin": "rope.sin"},
                          "outputs": out(p + which + "_rot", width),
                          "params": {"head_dim": cfg.head_dim, "interleaved": False}})
        nodes.append({"id": p + "attn", "opType": "CrossSDPA",
                      "inputs": {"q": p + "q_rot", "k": p + "k_rot", "v": p + "v_out"},
                      "outputs": out(p + "att", q), "params": {"causal": True}})
        linear(p + "o", L["o"], slice(None), p + "att", p + "o_out")
        nodes.append({"id": p + "add1", "opType": "Add", "inputs": {"a": stream, "b": p + "o_out"},
                      "outputs": out(p + "h1", cfg.hidden), "params": {}})
        nodes.append({"id": p + "norm2", "opType": "RMSNorm", "inputs": {"input": p + "h1", "weight": p + "norm2.weight"},
                      "outputs": out(p + "n2", cfg.hidden), "params": {"eps": cfg.eps}})
        linear(p + "gate", L["gate_up"], slice(0, cfg.inter), p + "n2", p + "gate_out")
        linear(p + "up", L["gate_up"], slice(cfg.inter, 2 * cfg.inter), p + "n2", p + "up_out")
        nodes.append({"id": p + "silu", "opType": "SiLU", "inputs": {"input": p + "gate_out"},
                      "outputs": out(p + "gate_act", cfg.inter), "params": {}})
        nodes.append({"id": p + "mul", "opType": "Mul", "inputs": {"a": p + "gate_act", "b": p + "up_out"},
                      "outputs": out(p + "act", cfg.inter), "params": {}})
        linear(p + "down", L["down"], slice(None), p + "act", p + "down_out")
        nodes.append({"id": p + "add2", "opType": "Add", "inputs": {"a": p + "h1", "b": p + "down_out"},
                      "outputs": out(p + "h2", cfg.hidden), "params": {}})
        stream = p + "h2"
    nodes.append({"id": "norm_f", "opType": "RMSNorm", "inputs": {"input": stream, "weight": "norm_f.weight"},
                  "outputs": out("hf", cfg.hidden), "params": {"eps": cfg.eps}})
    tensors["lm_head.weight#as_i32"] = pack_w8_words(weights["lm_head"]["w"])
    tensors["lm_head.scale"] = weights["lm_head"]["scales"]
    nodes.append({"id": "lm_head", "opType": "PackedLinear",
                  "inputs": {"input": "hf", "weight": "lm_head.weight", "scale": "lm_head.scale"},
                  "outputs": {"out": {"tensor": "logits", "shape": [slots, cfg.vocab], "dtype": "float32"}},
                  "params": {"group_size": cfg.group, "weight_bits": 8}})
    nodes.append({"id": "pick", "opType": "ArgMax", "inputs": {"input": "logits"},
                  "outputs": {"out": {"tensor": "next_token_ids", "shape": [slots], "dtype": "int32"}},
                  "params": {"axis": -1}})
    graph = {"format": "volvox-graph/v1", "dimensions": {},
             "inputs": {"token_ids": {"shape": lead, "dtype": "int32"}}, "nodes": nodes,
             "outputs": ["next_token_ids"] + (["logits"] if with_logits else [])}
    if mutate:
        mutate(graph, tensors)
    tmp.mkdir(parents=True, exist_ok=True)
    (tmp / "graph.json").write_text(json.dumps(graph, separators=(",", ":")))
    write_safetensors(tmp / "model.safetensors", tensors)
    return tmp / "graph.json", tmp / "model.safetensors"


def small_config():
    from volvoxai_amd.decoder import DecoderConfig
    return DecoderConfig(layers=2, hidden=256, q_heads=4, kv_heads=2, head_dim=64, inter=384, vocab=500, group=128,
                         max_seq=32)


@pytest.fixture(scope="module")
def libs():
    import volvoxai_amd as vx
    vx.library()
    mock = C.CDLL(str(MOCK), mode=C.RTLD_GLOBAL)
    provider = C.CDLL(str(PROVIDER))
    mock.mock_host_run_decode.argtypes = [C.POINTER(MockDecode)]
    mock.mock_host_registered_name.restype = C.c_char_p
    if not mock.mock_host_registered_name():  # (tests/test_provider.py may have registered it already)
        mock.mock_host_register.argtypes = [C.c_void_p]
        assert mock.mock_host_register(C.cast(provider.volvoxai_hip_gfx950_backend_register, C.c_void_p)) == 0
    provider.volvoxai_hip_gfx950_inspect_package.argtypes = [
        C.POINTER(ModelSource), C.c_int32, C.POINTER(C.c_uint32), C.POINTER(C.c_uint32), C.POINTER(C.c_int32),
        C.c_char_p, C.c_size_t]
    return mock, provider


def inspect(provider, graph, weights, arithmetic=1):
    paths = (C.c_char_p * 1)(str(weights).encode())
    src = ModelSource(C.sizeof(ModelSource), str(graph).encode(), paths, 1, None, 0)
    msg = C.create_string_buffer(256)
    packed = C.c_int32(0)
    st = provider.volvoxai_hip_gfx950_inspect_package(C.byref(src), arithmetic, None, None, C.byref(packed), msg, 256)
    return st, msg.value.decode(), packed.value


def test_decoder_graph_is_read_and_its_deviations_refused(libs, tmp_path):
    """The graph reader without a device: the pattern is accepted; another operator order, a branch
    that does not return to the stream, interleaved rotation, another arithmetic and a missing
    tensor are refused with the node named."""
    from volvoxai_amd.decoder import init_weights
    _, provider = libs
    cfg = small_config()
    weights = init_weights(cfg, 3)
    g, w = decoder_package(tmp_path / "ok", cfg, weights, 2, 16)
    assert inspect(provider, g, w)[::2] == (0, 1)
    assert inspect(provider, g, w, arithmetic=3)[0] == -7  # F32 arithmetic is not what this route runs

    def swap(graph, tensors):
        graph["nodes"][1], graph["nodes"][2] = graph["nodes"][2], graph["nodes"][1]

    def stray_add(graph, tensors):
        next(n for n in graph["nodes"] if n["id"] == "l0.add1")["inputs"]["b"] = "l0.n1"

    def interleaved(graph, tensors):
        next(n for n in graph["nodes"] if n["id"] == "l1.rope_q")["params"]["interleaved"] = True

    def no_gain(graph, tensors):
        del tensors["l1.norm2.weight"]

    def extra_node(graph, tensors):
        graph["nodes"].insert(3, dict(graph["nodes"][3], id="again"))

    for name, mutate, status, needle in (("swap", swap, -7, "l0.q"), ("add", stray_add, -7, "l0.add1"),
                                         ("rope", interleaved, -7, "l1.rope_q"), ("gain", no_gain, -5, "l1.norm2.weight"),
                                         ("extra", extra_node, -7, "16 * layers")):
        g, w = decoder_package(tmp_path / name, cfg, weights, 2, 16, mutate=mutate)
        st, message, _ = inspect(provider, g, w)
        assert st == status and needle in message, (name, st, message)


@pytest.mark.gpu
@pytest.mark.parametrize("with_logits", [True, False])
def test_prefill_and_steps_through_the_decode_callbacks(libs, oracle, tmp_path, with_logits):
    """Prefill of a 5-token prompt and 6 steps for 3 slots through context_decode_prefill /
    context_decode_step: the ids of every step equal the CPU restatement's, the first logits agree
    to rounding noise, a step at a skipped position is refused, a reset repeats the prefill."""
    from _decoder_ref import DecoderRef
    from volvoxai_amd.decoder import init_weights, rope_tables
    mock, _ = libs
    cfg = small_config()
    weights = init_weights(cfg, 11)
    slots, capacity, prompt_len, steps = 3, cfg.max_seq, 5, 6
    prompt = np.random.default_rng(2).integers(0, cfg.vocab, (slots, prompt_len))
    want_tokens, want_logits = DecoderRef(cfg, weights, oracle, rope_tables).generate(prompt, steps + 1)
    g, w = decoder_package(tmp_path / "dec", cfg, weights, slots, capacity, with_logits=with_logits)
    ids = np.zeros((slots, capacity), np.int32)
    ids[:, :prompt_len] = prompt
    generated = np.full((steps + 1, slots), -1, np.int32)
    logits = np.zeros((slots, cfg.vocab), np.float32)
    run = MockDecode(str(g).encode(), str(w).encode(), b"token_ids", b"next_token_ids",
                     b"logits" if with_logits else None, slots, capacity, cfg.vocab, prompt_len, steps,
                     ids.ctypes.data, generated.ctypes.data, logits.ctypes.data)
    st = mock.mock_host_run_decode(C.byref(run))
    assert st == 0 and run.failed_stage == 0, (st, run.failed_stage, run.message)
    assert (generated == want_tokens).all(), (generated, want_tokens)
    assert run.wrong_step_refused == 1 and run.reset_repeats == 1 and run.attested == 1
    assert run.writes == (steps + 2) * (2 if with_logits else 1)
    assert run.replayed_steps == steps - 1   # every step after the first runs from the recording of the second
    assert b"hip.decoder.w8a8-packed-linear.layers2" in run.compile_route and b"nodes=36" in run.execute_route
    # the generated ids were fed back into the id rows behind the prompt
    assert (ids[:, prompt_len:prompt_len + steps] == want_tokens[:steps].T).all()
    if with_logits:
        scale = np.abs(want_logits[0]).max()
        assert np.abs(logits - want_logits[0]).max() <= 2e-4 * scale


@pytest.mark.gpu
@pytest.mark.parametrize("slots", [32, 1, 2])
def test_decode_callbacks_at_benchmark_widths_match_the_python_wiring(libs, tmp_path, slots):
    """Two layers at the benchmark decoder's widths (hidden 1024, 16 query / 8 KV heads of 128,
    SwiGLU 3072, vocabulary 32000), 32 slots, a 24-token prompt and 4 steps: the SPI route and
    volvoxai_amd.decoder.W8A8Decoder launch the same kernels in the same order, so their ids are
    identical (the CPU restatement pins those kernels stage by stage in tests/test_decoder.py).
    One slot: both take the fused single-row linears in their steps."""
    import torch
    from volvoxai_amd.decoder import DecoderConfig, W8A8Decoder, init_weights
    mock, _ = libs
    cfg = DecoderConfig(layers=2, max_seq=64)
    weights = init_weights(cfg, 21)
    capacity, prompt_len, steps = cfg.max_seq, 24, 4
    prompt = np.random.default_rng(4).integers(0, cfg.vocab, (slots, prompt_len))
    dec = W8A8Decoder(cfg, weights, slots)
    assert dec.rows_fused == (slots == 1)
    first = dec.prefill(torch.from_numpy(prompt).cuda()).cpu().numpy()
    want = dec.decode(steps).cpu().numpy()
    dec.close()
    assert (want[0] == first).all()
    g, w = decoder_package(tmp_path / "dec", cfg, weights, slots, capacity, with_logits=False)
    ids = np.zeros((slots, capacity), np.int32)
    ids[:, :prompt_len] = prompt
    generated = np.full((steps + 1, slots), -1, np.int32)
    run = MockDecode(str(g).encode(), str(w).encode(), b"token_ids", b"next_token_ids", None, slots, capacity, cfg.vocab,
                     prompt_len, steps, ids.ctypes.data, generated.ctypes.data, None)
    st = mock.mock_host_run_decode(C.byref(run))
    assert st == 0 and run.failed_stage == 0, (st, run.failed_stage, run.message)
    assert (generated == want).all()
    assert run.wrong_step_refused == 1 and run.reset_repeats == 1 and run.attested == 1
    # the first step is launched plainly, the second is recorded and run from the recording, like every later one
    assert run.replayed_steps == steps - 1


@pytest.mark.gpu
def test_one_slot_with_a_linear_the_fused_form_declines(libs, tmp_path, monkeypatch):
    """One slot, hidden 1024 (which the fused single-row forms take) and a SwiGLU width above what they
    take (the down projection would decline after the stream had been updated in place): the route is
    decided over every linear up front, so the steps run the separate launches and succeed, with the
    ids of the Python wiring -- also with the recording switched off."""
    import torch
    from volvoxai_amd.decoder import DecoderConfig, W8A8Decoder, init_weights
    mock, _ = libs
    cfg = DecoderConfig(layers=2, hidden=1024, q_heads=8, kv_heads=4, head_dim=128, inter=8448, vocab=640, max_seq=48)
    weights = init_weights(cfg, 31)
    slots, capacity, prompt_len, steps = 1, cfg.max_seq, 9, 5
    prompt = np.random.default_rng(5).integers(0, cfg.vocab, (slots, prompt_len))
    dec = W8A8Decoder(cfg, weights, slots)
    assert not dec.rows_fused
    first = dec.prefill(torch.from_numpy(prompt).cuda()).cpu().numpy()
    want = dec.decode(steps).cpu().numpy()
    dec.close()
    g, w = decoder_package(tmp_path / "dec", cfg, weights, slots, capacity, with_logits=False)
    for no_replay in (False, True):
        if no_replay:
            monkeypatch.setenv("VXHIP_PROVIDER_NO_REPLAY", "1")
        ids = np.zeros((slots, capacity), np.int32)
        ids[:, :prompt_len] = prompt
        generated = np.full((steps + 1, slots), -1, np.int32)
        run = MockDecode(str(g).encode(), str(w).encode(), b"token_ids", b"next_token_ids", None, slots, capacity, cfg.vocab,
                         prompt_len, steps, ids.ctypes.data, generated.ctypes.data, None)
        st = mock.mock_host_run_decode(C.byref(run))
        assert st == 0 and run.failed_stage == 0, (st, run.failed_stage, run.message)
        assert (generated[0] == first).all() and (generated == want).all()
        assert run.replayed_steps == (0 if no_replay else steps - 1)
