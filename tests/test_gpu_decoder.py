"""The decode loop over a synthetic llama-style GGUF file: loader -> resident weights -> per-token projections.

Checks: logits against a CPU restatement (oracle dequantizer, float64 mat-vecs, the oracle's FP32 row operations) within
the mat-vec bar; the fused loop, the one-launch-per-operation loop and the graph replay agree bit for bit; launch
counts; greedy generation and its timing record; the loader's directory checks.
"""
import struct

import numpy as np
import pytest

import oracle
from gguf_writer import write_gguf
from nntrain_amd import (GGML_Q4_K, GGML_Q5_K, GGML_Q6_K, GGML_Q8_0, GgufReader, HipExecutionLane, InvalidDataError,
                         NotSupportedError, synth)
from nntrain_amd.decoder import DecoderDescriptor, QuantizedDecoder

pytestmark = pytest.mark.gpu

LAYERS, EMB, FFN, HEADS, KV, HW, VOCAB, EPS = 2, 256, 512, 4, 2, 64, 320, 1e-5


@pytest.fixture(scope="module")
def lane():
    with HipExecutionLane(0) as ln:
        yield ln


def _kv(key, value):
    if isinstance(value, str):
        b = value.encode()
        return key, 8, struct.pack("<Q", len(b)) + b
    if isinstance(value, float):
        return key, 6, struct.pack("<f", value)
    return key, 4, struct.pack("<I", value)


def _model(tmp_path, name, qkv_types=(GGML_Q4_K,) * 3, tied=False, extra=None, drop=None):
    rng = np.random.default_rng(3)
    tensors, host = [], {}

    def mat(tname, typ, out_w, in_w, seed):
        raw = synth.matrix(typ, out_w, in_w, seed)
        host[tname] = (typ, raw, out_w, in_w)
        tensors.append((tname, (in_w, out_w), typ, raw.tobytes()))

    def vec(tname, width):
        v = rng.uniform(0.5, 1.5, width).astype(np.float32)
        host[tname] = v
        tensors.append((tname, (width,), 0, v.tobytes()))

    mat("token_embd.weight", GGML_Q8_0, VOCAB, EMB, 1)
    for i in range(LAYERS):
        p = f"blk.{i}."
        vec(p + "attn_norm.weight", EMB)
        mat(p + "attn_q.weight", qkv_types[0], HEADS * HW, EMB, 10 + i)
        mat(p + "attn_k.weight", qkv_types[1], KV * HW, EMB, 20 + i)
        mat(p + "attn_v.weight", qkv_types[2], KV * HW, EMB, 30 + i)
        mat(p + "attn_output.weight", GGML_Q6_K, EMB, HEADS * HW, 40 + i)
        vec(p + "ffn_norm.weight", EMB)
        mat(p + "ffn_gate.weight", GGML_Q5_K, FFN, EMB, 50 + i)
        mat(p + "ffn_up.weight", GGML_Q5_K, FFN, EMB, 60 + i)
        mat(p + "ffn_down.weight", GGML_Q8_0, EMB, FFN, 70 + i)
    vec("output_norm.weight", EMB)
    if not tied:
        mat("output.weight", GGML_Q6_K, VOCAB, EMB, 2)
    if extra:
        tensors.append(extra)
    if drop:
        tensors = [t for t in tensors if t[0] != drop]
    kvs = [_kv("general.architecture", "llama"), _kv("llama.block_count", LAYERS), _kv("llama.embedding_length", EMB),
           _kv("llama.feed_forward_length", FFN), _kv("llama.attention.head_count", HEADS),
           _kv("llama.attention.head_count_kv", KV), _kv("llama.attention.key_length", HW),
           _kv("llama.attention.layer_norm_rms_epsilon", EPS)]
    return write_gguf(tmp_path / name, tensors, kvs), host


def _cpu_logits(host, token, tied=False, trace=None):
    def w(name):
        typ, raw, out_w, in_w = host[name]
        return oracle.dequantize(typ, raw).reshape(out_w, in_w).astype(np.float64)

    def mv(name, x):
        return (w(name) @ x.astype(np.float64)).astype(np.float32)

    hidden = w("token_embd.weight")[token].astype(np.float32)
    for i in range(LAYERS):
        p = f"blk.{i}."
        n = oracle.rms_norm(hidden, host[p + "attn_norm.weight"], 1, EMB, EPS).ravel()
        v = mv(p + "attn_v.weight", n).reshape(KV, HW)
        if trace is not None:           # (the last layer's projections stay: the loop's q|k|v buffer holds them afterwards)
            trace["qkv"] = np.concatenate([mv(p + "attn_q.weight", n), mv(p + "attn_k.weight", n), v.ravel()])
        ctx = np.repeat(v, HEADS // KV, axis=0).ravel()
        attn = mv(p + "attn_output.weight", ctx)
        hidden, m = oracle.add_rms_norm(hidden, attn, host[p + "ffn_norm.weight"], 1, EMB, EPS)
        act = oracle.silu_multiply(mv(p + "ffn_gate.weight", m.ravel()), mv(p + "ffn_up.weight", m.ravel()))
        hidden = hidden + mv(p + "ffn_down.weight", act)
    n = oracle.rms_norm(hidden, host["output_norm.weight"], 1, EMB, EPS).ravel()
    return mv("token_embd.weight" if tied else "output.weight", n)


def test_logits_match_the_cpu_restatement_and_all_three_loops_agree_bitwise(lane, tmp_path):
    path, host = _model(tmp_path, "m.gguf")
    with GgufReader(path) as reader:
        d = DecoderDescriptor.inspect(reader)
        assert (d.layer_count, d.embedding_length, d.feed_forward_length, d.head_count, d.kv_head_count, d.head_width,
                d.vocabulary) == (LAYERS, EMB, FFN, HEADS, KV, HW, VOCAB)
        with QuantizedDecoder(lane, reader, fused=True) as fused, QuantizedDecoder(lane, reader, fused=False) as plain:
            for token in (0, 7, VOCAB - 1):
                before = lane.counters()
                got = lane.read(fused.forward_token(token), count=VOCAB)
                mid = lane.counters()
                ref = lane.read(plain.forward_token(token), count=VOCAB)
                after = lane.counters()
                # launches: embedding + 4 per layer + head, against embedding + 12 per layer + 2
                assert mid["kernel_launches"] - before["kernel_launches"] == 1 + 4 * LAYERS + 1
                assert after["kernel_launches"] - mid["kernel_launches"] == 1 + 12 * LAYERS + 2
                assert mid["h2d_bytes"] == before["h2d_bytes"] and mid["allocated_bytes"] == before["allocated_bytes"]
                assert np.array_equal(got.view(np.uint32), ref.view(np.uint32))
                trace = {}
                want = _cpu_logits(host, token, trace=trace)
                assert oracle.rel_l2(got, want) <= 1e-5
                assert int(np.argmax(got)) == int(np.argmax(want))
                # the query and key projections feed nothing in a first-token pass (attention over one position returns
                # the values), so the logits do not cover them: the last layer's q | k | v against the CPU, piece by piece
                for dec in (fused, plain):
                    qkv = lane.read(dec._qkv, count=(HEADS + 2 * KV) * HW)
                    for lo, hi in ((0, HEADS * HW), (HEADS * HW, (HEADS + KV) * HW), ((HEADS + KV) * HW, (HEADS + 2 * KV) * HW)):
                        assert oracle.rel_l2(qkv[lo:hi], trace["qkv"][lo:hi]) <= 1e-5, (dec is fused, lo)
            # graph replay of the layers and the head
            eager = [lane.read(fused.forward_token(t), count=VOCAB) for t in (3, 11, 5)]
            fused.capture_graph()
            for rep in range(2):
                for t, e in zip((3, 11, 5), eager):
                    lane.synchronize()
                    assert np.array_equal(lane.read(fused.forward_token(t), count=VOCAB).view(np.uint32), e.view(np.uint32))
            with pytest.raises(IndexError):
                fused.forward_token(VOCAB)


def test_mixed_projection_types_and_tied_head(lane, tmp_path):
    path, host = _model(tmp_path, "mixed.gguf", qkv_types=(GGML_Q4_K, GGML_Q5_K, GGML_Q6_K), tied=True)
    with GgufReader(path) as reader, QuantizedDecoder(lane, reader, fused=True) as dec:
        assert dec.layers[0].qkv is None and dec.layers[0].gate_up is not None and dec.output is dec.embedding
        got = lane.read(dec.forward_token(9), count=VOCAB)
        assert oracle.rel_l2(got, _cpu_logits(host, 9, tied=True)) <= 1e-5


def test_generation_and_timing_record(lane, tmp_path):
    path, host = _model(tmp_path, "g.gguf")
    with GgufReader(path) as reader, QuantizedDecoder(lane, reader) as dec:
        seen = []
        tokens, timing = dec.generate(5, 4, on_token=seen.append)
        want, t = [], 5
        for _ in range(4):
            t = int(np.argmax(_cpu_logits(host, t)))
            want.append(t)
        assert tokens == want == seen
        assert timing.generated_tokens == 4 and timing.first_token_milliseconds > 0
        assert timing.total_milliseconds >= timing.first_token_milliseconds
        assert timing.decode_tokens_per_second is None or timing.decode_tokens_per_second > 0
        _, none = dec.generate(5, 0)
        assert (none.generated_tokens, none.first_token_milliseconds, none.decode_tokens_per_second) == (0, None, None)
        lane.collect_kernel_events = True
        dec.forward_token(1)
        lane.synchronize()
        lane.collect_kernel_events = False
        assert set(lane.kernel_timings) == {"dequantize", "quant_matvec_fused"}
        assert abs(sum(lane.kernel_timings.values()) - lane.kernel_milliseconds) < 1e-6 and lane.kernel_milliseconds > 0
        lane.reset_profile()
        assert lane.kernel_milliseconds == 0.0 and not lane.kernel_timings


def test_directory_checks(lane, tmp_path):
    path, _ = _model(tmp_path, "missing.gguf", drop="blk.1.ffn_up.weight")
    with GgufReader(path) as reader, pytest.raises(InvalidDataError, match="blk.1.ffn_up.weight"):
        QuantizedDecoder(lane, reader)
    path, _ = _model(tmp_path, "extra.gguf", extra=("blk.0.surprise", (4,), 0, b"\0" * 16))
    with GgufReader(path) as reader, pytest.raises(NotSupportedError, match="surprise"):
        QuantizedDecoder(lane, reader)
    before = lane.counters()["allocated_bytes"]
    path, _ = _model(tmp_path, "ok.gguf")
    with GgufReader(path) as reader:
        QuantizedDecoder(lane, reader).dispose()
    assert lane.counters()["allocated_bytes"] == before           # everything the decoder allocated was returned
