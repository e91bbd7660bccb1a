"""A decode loop over a GGUF file's quantized projections, shaped like the reference's per-token path.

The reference's ForwardTokenDevice (NNtrain.Core/Modules/Qwen35QuantizedModel.cs:451-513) walks the layers as
    n = RMSNorm(hidden) -> attention(n) -> hidden += attention; m = RMSNorm(hidden) ->
    hidden += W_down(SiLU(W_gate m) * W_up m)                                  -> ... -> logits = W_out RMSNorm(hidden)
with one launch per operation.  This module runs the same sequence of projections from a llama-style GGUF file
(token_embd, blk.N.attn_norm / attn_q / attn_k / attn_v / attn_output / ffn_norm / ffn_gate / ffn_up / ffn_down,
output_norm, output) on one lane, either that way (`fused=False`) or with the launches this library fuses
(`fused=True`: q|k|v and gate|up stacked, the norms and the SiLU product folded into the projections that consume them,
the residual adds folded into the o and down projections, the value heads read by the o projection itself, SiLU(gate) * up
left by the stacked gate|up projection): four launches per layer instead of twelve, same bits.

What is NOT here: the attention core and the key/value cache (outside the quantized-linear path).  Every token is
decoded as the first token of its own sequence, where causal attention is exact without a cache: the single key has
softmax weight 1, so each query head receives its group's value head (qwen35_gpu.first_token_attention).  All the
projections of a real decode step run, with their real shapes, which is what the per-token timing is about.

Timing follows QwenGgufCommand.WriteGeneration (NNtrain.Cli/QwenGgufCommand.cs:119-157): first-token latency and the
decode rate over the tokens after the first.
"""
from __future__ import annotations

import time
from dataclasses import dataclass

import numpy as np

from . import qwen35_gpu
from .gguf import GgufReader, InvalidDataError
from .lane import HipBuffer, HipExecutionLane
from .loader import GgufTensorDirectory, HipGgufLoader, NotSupportedError
from .native import POST_SILU_PAIR
from .quantized_matrix import PRE_RMS_NORM, PRE_SILU_MULTIPLY, HipQuantizedMatrix


@dataclass(frozen=True)
class DecoderDescriptor:
    """The metadata a llama-style GGUF file gives for this loop (Qwen35Gguf.Inspect keeps the same fields,
    NNtrain.Core/Serialization/Qwen35Gguf.cs:40-108)."""
    architecture: str
    layer_count: int
    embedding_length: int
    feed_forward_length: int
    head_count: int
    kv_head_count: int
    head_width: int
    rms_epsilon: float
    vocabulary: int

    @staticmethod
    def inspect(reader: GgufReader) -> "DecoderDescriptor":
        md = reader.metadata
        arch = md.get("general.architecture")
        if not isinstance(arch, str) or not arch:
            raise InvalidDataError("GGUF metadata 'general.architecture' is missing.")

        def need(key: str, kind=int):
            value = md.get(f"{arch}.{key}")
            if value is None or isinstance(value, (str, list)):
                raise InvalidDataError(f"GGUF metadata '{arch}.{key}' is missing.")
            return kind(value)

        emb, heads = need("embedding_length"), need("attention.head_count")
        kv = md.get(f"{arch}.attention.head_count_kv")
        kv = heads if kv is None else int(kv)
        head_width = md.get(f"{arch}.attention.key_length")
        head_width = emb // heads if head_width is None else int(head_width)
        token = reader.get_tensor("token_embd.weight")
        if len(token.shape) != 2:
            raise InvalidDataError("GGUF tensor 'token_embd.weight' is not a matrix.")
        d = DecoderDescriptor(arch, need("block_count"), emb, need("feed_forward_length"), heads, kv, head_width,
                              need("attention.layer_norm_rms_epsilon", float), int(token.shape[1]))
        if min(d.layer_count, d.embedding_length, d.feed_forward_length, d.head_count, d.kv_head_count, d.head_width) <= 0:
            raise InvalidDataError("GGUF decoder dimensions must be positive.")
        if d.head_count % d.kv_head_count != 0:
            raise InvalidDataError("attention.head_count must be a multiple of attention.head_count_kv.")
        if not np.isfinite(d.rms_epsilon) or d.rms_epsilon < 0:
            raise InvalidDataError("attention.layer_norm_rms_epsilon must be finite and not negative.")
        return d


@dataclass
class GenerationTiming:
    """QwenGgufCommand.GenerationTiming (QwenGgufCommand.cs:165-169)."""
    generated_tokens: int
    total_milliseconds: float
    first_token_milliseconds: float | None
    decode_tokens_per_second: float | None


class _Layer:
    __slots__ = ("attn_norm", "ffn_norm", "q", "k", "v", "o", "gate", "up", "down", "qkv", "gate_up")


class QuantizedDecoder:
    """Weights of one GGUF file resident on one lane, and the per-token loop over them."""

    def __init__(self, lane: HipExecutionLane, reader: GgufReader, fused: bool = True, chunk_bytes: int = 64 << 20):
        descriptor = DecoderDescriptor.inspect(reader)
        directory = GgufTensorDirectory(reader)
        loader = HipGgufLoader(lane, reader, chunk_bytes)
        self._build(lane, descriptor, fused,
                    matrix=lambda name, in_w, out_w: loader.load_matrix(directory.matrix(name, in_w, out_w)),
                    dense=lambda name, width: loader.load_dense(directory.dense(name, width)),
                    has_output="output.weight" in directory, finish=directory.reject_unexpected)
        self.quantized_bytes, self.dense_bytes = loader.quantized_bytes, loader.dense_bytes

    @classmethod
    def from_weights(cls, lane: HipExecutionLane, descriptor: DecoderDescriptor, matrix, dense, has_output: bool,
                     fused: bool = True) -> "QuantizedDecoder":
        """The same loop over weights that are already on the lane: matrix(name, in_w, out_w) returns a
        HipQuantizedMatrix whose payload is resident, dense(name, width) an FP32 HipBuffer; the decoder owns both."""
        self = cls.__new__(cls)
        self._build(lane, descriptor, fused, matrix, dense, has_output, finish=lambda: None)
        self.quantized_bytes = sum(m.storage_bytes for m in self._owned if isinstance(m, HipQuantizedMatrix))
        self.dense_bytes = sum(b.nbytes for b in self._owned if isinstance(b, HipBuffer))
        return self

    def _build(self, lane, descriptor, fused, matrix, dense, has_output, finish) -> None:
        self.lane = lane
        self.fused = fused
        self.descriptor = d = descriptor
        q_width, kv_width = d.head_count * d.head_width, d.kv_head_count * d.head_width
        self._owned: list = []

        def own(item):
            self._owned.append(item)
            return item

        def stack(parts):
            """One matrix from projections of the same vector; the parts are freed, the stack replaces them."""
            whole = own(HipQuantizedMatrix.stacked(lane, parts))
            for m in parts:
                self._owned.remove(m)
                m.dispose()
            return whole

        try:
            self.embedding = own(matrix("token_embd.weight", d.embedding_length, d.vocabulary))
            self.layers: list[_Layer] = []
            for i in range(d.layer_count):
                p, L = f"blk.{i}.", _Layer()
                L.attn_norm = own(dense(p + "attn_norm.weight", d.embedding_length))
                L.q = own(matrix(p + "attn_q.weight", d.embedding_length, q_width))
                L.k = own(matrix(p + "attn_k.weight", d.embedding_length, kv_width))
                L.v = own(matrix(p + "attn_v.weight", d.embedding_length, kv_width))
                L.o = own(matrix(p + "attn_output.weight", q_width, d.embedding_length))
                L.ffn_norm = own(dense(p + "ffn_norm.weight", d.embedding_length))
                L.gate = own(matrix(p + "ffn_gate.weight", d.embedding_length, d.feed_forward_length))
                L.up = own(matrix(p + "ffn_up.weight", d.embedding_length, d.feed_forward_length))
                L.down = own(matrix(p + "ffn_down.weight", d.feed_forward_length, d.embedding_length))
                L.qkv = L.gate_up = None
                if fused:
                    # projections of the same vector become one launch when their storage types agree
                    if L.q.ggml_type == L.k.ggml_type == L.v.ggml_type:
                        L.qkv = stack([L.q, L.k, L.v])
                        L.q = L.k = L.v = None
                    if L.gate.ggml_type == L.up.ggml_type:
                        L.gate_up = stack([L.gate, L.up])
                        L.gate = L.up = None
                self.layers.append(L)
            self.output_norm = own(dense("output_norm.weight", d.embedding_length))
            # a file without output.weight ties the head to the embedding, as llama.cpp does
            self.output = own(matrix("output.weight", d.embedding_length, d.vocabulary)) if has_output else self.embedding
            finish()
        except BaseException:
            self.dispose()
            raise

        # activations: allocated once, so a token step allocates nothing (and can be captured in a graph)
        alloc = lane.allocate
        self._hidden = [alloc(d.embedding_length), alloc(d.embedding_length)]
        self._cur = 0
        self._norm = alloc(d.embedding_length)
        self._qkv = alloc(q_width + 2 * kv_width)
        self._ctx = alloc(q_width)
        self._attn = alloc(d.embedding_length)
        self._gate_up = alloc(2 * d.feed_forward_length)
        self._act = alloc(d.feed_forward_length)
        self._down = alloc(d.embedding_length)
        self.logits = alloc(d.vocabulary)
        self._owned += self._hidden + [self._norm, self._qkv, self._ctx, self._attn, self._gate_up, self._act, self._down,
                                       self.logits]
        self._graph = None
        self._graph_start = 0

    # ---------------------------------------------------------------------------------------------- one token
    def _layers_and_head(self) -> None:
        d, lane = self.descriptor, self.lane
        q_width, kv_width, ffn, eps = d.head_count * d.head_width, d.kv_head_count * d.head_width, d.feed_forward_length, d.rms_epsilon
        q_view = self._qkv.view(0, 4 * q_width)
        k_view = self._qkv.view(4 * q_width, 4 * kv_width)
        v_view = self._qkv.view(4 * (q_width + kv_width), 4 * kv_width)
        gate_view, up_view = self._gate_up.view(0, 4 * ffn), self._gate_up.view(4 * ffn, 4 * ffn)
        for L in self.layers:
            cur, nxt = self._hidden[self._cur], self._hidden[self._cur ^ 1]
            if self.fused and L.qkv is not None and L.gate_up is not None:
                # Four launches.  The o projection reads the value heads itself (what first-token attention would have
                # copied) and adds the residual stream; the stacked gate | up projection leaves SiLU(gate) * up, so the
                # down projection reads one vector and nobody forms the product twice.  Every value has the bits of the
                # one-launch-per-operation sequence.
                L.qkv.forward_fused(lane, cur, pre_op=PRE_RMS_NORM, norm_weight=L.attn_norm, epsilon=eps, out=self._qkv)
                L.o.forward_fused(lane, v_view, addend=cur, out=nxt, x_head_width=d.head_width,
                                  x_head_group=d.head_count // d.kv_head_count)
                L.gate_up.forward_fused(lane, nxt, pre_op=PRE_RMS_NORM, norm_weight=L.ffn_norm, epsilon=eps, out=self._act,
                                        post_op=POST_SILU_PAIR)
                L.down.forward_fused(lane, self._act, addend=nxt, out=nxt)
                self._cur ^= 1
            elif self.fused:
                if L.qkv is not None:
                    L.qkv.forward_fused(lane, cur, pre_op=PRE_RMS_NORM, norm_weight=L.attn_norm, epsilon=eps, out=self._qkv)
                else:
                    L.q.forward_fused(lane, cur, pre_op=PRE_RMS_NORM, norm_weight=L.attn_norm, epsilon=eps, x_out=self._norm, out=q_view)
                    L.k.forward(lane, self._norm, None, out=k_view)
                    L.v.forward(lane, self._norm, None, out=v_view)
                qwen35_gpu.first_token_attention(lane, v_view, d.head_count, d.kv_head_count, d.head_width, out=self._ctx)
                L.o.forward(lane, self._ctx, None, out=self._attn)
                if L.gate_up is not None:
                    L.gate_up.forward_fused(lane, cur, pre_op=PRE_RMS_NORM, x2=self._attn, norm_weight=L.ffn_norm, epsilon=eps,
                                            sum_out=nxt, out=self._gate_up)
                else:
                    L.gate.forward_fused(lane, cur, pre_op=PRE_RMS_NORM, x2=self._attn, norm_weight=L.ffn_norm, epsilon=eps,
                                         x_out=self._norm, sum_out=nxt, out=gate_view)
                    L.up.forward(lane, self._norm, None, out=up_view)
                L.down.forward_fused(lane, gate_view, pre_op=PRE_SILU_MULTIPLY, x2=up_view, addend=nxt, out=nxt)
                self._cur ^= 1
            else:
                qwen35_gpu.rms_norm(lane, cur, L.attn_norm, 1, d.embedding_length, eps, out=self._norm)
                L.q.forward(lane, self._norm, None, out=q_view)
                L.k.forward(lane, self._norm, None, out=k_view)
                L.v.forward(lane, self._norm, None, out=v_view)
                qwen35_gpu.first_token_attention(lane, v_view, d.head_count, d.kv_head_count, d.head_width, out=self._ctx)
                L.o.forward(lane, self._ctx, None, out=self._attn)
                qwen35_gpu.add_residual_and_rms_norm(lane, cur, self._attn, L.ffn_norm, d.embedding_length, eps, out=self._norm)
                L.gate.forward(lane, self._norm, None, out=gate_view)
                L.up.forward(lane, self._norm, None, out=up_view)
                qwen35_gpu.silu_multiply(lane, gate_view, up_view, ffn, out=self._act)
                L.down.forward(lane, self._act, None, out=self._down)
                qwen35_gpu.add_in_place(lane, cur, self._down, d.embedding_length)
        hidden = self._hidden[self._cur]
        if self.fused:
            self.output.forward_fused(lane, hidden, pre_op=PRE_RMS_NORM, norm_weight=self.output_norm, epsilon=eps, out=self.logits)
        else:
            qwen35_gpu.rms_norm(lane, hidden, self.output_norm, 1, d.embedding_length, eps, out=self._norm)
            self.output.forward(lane, self._norm, None, out=self.logits)

    def forward_token(self, token_id: int) -> HipBuffer:
        """Logits of `token_id` decoded as the first token of a sequence; the buffer is reused by the next call."""
        if not 0 <= token_id < self.descriptor.vocabulary:
            raise IndexError(f"Embedding index {token_id} is outside the vocabulary.")
        if self._graph is not None:
            self._cur = self._graph_start
            self.embedding.dequantize(self.lane, row=token_id, out=self._hidden[self._cur])
            self.lane.graph_launch(self._graph)
            self._cur = self._graph_end
        else:
            self.embedding.dequantize(self.lane, row=token_id, out=self._hidden[self._cur])
            self._layers_and_head()
        return self.logits

    def capture_graph(self) -> None:
        """Records the layers and the head of a token step into a HIP graph that forward_token then replays (the
        embedding lookup stays outside: its source row changes with the token).  One eager step must have run."""
        if self._graph is not None:
            return
        self._graph_start = self._cur
        self.lane.graph_begin()
        try:
            self._layers_and_head()
        finally:
            graph = self.lane.graph_end()
        self._graph, self._graph_end = graph, self._cur

    # ---------------------------------------------------------------------------------------------- generation
    def generate(self, first_token: int, max_new_tokens: int, on_token=None) -> tuple[list[int], GenerationTiming]:
        """Greedy decoding, one token per step (each step sees only its own token: no cache).  The argmax runs on the
        host over the downloaded logits; first tie wins, as the reference's device ArgMax does."""
        if max_new_tokens < 0:
            raise ValueError("max_new_tokens must not be negative.")
        tokens: list[int] = []
        first = last = None
        started = time.perf_counter()
        token = first_token
        for _ in range(max_new_tokens):
            logits = self.lane.read(self.forward_token(token), count=self.descriptor.vocabulary)
            token = int(np.argmax(logits))
            last = (time.perf_counter() - started) * 1e3
            first = last if first is None else first
            tokens.append(token)
            if on_token is not None:
                on_token(token)
        total = (time.perf_counter() - started) * 1e3
        rate = (len(tokens) - 1) * 1000.0 / (last - first) if len(tokens) > 1 and last > first else None
        return tokens, GenerationTiming(len(tokens), total, first, rate)

    def dispose(self) -> None:
        if getattr(self, "_graph", None) is not None and not self.lane.disposed:
            self.lane.graph_destroy(self._graph)
        self._graph = None
        for item in reversed(getattr(self, "_owned", [])):
            item.dispose()
        self._owned = []

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.dispose()


__all__ = ["DecoderDescriptor", "GenerationTiming", "QuantizedDecoder", "NotSupportedError"]
