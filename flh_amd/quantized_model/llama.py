"""A W4A4 Llama model around the decoder layer: embedding, N layers, final norm, fp16 language-model head, and a
decode step that runs from a preallocated key / value cache and can be captured into one graph.

Data flow of the reference's FLH_LlamaForCausalLM.forward (flh/quantized_model/modeling_llama.py:668-693:
embedding -> [group configuration only: Hadamard of every 128 channels of the embeddings] -> decoder layers ->
final RMSNorm -> lm_head), with the layers of decoder_layer.py.  The int4 linears, the rotary embedding, attention and
the norms (the final one with the last residual addition in its launch) are this library's kernels on the fused path;
the embedding and the head are stock torch ops, as in the reference.
Weights are random (there are no checkpoints here): `random_init` draws fp16 weights layer by layer on the device and
quantises them through the same kernels a loader would use.
"""
import json
import math
import os

import torch

from ..nn.normalization import RMSNorm
from ..nn.quantization import fast_hadamard_transform
from .decoder_layer import StaticKVCache, W4A4DecoderLayer, rotary_tables


class LlamaShape:
    """The numbers that define a Llama-style stack."""

    def __init__(self, hidden_size=4096, num_heads=32, num_kv_heads=8, intermediate_size=14336, num_layers=32,
                 vocab_size=128256, eps=1e-5, rope_theta=500000.0):
        self.hidden_size, self.num_heads, self.num_kv_heads = hidden_size, num_heads, num_kv_heads
        self.intermediate_size, self.num_layers, self.vocab_size = intermediate_size, num_layers, vocab_size
        self.eps, self.rope_theta = eps, rope_theta
        self.head_dim = hidden_size // num_heads

    @classmethod
    def llama3_8b(cls, num_layers=32):
        return cls(4096, 32, 8, 14336, num_layers, 128256, 1e-5, 500000.0)

    @classmethod
    def llama2_7b(cls, num_layers=32):
        return cls(4096, 32, 32, 11008, num_layers, 32000, 1e-5, 10000.0)


_ATTENTION = ("q_proj", "k_proj", "v_proj", "o_proj")
_MLP = ("gate_proj", "up_proj", "down_proj")


def reference_key(key):
    """This model's state-dict key -> the key of the reference's model (a transformers LlamaForCausalLM subclass:
    `model.layers.N.self_attn.q_proj.w_packed`, `model.layers.N.mlp.up_proj.w_scale`, `model.norm.weight`, `lm_head.weight`)."""
    if key.startswith("lm_head."):
        return key
    parts = key.split(".")
    if parts[0] == "layers" and parts[2] in _ATTENTION:
        parts.insert(2, "self_attn")
    elif parts[0] == "layers" and parts[2] in _MLP:
        parts.insert(2, "mlp")
    return "model." + ".".join(parts)


class W4A4LlamaModel(torch.nn.Module):
    def __init__(self, shape, activation="token", weight_group_size=128, fused=True, device="cpu"):
        super().__init__()
        self.shape, self.activation, self.fused = shape, activation, fused
        self._norm16 = None                 # (version key, fp16 copy) of the final norm's weight
        self.embed_tokens = torch.nn.Embedding(shape.vocab_size, shape.hidden_size, device=device, dtype=torch.float16)
        self.layers = torch.nn.ModuleList(
            W4A4DecoderLayer(shape.hidden_size, shape.num_heads, shape.num_kv_heads, shape.intermediate_size, shape.eps,
                             128, weight_group_size, fused, device, activation) for _ in range(shape.num_layers))
        self.norm = RMSNorm(shape.hidden_size, shape.eps).to(device)
        self.lm_head = torch.nn.Linear(shape.hidden_size, shape.vocab_size, bias=False, device=device, dtype=torch.float16)

    @classmethod
    def random_init(cls, shape, activation="token", weight_group_size=128, fused=True, device="cuda", seed=0, six_bit=False):
        """Random fp16 weights ~ N(0, 1/K) per linear (norm weights ~ U(0.5, 1.5)), quantised on the device one layer
        at a time so that no more than one layer's fp16 weights exist at once.  `six_bit`: see set_six_bit."""
        model = cls(shape, activation, weight_group_size, fused, device="meta")
        model.embed_tokens = torch.nn.Embedding(shape.vocab_size, shape.hidden_size, device=device, dtype=torch.float16)
        model.lm_head = torch.nn.Linear(shape.hidden_size, shape.vocab_size, bias=False, device=device, dtype=torch.float16)
        model.norm = RMSNorm(shape.hidden_size, shape.eps).to(device)
        gen = torch.Generator(device=device).manual_seed(seed)
        with torch.no_grad():
            model.embed_tokens.weight.normal_(0.0, 1.0, generator=gen)
            model.lm_head.weight.normal_(0.0, 1.0 / math.sqrt(shape.hidden_size), generator=gen)
            model.norm.weight.uniform_(0.5, 1.5, generator=gen)
            model.norm.weight.copy_(model.norm.weight.half().float())     # as a checkpoint's fp16 norm weight would be
            kv = shape.num_kv_heads * shape.head_dim
            dims = {"q_proj": (shape.hidden_size, shape.hidden_size), "k_proj": (kv, shape.hidden_size),
                    "v_proj": (kv, shape.hidden_size), "o_proj": (shape.hidden_size, shape.hidden_size),
                    "gate_proj": (shape.intermediate_size, shape.hidden_size),
                    "up_proj": (shape.intermediate_size, shape.hidden_size),
                    "down_proj": (shape.hidden_size, shape.intermediate_size)}
            layers = []
            for _ in range(shape.num_layers):
                w = {name: (torch.randn(n, k, device=device, generator=gen) / math.sqrt(k)).half() for name, (n, k) in dims.items()}
                for name in ("input_layernorm", "post_attention_layernorm"):
                    w[name] = (torch.rand(shape.hidden_size, device=device, generator=gen) + 0.5).half()
                layers.append(W4A4DecoderLayer.from_float(w, shape.num_heads, shape.num_kv_heads, shape.eps, 128,
                                                          weight_group_size if activation == "token" else 128, fused,
                                                          activation, six_bit))
                del w
            model.layers = torch.nn.ModuleList(layers)
        return model

    # ------------------------------------------------------------------ the reference's checkpoint directory
    def reference_state_dict(self):
        """The state dict under the reference model's key names, float32 tensors as float16 (as its save_quantized
        stores them, flh/quantized_model/modeling_llama.py:1099-1107)."""
        out = {}
        for key, value in self.state_dict().items():
            value = value.detach().cpu()
            out[reference_key(key)] = value.half() if value.dtype == torch.float32 else value
        return out

    def load_reference_state_dict(self, state, strict=True):
        """Load a state dict with the reference model's key names (what its save_quantized wrote).  Keys this model has no
        counterpart for (rotary buffers, quantiser settings) are ignored; with `strict`, every tensor of this model must
        be present with its shape."""
        own = self.state_dict()
        missing = []
        with torch.no_grad():
            for key, dst in own.items():
                src = state.get(reference_key(key))
                if src is None:
                    missing.append(reference_key(key))
                    continue
                if tuple(src.shape) != tuple(dst.shape):
                    if src.numel() == dst.numel() and key.endswith("w_packed"):   # LinearFLHGS keeps [N, K/2], LinearFLH flat
                        src = src.reshape(dst.shape)
                    else:
                        raise ValueError(f"{reference_key(key)}: shape {tuple(src.shape)}, expected {tuple(dst.shape)}")
                dst.copy_(src.to(dst.dtype))
        if strict and missing:
            raise KeyError(f"missing in the checkpoint: {missing[:5]}{' ...' if len(missing) > 5 else ''}")
        return missing

    def save_quantized(self, save_directory, **quant_config):
        """Write the reference's checkpoint directory (modeling_llama.py:1079-1137): `model.pt` (pickle protocol 4, the
        reference model's key names), `quantization_config.json`, and `config.json` with the transformers fields that
        define the architecture."""
        from ..nn.checkpoint import QUANT_CONFIG_DEFAULTS
        unknown = set(quant_config) - set(QUANT_CONFIG_DEFAULTS)
        if unknown:
            raise ValueError(f"unknown quantisation settings: {sorted(unknown)}")
        os.makedirs(save_directory, exist_ok=True)
        torch.save(self.reference_state_dict(), os.path.join(save_directory, "model.pt"), pickle_protocol=4)
        first = self.layers[0].q_proj
        grouped = first.w_scale.view(first.out_features, -1).size(1) > 1       # else one scale per output channel
        settings = {**QUANT_CONFIG_DEFAULTS, "weight_group_size": first.weight_group_size if grouped else -1, **quant_config}
        with open(os.path.join(save_directory, "quantization_config.json"), "w") as f:
            json.dump(settings, f, indent=2)
        sh = self.shape
        with open(os.path.join(save_directory, "config.json"), "w") as f:
            json.dump({"architectures": ["LlamaForCausalLM"], "model_type": "llama", "hidden_size": sh.hidden_size,
                       "num_attention_heads": sh.num_heads, "num_key_value_heads": sh.num_kv_heads,
                       "intermediate_size": sh.intermediate_size, "num_hidden_layers": sh.num_layers,
                       "vocab_size": sh.vocab_size, "rms_norm_eps": sh.eps, "rope_theta": sh.rope_theta,
                       "hidden_act": "silu", "torch_dtype": "float16",
                       "flh_activation": self.activation}, f, indent=2)

    @classmethod
    def from_quantized(cls, load_directory, device="cuda", activation=None, fused=True, six_bit=False,
                       assume_symmetric_weights=False):
        """Build the model a checkpoint directory describes and load its tensors (modeling_llama.py:1139-1260).  The file
        is read without executing anything from it (flh_amd.nn.checkpoint.read_state_dict).  `activation`: "group" (the
        reference's own models) or "token"; default: what the directory's config says, else "group".  `six_bit`: see
        set_six_bit.

        Weight symmetry.  This path has kernels for symmetric codes only (signed nibbles, `w_zero` unused).  A directory
        whose quantization_config.json says `weight_sym: false` -- or lacks the key, which the reference's loader reads as
        false (modeling_llama.py:1153) -- is refused: the reference's default flow (from_float / save_quantized) writes
        exactly that flag, although its kernel forward never reads `w_zero` (flh/nn/linear.py:125-132) and the stored
        nibbles may well be what this path expects.  A caller who knows that the stored codes are signed nibbles with
        `w_zero` unused passes `assume_symmetric_weights=True`."""
        from ..nn.checkpoint import read_state_dict
        with open(os.path.join(load_directory, "config.json")) as f:
            cfg = json.load(f)
        with open(os.path.join(load_directory, "quantization_config.json")) as f:
            quant = json.load(f)
        for key, want in (("weight_bits", 4), ("act_bits", 4)):
            if quant.get(key, want) != want:
                raise ValueError(f"{key} = {quant[key]}: this path is W4A4")
        if not quant.get("act_sym", True):
            raise ValueError("asymmetric activation quantisation has no kernel on this path")
        if not quant.get("weight_sym", False) and not assume_symmetric_weights:
            raise ValueError("quantization_config.json does not say weight_sym: true (a missing key means false, as in the "
                             "reference's loader); asymmetric weight codes have no kernel on this path -- pass "
                             "assume_symmetric_weights=True if the stored codes are signed nibbles with w_zero unused")
        shape = LlamaShape(cfg["hidden_size"], cfg["num_attention_heads"],
                           cfg.get("num_key_value_heads", cfg["num_attention_heads"]), cfg["intermediate_size"],
                           cfg["num_hidden_layers"], cfg["vocab_size"], cfg.get("rms_norm_eps", 1e-5),
                           cfg.get("rope_theta", 10000.0))
        activation = activation or cfg.get("flh_activation", "group")
        model = cls(shape, activation, quant.get("weight_group_size", 128), fused, device="cpu")
        model.load_reference_state_dict(read_state_dict(os.path.join(load_directory, "model.pt")))
        model = model.to(device)
        model.set_six_bit(six_bit)
        return model

    @classmethod
    def from_float(cls, state, shape, activation="token", weight_group_size=128, fused=True, device="cuda", six_bit=False):
        """Quantise a float Llama checkpoint given as a state dict with the transformers key names
        (`model.layers.N.self_attn.q_proj.weight`, ..., `model.embed_tokens.weight`, `model.norm.weight`, `lm_head.weight`):
        round-to-nearest through the same kernels a loader of quantised weights uses, one layer on the device at a time
        (what the reference's `quantize` does layer by layer, modeling_llama.py:789-868, without its GPTQ option -- that is
        flh_amd.nn.FLHGPTQ on a layer's float weights before this call).  `six_bit`: see set_six_bit."""
        model = cls(shape, activation, weight_group_size, fused, device="meta")
        emb = state["model.embed_tokens.weight"]
        model.embed_tokens = torch.nn.Embedding(shape.vocab_size, shape.hidden_size, device=device, dtype=torch.float16)
        model.lm_head = torch.nn.Linear(shape.hidden_size, shape.vocab_size, bias=False, device=device, dtype=torch.float16)
        model.norm = RMSNorm(shape.hidden_size, shape.eps).to(device)
        layers = []
        with torch.no_grad():
            model.embed_tokens.weight.copy_(emb)
            model.lm_head.weight.copy_(state.get("lm_head.weight", emb))       # tied embeddings: no separate head
            model.norm.weight.copy_(state["model.norm.weight"].float())
            for i in range(shape.num_layers):
                pre = f"model.layers.{i}."
                w = {name: state[pre + ("self_attn." if name in _ATTENTION else "mlp.") + name + ".weight"].to(device).half()
                     for name in _ATTENTION + _MLP}
                for name in ("input_layernorm", "post_attention_layernorm"):
                    w[name] = state[pre + name + ".weight"].to(device).half()
                layers.append(W4A4DecoderLayer.from_float(w, shape.num_heads, shape.num_kv_heads, shape.eps, 128,
                                                          weight_group_size, fused, activation, six_bit))
                del w
        model.layers = torch.nn.ModuleList(layers)
        return model

    def set_six_bit(self, six_bit):
        """Whether prefill-sized calls of the layers' linears run on the 6-bit matrix instruction: False (default), True,
        or "auto" (only where it pays even with a re-encoding pass: weights with a scale per group of 128).  Anything but
        False makes every such linear hold a second, 6-bit copy of its weights -- 0.75 byte per weight on top of 0.5,
        about + 5 GB for a 7B model -- which is built here, not inside the first long call."""
        for layer in self.layers:
            layer.set_six_bit(six_bit)

    def new_cache(self, batch, max_len):
        s = self.shape
        dev = self.embed_tokens.weight.device
        return StaticKVCache(s.num_layers, batch, s.num_kv_heads, max_len, s.head_dim, dev, q_heads=s.num_heads)

    def embed(self, input_ids):
        x = self.embed_tokens(input_ids)
        if self.activation == "group":     # modeling_llama.py:672: the rotations of this arrangement live in the weights
            x = fast_hadamard_transform(x, group_size=128, normalize=True)
        return x

    def _rotary(self, positions, cache):
        """cos / sin [T, head_dim] of `positions`.  With a static cache the table of all its slots is computed once and
        the step's rows are gathered from it (two small launches instead of the dozen that build a table), the same
        values either way."""
        if cache is None:
            return rotary_tables(positions, self.shape.head_dim, self.shape.rope_theta)
        table = getattr(cache, "rotary_table", None)
        if table is None:
            table = rotary_tables(torch.arange(cache.max_len, device=positions.device), self.shape.head_dim,
                                  self.shape.rope_theta)
            cache.rotary_table = table
        return table[0].index_select(0, positions), table[1].index_select(0, positions)

    def forward(self, input_ids, positions, cache=None, return_hidden=False):
        """input_ids [B, T] int64, positions [T] int64 (the same for every sequence of the batch).  cache: None (a
        fresh prefill without cache), or a StaticKVCache whose kv_len is the number of slots attention reads, with
        positions == arange(kv_len - T, kv_len) (what cache.advance(T) returns; see StaticKVCache for why nothing else
        is meaningful).  Returns logits [B, T, vocab] fp16 (or the final hidden state)."""
        if cache is not None:
            t = input_ids.size(1)
            if positions.numel() != t or not 0 < t <= cache.kv_len <= cache.max_len:
                raise ValueError(f"a step over {t} tokens needs {t} positions and a cache with {t} <= kv_len "
                                 f"({cache.kv_len}) <= max_len ({cache.max_len})")
            if not torch.cuda.is_current_stream_capturing() and not torch.equal(
                    positions, torch.arange(cache.kv_len - t, cache.kv_len, dtype=positions.dtype, device=positions.device)):
                raise ValueError("positions must be arange(kv_len - T, kv_len) of the cache (cache.advance(T) returns them)")
        x = self.embed(input_ids)
        cos, sin = self._rotary(positions, cache)
        pending = None            # the last MLP output, added inside the next layer's first launch
        for i, layer in enumerate(self.layers):
            x, pending, _ = layer.forward_deferred(x, pending, cos, sin, cache.layer(i) if cache is not None else None,
                                                   positions)
        x = self._final_norm(x, pending)
        return x if return_hidden else self.lm_head(x)

    def _final_norm(self, x, pending):
        """The last residual addition and the final RMSNorm: one launch on the fused path (the roundings of the two
        torch expressions: fp16 sum, float32 statistics, two float32 products, fp16), torch's ten otherwise."""
        w = self.norm.weight
        if not (self.fused and x.is_cuda and x.dtype == torch.float16 and x.size(-1) % 8 == 0 and x.size(-1) <= 16384):
            return self.norm(x if pending is None else x + pending)
        key = (w.data_ptr(), w._version)
        if self._norm16 is None or self._norm16[0] != key:
            self._norm16 = (key, w.detach().to(torch.float16).contiguous())
        import flh_amd
        return flh_amd._CUDA.add_rmsnorm(x.contiguous(), self._norm16[1], self.norm.eps,
                                         add=None if pending is None else pending.contiguous())

    def capture_decode_step(self, batch, kv_len, cache=None, with_head=True):
        """Record one decode step (batch x 1 token, attention over `kv_len` cached positions, the new token in slot
        kv_len - 1) into a graph.  Returns (graph, static): `static` holds the input ids, the position tensor and the
        output logits the replays read and write; the cache must already hold the earlier positions.  The graph serves
        this kv_len only (the range attention reads is a launch parameter): a replay for another length needs a graph of
        its own, and `static["positions"]` is to be left at kv_len - 1."""
        dev = self.embed_tokens.weight.device
        cache = cache if cache is not None else self.new_cache(batch, kv_len)
        cache.kv_len = kv_len
        ids = torch.zeros(batch, 1, dtype=torch.int64, device=dev)
        pos = torch.full((1,), kv_len - 1, dtype=torch.int64, device=dev)
        side = torch.cuda.Stream(device=dev)
        side.wait_stream(torch.cuda.current_stream(dev))
        with torch.cuda.stream(side), torch.no_grad():
            for _ in range(2):              # every kernel variant runs once eagerly before the capture
                out = self.forward(ids, pos, cache, return_hidden=not with_head)
        torch.cuda.current_stream(dev).wait_stream(side)
        torch.cuda.synchronize(dev)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph), torch.no_grad():
            out = self.forward(ids, pos, cache, return_hidden=not with_head)
        return graph, {"input_ids": ids, "positions": pos, "output": out, "cache": cache}
