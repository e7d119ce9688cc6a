"""The W4A4 Llama harness (flh_amd.quantized_model) against the CPU oracle layer (oracle/layer.py), at full width.

Two workloads:
  * the Llama-3-8B decode step: batch {1, 8, 16} x 1 token, attention over 2048 cached positions, grouped queries
    32 / 8, intermediate 14336 with the 28 x 512 online rotation, group-of-128 weight scales, per-token activation
    scales, final norm and the fp16 head of 128 256 rows -- two full-width layers here (the 32 of the full model repeat
    them; bench.py runs all 32);
  * a Llama-2-7B decoder layer at 8 x 512 tokens (per-token activations, per-channel weight scales, 172 x 64 rotation).

Every stage of the device layer is checked with the oracle fed the device's own input of that stage (its `record`
taps): quantised operands bit for bit where the arithmetic is this library's (the float32-butterfly rotation of 4096
and the quantiser), by mismatch rate where the device's float32 order is not the oracle's (RMSNorm statistics in front
of the rotation; the matrix-core rotation of 11008 / 14336); every linear's fp16 output within rtol 1e-3 / atol 1e-2 of
the oracle GEMM on the same codes and scales; the attention block (RoPE, cache write, grouped queries, masking) against
the float64 attention.  On top, the free-running oracle model from the same inputs bounds the end-to-end difference.
"""
import numpy as np
import pytest
import torch

from flh_amd.quantized_model import LlamaShape, StaticKVCache, W4A4DecoderLayer, W4A4LlamaModel, rotary_tables

pytestmark = pytest.mark.gpu


def host(t):
    return t.detach().cpu().numpy()


def oracle_weights(layer, activation, weight_group):
    from oracle import layer as OL
    packed = {n: host(getattr(layer, n).w_packed).reshape(getattr(layer, n).out_features, -1) for n in layer.PROJECTIONS}
    scales = {n: host(getattr(layer, n).w_scale).reshape(getattr(layer, n).out_features, -1) for n in layer.PROJECTIONS}
    norms = {n: host(getattr(layer, n).weight).astype(np.float16) for n in ("input_layernorm", "post_attention_layernorm")}
    for n in norms:      # the device holds float32 norm weights that came from fp16 values: the conversion is exact
        assert np.array_equal(norms[n].astype(np.float32), host(getattr(layer, n).weight))
    return OL.LayerWeights(packed, scales, norms, layer.num_heads, layer.num_kv_heads, layer.eps, activation, weight_group)


def mismatch(a, b):
    return float(np.mean(a != b))


def nibble_step(a, b):
    """largest difference between the int4 codes of two packed arrays"""
    from oracle.pack import unpack_i4
    return int(np.abs(unpack_i4(a).astype(np.int32) - unpack_i4(b).astype(np.int32)).max())


def ulp_distance(a, b):
    return int(np.abs(a.view(np.int16).astype(np.int32) - b.view(np.int16).astype(np.int32)).max())


def check_layer_stages(rec, w, x_rows, cos, sin, b, t, past_kv, sample=None, label=""):
    """rec: the device layer's taps (host arrays); w: oracle weights; x_rows fp16 [b * t, hidden]: the layer's input;
    past_kv: None or (keys, values) host arrays [b, Hkv, past, d].  `sample`: row indices for the GEMM checks."""
    from oracle import gemm as G
    from oracle import layer as OL
    from oracle import prologue
    rec = {k: v.reshape(-1, v.shape[-1]) for k, v in rec.items()}     # linear outputs arrive as [b, t, N]
    rows = np.arange(b * t) if sample is None else sample
    hidden = x_rows.shape[1]
    hd = hidden // w.num_heads

    def gemm_stage(name, codes, scales):
        ref, _ = G.gemm_i4_dequant(codes[rows], w.packed[name], scales[rows], w.scales[name], group=w.weight_group)
        got = rec[name][rows]
        assert np.allclose(got.astype(np.float64), ref.astype(np.float64), rtol=1e-3, atol=1e-2), (label, name)
        return mismatch(got.view(np.uint16), ref.view(np.uint16))

    report = {}
    # quantiser behind RMSNorm: the device's float32 statistics / rsqrt are its own -> codes by mismatch rate
    assert np.array_equal(rec["attn_in.input"], x_rows)
    q, s, _ = OL.quantise(w, x_rows, w.norms["input_layernorm"])
    report["attn_in codes"] = mismatch(rec["attn_in.codes"], q)
    assert report["attn_in codes"] < 2e-3 and nibble_step(rec["attn_in.codes"], q) <= 1, (label, report)
    assert ulp_distance(rec["attn_in.scales"], s) <= 2
    for name in ("q_proj", "k_proj", "v_proj"):
        report[name] = gemm_stage(name, rec["attn_in.codes"], rec["attn_in.scales"])
    # attention block from the device's own projections
    heads = {n: rec[n].reshape(b, t, nh, hd).transpose(0, 2, 1, 3) for n, nh in
             (("q_proj", w.num_heads), ("k_proj", w.num_kv_heads), ("v_proj", w.num_kv_heads))}
    qs, ks, vs = OL.apply_rotary(heads["q_proj"], cos, sin), OL.apply_rotary(heads["k_proj"], cos, sin), heads["v_proj"]
    past = 0
    if past_kv is not None:
        past = past_kv[0].shape[2]
        ks, vs = np.concatenate((past_kv[0], ks), axis=2), np.concatenate((past_kv[1], vs), axis=2)
    att = OL.attention_f64(qs, ks, vs, past).transpose(0, 2, 1, 3).reshape(b * t, hidden)
    diff = np.abs(rec["attn_out.input"].astype(np.float64) - att.astype(np.float64))
    report["attention max abs diff"] = float(diff.max())
    assert diff.max() <= 4e-3 * max(1.0, float(np.abs(att.astype(np.float64)).max())), (label, report)
    # quantiser without norm at the hidden width: this library's arithmetic end to end -> bit for bit
    q, s, _ = OL.quantise(w, rec["attn_out.input"])
    if w.activation == "group" or hidden & (hidden - 1) == 0:
        assert np.array_equal(rec["attn_out.codes"], q) and np.array_equal(rec["attn_out.scales"].view(np.uint16), s.view(np.uint16)), label
    report["o_proj"] = gemm_stage("o_proj", rec["attn_out.codes"], rec["attn_out.scales"])
    resid = (x_rows.astype(np.float32) + rec["o_proj"].astype(np.float32)).astype(np.float16)
    assert np.array_equal(rec["mlp_in.input"], resid), label
    q, s, _ = OL.quantise(w, resid, w.norms["post_attention_layernorm"])
    report["mlp_in codes"] = mismatch(rec["mlp_in.codes"], q)
    assert report["mlp_in codes"] < 2e-3 and nibble_step(rec["mlp_in.codes"], q) <= 1, (label, report)
    for name in ("gate_proj", "up_proj"):
        report[name] = gemm_stage(name, rec["mlp_in.codes"], rec["mlp_in.scales"])
    mid = prologue.silu_mul_f16(rec["gate_proj"], rec["up_proj"])
    report["silu*up fp16 mismatch"] = mismatch(rec["mlp_mid.input"].view(np.uint16), mid.view(np.uint16))
    assert report["silu*up fp16 mismatch"] < 5e-3, (label, report)          # device exp / division: last-bit differences
    # the intermediate width (172 x 64 / 28 x 512): matrix-core rotation on the device, float32 matmul_hadU in the oracle
    q, s, _ = OL.quantise(w, rec["mlp_mid.input"])
    report["mlp_mid codes"] = mismatch(rec["mlp_mid.codes"], q)
    inter = rec["mlp_mid.input"].shape[1]
    if w.activation == "token" and inter & (inter - 1):
        assert report["mlp_mid codes"] < 3e-3 and nibble_step(rec["mlp_mid.codes"], q) <= 1, (label, report)
        assert ulp_distance(rec["mlp_mid.scales"], s) <= 2
    else:
        assert np.array_equal(rec["mlp_mid.codes"], q) and np.array_equal(rec["mlp_mid.scales"].view(np.uint16), s.view(np.uint16)), label
    report["down_proj"] = gemm_stage("down_proj", rec["mlp_mid.codes"], rec["mlp_mid.scales"])
    out = (resid.astype(np.float32) + rec["down_proj"].astype(np.float32)).astype(np.float16)
    return out, report


@pytest.fixture(scope="module")
def llama3_two_layers():
    assert torch.cuda.is_available()
    shape = LlamaShape.llama3_8b(num_layers=2)
    with torch.no_grad():
        model = W4A4LlamaModel.random_init(shape, activation="token", weight_group_size=128, fused=True, seed=3)
    weights = [oracle_weights(l, "token", 128) for l in model.layers]
    return model, weights


@pytest.mark.parametrize("batch", [1, 8, 16])
def test_llama3_decode_step_against_the_oracle(llama3_two_layers, batch):
    from oracle import layer as OL
    model, weights = llama3_two_layers
    shape = model.shape
    kv_len = 2048
    gen = torch.Generator(device="cuda").manual_seed(100 + batch)
    cache = model.new_cache(batch, kv_len)
    # A cache state as a 2047-token prefill would leave it, with synthetic contents.  Keys ~ N(0, 0.25^2): with unit-variance
    # random keys the scores of this random-weight model have a spread of ~ 11, softmax is nearly one-hot over 2048
    # positions and the free-running comparison at the end turns into a test of which near-tied key wins.
    for i in range(shape.num_layers):
        cache.keys[i][:, :, :kv_len - 1].normal_(0.0, 0.25, generator=gen)
        cache.values[i][:, :, :kv_len - 1].normal_(0.0, 1.0, generator=gen)
    past = [(host(cache.keys[i][:, :, :kv_len - 1]), host(cache.values[i][:, :, :kv_len - 1])) for i in range(shape.num_layers)]
    cache.kv_len = kv_len
    ids = torch.randint(0, shape.vocab_size, (batch, 1), device="cuda", generator=gen)
    pos = torch.tensor([kv_len - 1], device="cuda")
    print(f"case llama3 decode step batch={batch}", flush=True)
    # recorded run (module-by-module o_proj so that every stage is visible)
    recs = [dict() for _ in model.layers]
    for layer, r in zip(model.layers, recs):
        layer.record = r
    with torch.no_grad():
        hidden_rec = model(ids, pos, cache, return_hidden=True)
    for layer in model.layers:
        layer.record = None
    new_k = [host(cache.keys[i][:, :, kv_len - 1]) for i in range(shape.num_layers)]
    # the production run: fused decode path, then head
    with torch.no_grad():
        logits = model(ids, pos, cache)
        hidden = model(ids, pos, cache, return_hidden=True)
    assert torch.equal(hidden, hidden_rec), "the single-launch decode path must give the recorded path's bits"
    for i in range(shape.num_layers):       # replaying the step rewrites the same slot with the same keys
        assert np.array_equal(host(cache.keys[i][:, :, kv_len - 1]), new_k[i])
        assert np.array_equal(host(cache.keys[i][:, :, :kv_len - 1]), past[i][0])

    x = host(model.embed(ids)).reshape(batch, shape.hidden_size)
    cos, sin = OL.rotary_tables(np.array([kv_len - 1]), shape.head_dim, shape.rope_theta)
    dcos, dsin = rotary_tables(pos, shape.head_dim, shape.rope_theta)
    assert np.abs(host(dcos).astype(np.float64) - cos.astype(np.float64)).max() <= 1e-3
    assert np.abs(host(dsin).astype(np.float64) - sin.astype(np.float64)).max() <= 1e-3
    cos, sin = host(dcos), host(dsin)           # the device's tables (they differ from float64 in the last fp16 bit at most)
    rows = x
    for i, (w, r) in enumerate(zip(weights, recs)):
        rec = {k: host(v) for k, v in r.items()}
        rows, report = check_layer_stages(rec, w, rows, cos, sin, batch, 1, past[i], label=f"layer {i} batch {batch}")
        print(f"  layer {i}: " + ", ".join(f"{k} {v:.2e}" for k, v in report.items()), flush=True)
    # final norm and head (stock torch ops) on the device's last hidden state
    from oracle import prologue
    fn = host(model.norm.weight).astype(np.float16)
    want_hidden = prologue.rmsnorm_f16(rows, fn, shape.eps)
    got_hidden = host(hidden).reshape(batch, -1)
    assert mismatch(got_hidden.view(np.uint16), want_hidden.view(np.uint16)) < 5e-3
    assert np.allclose(got_hidden.astype(np.float64), want_hidden.astype(np.float64), rtol=2e-3, atol=1e-3)
    sample = np.random.default_rng(batch).choice(shape.vocab_size, 2048, replace=False)
    head = host(model.lm_head.weight[torch.from_numpy(sample).cuda()]).astype(np.float64)
    want_logits = got_hidden.astype(np.float64) @ head.T
    got_logits = host(logits).reshape(batch, -1)[:, sample].astype(np.float64)
    assert logits.shape == (batch, 1, shape.vocab_size)
    assert np.allclose(got_logits, want_logits, rtol=2e-3, atol=2e-2)
    # Free-running oracle model from the same inputs.  An int4 quantiser amplifies a small input difference: a relative
    # perturbation e of a row moves every value by ~ 2.5 e quantisation steps, flips that fraction of the codes by one
    # step and so changes the next linear's output by ~ sqrt(2.5 e) / 2.5 -- the 4e-4 of differing codes behind the
    # matrix-core rotation (0.8 % of one down_proj output) become 5 % at the next layer's projections.  The end-to-end
    # bound is therefore loose and only guards the wiring; the stage checks above are the parity statement.
    ocos, osin = OL.rotary_tables(np.array([kv_len - 1]), shape.head_dim, shape.rope_theta)
    free = x.reshape(batch, 1, -1)
    for i, (w, r) in enumerate(zip(weights, recs)):
        taps = {}
        free, _ = OL.decoder_layer(w, free, ocos, osin, past[i], taps=taps)
        drift = {}
        for name in ("q_proj", "attn_out.input", "o_proj", "gate_proj", "mlp_mid.input", "down_proj"):
            a, d = taps[name].astype(np.float64).reshape(batch, -1), host(r[name]).astype(np.float64).reshape(batch, -1)
            drift[name] = np.linalg.norm(a - d) / np.linalg.norm(d)
        print(f"  free-running oracle, layer {i}: " + ", ".join(f"{k} {v:.1e}" for k, v in drift.items()), flush=True)
        if i == 0:      # the first quantiser sees identical inputs; behind it only last-bit differences, amplified once or twice
            assert drift["q_proj"] < 1e-3 and drift["attn_out.input"] < 2e-3 and max(drift.values()) < 0.15
    free = prologue.rmsnorm_f16(free, fn, shape.eps)
    err = np.linalg.norm(free.reshape(batch, -1).astype(np.float64) - got_hidden.astype(np.float64)) / np.linalg.norm(got_hidden.astype(np.float64))
    print(f"  free-running oracle vs device, final hidden state: relative difference {err:.3e}", flush=True)
    assert err < 0.3


@pytest.mark.parametrize("tokens", [1, 24, 600])
def test_residual_additions_inside_the_next_launch_change_no_bit(llama3_two_layers, tokens):
    """The stack hands (stream, pending addition) from layer to layer, so that every residual addition runs inside the
    norm + quantiser launch that reads it; layer by layer with torch's additions in between must give the same bits
    (decode-sized, short and prefill-sized row counts take different kernels)."""
    model, _ = llama3_two_layers
    shape = model.shape
    gen = torch.Generator(device="cuda").manual_seed(tokens)
    ids = torch.randint(0, shape.vocab_size, (1, tokens), device="cuda", generator=gen)
    pos = torch.arange(tokens, device="cuda")
    print(f"case deferred residual tokens={tokens}", flush=True)
    with torch.no_grad():
        got = model(ids, pos, None, return_hidden=True)
        x = model.embed(ids)
        cos, sin = rotary_tables(pos, shape.head_dim, shape.rope_theta)
        for layer in model.layers:
            attn, _ = layer.attention(x, cos, sin)
            x = x + attn
            x = x + layer.mlp(x)
        want = model._final_norm(x, None)     # the model's own norm launch (its last-bit differences from torch's
        stock = model.norm(x)                 # expression -- summation order -- are tested on their own)
    assert torch.equal(got, want)
    d = (want.view(torch.int16).int() - stock.view(torch.int16).int()).abs()
    assert d.max().item() <= 1 and (d != 0).float().mean().item() <= 1e-3


def test_llama3_decode_step_replays_from_a_graph(llama3_two_layers):
    """The whole step (two layers, norm, head) captured once and replayed: the same logits as the eager step, on
    every replay, also after the token and the cache contents change between replays."""
    model, _ = llama3_two_layers
    shape = model.shape
    batch, kv_len = 8, 2048
    gen = torch.Generator(device="cuda").manual_seed(5)
    graph, st = model.capture_decode_step(batch, kv_len)
    cache = st["cache"]
    for round_ in range(3):
        for i in range(shape.num_layers):
            cache.keys[i][:, :, :kv_len - 1].normal_(0.0, 1.0, generator=gen)
            cache.values[i][:, :, :kv_len - 1].normal_(0.0, 1.0, generator=gen)
        st["input_ids"].copy_(torch.randint(0, shape.vocab_size, (batch, 1), device="cuda", generator=gen))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        got = st["output"].clone()
        with torch.no_grad():
            want = model(st["input_ids"], st["positions"], cache)
        torch.cuda.synchronize()
        assert torch.equal(got, want), f"replay {round_}"


def test_llama2_layer_8x512_against_the_oracle():
    """BASELINE configuration 4: one Llama-2-7B decoder layer, batch 8 x 512 tokens, per-token activations with the
    whole-row online rotation (4096, and 172 x 64 in front of down_proj), per-channel weight scales.  Quantiser and
    attention stages on the whole batch, GEMM stages on 192 sampled tokens (the oracle's matrix products)."""
    from oracle import layer as OL
    b, t, hidden, heads, inter = 8, 512, 4096, 32, 11008
    gen = torch.Generator(device="cuda").manual_seed(21)
    dims = {"q_proj": (hidden, hidden), "k_proj": (hidden, hidden), "v_proj": (hidden, hidden), "o_proj": (hidden, hidden),
            "gate_proj": (inter, hidden), "up_proj": (inter, hidden), "down_proj": (hidden, inter)}
    w16 = {n: (torch.randn(s, device="cuda", generator=gen) / s[1] ** 0.5).half() for n, s in dims.items()}
    for n in ("input_layernorm", "post_attention_layernorm"):
        w16[n] = (torch.rand(hidden, device="cuda", generator=gen) + 0.5).half()
    with torch.no_grad():
        layer = W4A4DecoderLayer.from_float(w16, heads, heads, activation="token", fused=True)
    del w16
    w = oracle_weights(layer, "token", 128)
    assert w.scales["q_proj"].shape == (hidden, 1)
    x = torch.randn(b, t, hidden, device="cuda", generator=gen).half()
    x[..., ::97] *= 12.0                                 # outlier channels
    cos, sin = rotary_tables(torch.arange(t, device="cuda"), hidden // heads)
    print("case llama2 layer 8x512", flush=True)
    rec = {}
    layer.record = rec
    with torch.no_grad():
        y_rec, (k_rec, v_rec) = layer(x, cos, sin)
    layer.record = None
    with torch.no_grad():
        y, (k, v) = layer(x, cos, sin)
    assert torch.equal(k, k_rec) and torch.equal(v, v_rec)
    # the production run computes silu(gate) * up inside the gate / up launch (device exponential) and attention with the
    # library's own kernel where the recorded run used torch's kernels: the same values but for a last fp16 bit here and
    # there, which the two int4 quantisers behind them turn into a few per cent of the layer's update (far below the
    # int4 noise itself, which the stage checks below bound against the oracle)
    rel = ((y.float() - y_rec.float()).norm() / (y_rec.float() - x.float()).norm()).item()
    print(f"  production launches vs module sequence: relative difference of the layer's update {rel:.2e}", flush=True)
    assert rel < 5e-2
    rec = {kk: host(vv).reshape(-1, vv.shape[-1]) for kk, vv in rec.items()}
    sample = np.sort(np.random.default_rng(4).choice(b * t, 192, replace=False))
    out, report = check_layer_stages(rec, w, host(x).reshape(b * t, hidden), host(cos), host(sin), b, t, None,
                                     sample=sample, label="llama2 8x512")
    print("  " + ", ".join(f"{kk} {vv:.2e}" for kk, vv in report.items()), flush=True)
    assert np.array_equal(host(y_rec).reshape(b * t, hidden), out)
    # whole-batch invariants of the outputs the sampled GEMM checks did not see: every row of every projection is
    # the row the same launch gives for that token alone (prefill kernel against the decode kernel, same bits)
    ops = __import__("flh_amd")._CUDA
    for name, codes, scales in (("q_proj", "attn_in", "attn_in"), ("down_proj", "mlp_mid", "mlp_mid")):
        lin = getattr(layer, name)
        pick = torch.from_numpy(sample[:48]).cuda()
        qd, sd = torch.from_numpy(rec[codes + ".codes"]).cuda()[pick].contiguous(), torch.from_numpy(rec[scales + ".scales"]).cuda()[pick].contiguous()
        small = ops.gemm_i4_dequant(qd, lin.w_packed.view(lin.out_features, -1), sd, lin.w_scale, 128)
        assert np.array_equal(host(small), rec[name][sample[:48]])
    # free-running oracle on a few sequences would repeat the stage checks; the end-to-end bound on one sequence:
    free, _ = OL.decoder_layer(w, host(x[:1]), host(cos), host(sin))
    got = host(y_rec[:1]).astype(np.float64)
    err = np.linalg.norm(free.astype(np.float64) - got) / np.linalg.norm(got - host(x[:1]).astype(np.float64))
    print(f"  free-running oracle layer vs device (sequence 0): relative difference of the update {err:.3e}", flush=True)
    assert err < 0.3          # see the note on quantiser amplification in the decode-step test


@pytest.mark.parametrize("activation,group", [("token", 128), ("token", 0), ("group", 128)])
def test_float_checkpoint_to_quantised_directory_and_back(tmp_path, activation, group):
    """A float checkpoint under the transformers key names -> W4A4LlamaModel.from_float -> save_quantized (the reference's
    directory layout) -> from_quantized: the reloaded model gives the same logits bit for bit, for prefill and for a
    decode step from the static cache."""
    import math
    shape = LlamaShape(512, 4, 2, 1024, 2, 320, 1e-5, 10000.0)
    gen = torch.Generator().manual_seed(7)
    state = {"model.embed_tokens.weight": torch.randn(shape.vocab_size, shape.hidden_size, generator=gen).half(),
             "model.norm.weight": (torch.rand(shape.hidden_size, generator=gen) + 0.5).half(),
             "lm_head.weight": (torch.randn(shape.vocab_size, shape.hidden_size, generator=gen) / math.sqrt(shape.hidden_size)).half()}
    kv = shape.num_kv_heads * shape.head_dim
    dims = {"self_attn.q_proj": (512, 512), "self_attn.k_proj": (kv, 512), "self_attn.v_proj": (kv, 512),
            "self_attn.o_proj": (512, 512), "mlp.gate_proj": (1024, 512), "mlp.up_proj": (1024, 512), "mlp.down_proj": (512, 1024)}
    for i in range(shape.num_layers):
        for name, (n, k) in dims.items():
            state[f"model.layers.{i}.{name}.weight"] = (torch.randn(n, k, generator=gen) / math.sqrt(k)).half()
        for name in ("input_layernorm", "post_attention_layernorm"):
            state[f"model.layers.{i}.{name}.weight"] = (torch.rand(shape.hidden_size, generator=gen) + 0.5).half()
    print(f"case checkpoint round trip activation={activation} group={group}", flush=True)
    with torch.no_grad():
        model = W4A4LlamaModel.from_float(state, shape, activation=activation, weight_group_size=group)
        model.save_quantized(tmp_path)
        again = W4A4LlamaModel.from_quantized(tmp_path, device="cuda")
        assert again.activation == activation
        ids = torch.randint(0, shape.vocab_size, (2, 40), device="cuda", generator=torch.Generator(device="cuda").manual_seed(1))
        pos = torch.arange(40, device="cuda")
        want, got = model(ids, pos), again(ids, pos)
        assert torch.isfinite(want).all() and torch.equal(want, got)
        # a decode step from a static cache filled by the prefill
        for m, ref in ((model, None), (again, None)):
            cache = m.new_cache(2, 64)
            assert torch.equal(cache.advance(40), pos) and cache.kv_len == 40
            m(ids, pos, cache)
            step = m(ids[:, :1], cache.advance(1), cache)
            assert cache.kv_len == 41
            if m is model:
                first = step
        assert torch.equal(first, step)
        # positions that are not the last T slots of what attention reads are refused, as is a cache that cannot grow
        with pytest.raises(ValueError):
            model(ids[:, :1], torch.tensor([17], device="cuda"), cache)
        with pytest.raises(ValueError):
            model(ids[:, :2], torch.tensor([40], device="cuda"), cache)
        with pytest.raises(ValueError):
            cache.advance(64)


def test_llama3_32_layer_decode_graph_against_the_oracle():
    """The step that the benchmark times for the Llama-3-8B decode configuration -- all 32 layers, norm and head, one
    captured graph, KV length 2048 -- on one sequence: a replay gives the eager step's logits bit for bit, every layer's
    input is the previous layer's residual stream plus its MLP output (all 32), and layers 0, 15 and 31 are checked stage
    by stage against the oracle with the device's own inputs and their own cache contents (a cache slot, position or
    layer-index mix-up that only shows deep in the stack would fail there)."""
    from oracle import layer as OL
    from oracle import prologue
    shape = LlamaShape.llama3_8b(num_layers=32)
    batch, kv_len = 1, 2048
    with torch.no_grad():
        model = W4A4LlamaModel.random_init(shape, activation="token", weight_group_size=128, fused=True, seed=1)
    gen = torch.Generator(device="cuda").manual_seed(77)
    cache = model.new_cache(batch, kv_len)
    for i in range(shape.num_layers):       # every layer its own contents
        cache.keys[i][:, :, :kv_len - 1].normal_(0.0, 0.25, generator=gen)
        cache.values[i][:, :, :kv_len - 1].normal_(0.0, 1.0, generator=gen)
    tapped = (0, 15, 31)
    past = {i: (host(cache.keys[i][:, :, :kv_len - 1]), host(cache.values[i][:, :, :kv_len - 1])) for i in tapped}
    print("case llama3 32-layer decode graph", flush=True)
    graph, st = model.capture_decode_step(batch, kv_len, cache=cache)
    ids = torch.randint(0, shape.vocab_size, (batch, 1), device="cuda", generator=gen)
    st["input_ids"].copy_(ids)
    torch.cuda.synchronize()
    graph.replay()
    torch.cuda.synchronize()
    replayed = st["output"].clone()
    graph.replay()                          # a second replay rewrites the same slots with the same values
    torch.cuda.synchronize()
    assert torch.equal(st["output"], replayed)
    recs = [dict() for _ in model.layers]
    for layer, r in zip(model.layers, recs):
        layer.record = r
    with torch.no_grad():
        hidden_rec = model(ids, st["positions"], cache, return_hidden=True)
    for layer in model.layers:
        layer.record = None
    with torch.no_grad():
        logits = model(ids, st["positions"], cache)
        hidden = model(ids, st["positions"], cache, return_hidden=True)
    assert torch.equal(hidden, hidden_rec), "the single-launch decode path must give the recorded path's bits"
    assert torch.equal(replayed, logits), "a graph replay must give the eager step's logits"
    assert torch.isfinite(logits).all()
    # the residual stream through all 32 layers, from the recorded tensors alone
    x0 = host(model.embed(ids)).reshape(batch, shape.hidden_size)
    carried = x0
    for i, r in enumerate(recs):
        assert np.array_equal(host(r["attn_in.input"]).reshape(batch, -1), carried), f"input of layer {i}"
        resid = host(r["mlp_in.input"]).reshape(batch, -1)
        want = (carried.astype(np.float32) + host(r["o_proj"]).reshape(batch, -1).astype(np.float32)).astype(np.float16)
        assert np.array_equal(resid, want), f"residual stream behind the attention of layer {i}"
        carried = (resid.astype(np.float32) + host(r["down_proj"]).reshape(batch, -1).astype(np.float32)).astype(np.float16)
    fn = host(model.norm.weight).astype(np.float16)
    want_hidden = prologue.rmsnorm_f16(carried, fn, shape.eps)
    got_hidden = host(hidden).reshape(batch, -1)
    assert mismatch(got_hidden.view(np.uint16), want_hidden.view(np.uint16)) < 5e-3
    sample = np.random.default_rng(3).choice(shape.vocab_size, 2048, replace=False)
    head = host(model.lm_head.weight[torch.from_numpy(sample).cuda()]).astype(np.float64)
    assert np.allclose(host(logits).reshape(batch, -1)[:, sample].astype(np.float64), got_hidden.astype(np.float64) @ head.T,
                       rtol=2e-3, atol=2e-2)
    # stage by stage, three layers
    dcos, dsin = rotary_tables(st["positions"], shape.head_dim, shape.rope_theta)
    cos, sin = host(dcos), host(dsin)
    for i in tapped:
        w = oracle_weights(model.layers[i], "token", 128)
        rec = {k: host(v) for k, v in recs[i].items()}
        rows = rec["attn_in.input"].reshape(batch, -1)
        # (this layer's slot kv_len - 1 now holds its new key; the oracle appends its own to the earlier positions)
        assert np.array_equal(host(cache.keys[i][:, :, :kv_len - 1]), past[i][0])
        _, report = check_layer_stages(rec, w, rows, cos, sin, batch, 1, past[i], label=f"32-layer graph, layer {i}")
        print(f"  layer {i}: " + ", ".join(f"{k} {v:.2e}" for k, v in report.items()), flush=True)
    del model, cache, graph
    torch.cuda.empty_cache()
