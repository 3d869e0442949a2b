"""The mechanisms of the Tirurax layers alone, each against its plain function: the
row-wise kernels, the attention options (values of another width, the norm over a whole
projection, chunks, distance slopes, the sink) with keys made to stand out just inside and
just outside a chunk and far away, the gated delta rule in portions, token by token and
with slots used again, the dense feed-forward, and the block that norms its sublayers'
outputs."""
import pytest
import torch

import plain_tirurax as plain
from helpers import assert_close_f32

pytestmark = pytest.mark.gpu
DEV = "cuda"
HIDDEN, VOCAB, EPS = 48, 31, 1e-5


def one_layer(mixer, ffn=None):
    from edge_infer_amd.config.specs import LayerSpec, ModelSpec, NormSpec, default_schedule
    norm = NormSpec(eps=EPS)
    return ModelSpec(architecture="test", vocab_size=VOCAB, hidden_size=HIDDEN,
                     layers=(LayerSpec(block="outnorm", norm=norm, mixer=mixer, feed_forward=ffn),),
                     schedule=default_schedule(1), final_norm=norm, tie_word_embeddings=False,
                     max_position_embeddings=1 << 20, bos_token_id=None, eos_token_id=None)


def params_for(spec, seed):
    """Order-one parameters by parameter path, float32 values that bfloat16 holds exactly."""
    from edge_infer_amd.engine.model import model_parameters
    g = torch.Generator().manual_seed(seed)
    out = {}
    for path, param in model_parameters(spec).items():
        if param.optional:
            continue
        shape = tuple(param.shape)
        if param.init == "norm":
            value = 1 + 0.2 * (torch.rand(shape, generator=g) - 0.5)
        elif param.init == "uniform":
            value = param.low + (param.high - param.low) * torch.rand(shape, generator=g)
        elif len(shape) == 2 and "conv" not in path:
            value = torch.randn(shape, generator=g) / shape[1] ** 0.5
        else:
            value = torch.randn(shape, generator=g) * 0.5
        out[path] = value.to(torch.bfloat16).float()
    return out


def session_for(spec, params, dtype="float32", max_tokens=1024, max_seqs=4):
    from edge_infer_amd.engine import DecoderModel, Session
    model = DecoderModel(spec, params, dtype, DEV)
    return model, Session(model, max_tokens=max_tokens, max_seqs=max_seqs, graphs=False)


def run_part(session, part, pieces):
    """`pieces`: (slot, start, x rows) per sequence of one step; the part's output rows."""
    from edge_infer_amd.config.specs import ScheduleEntry
    from edge_infer_amd.engine.batch import SeqStep
    seqs = [SeqStep(slot=slot, start=start, tokens=[0] * x.shape[0]) for slot, start, x in pieces]
    session.cache.grow([(s.slot, s.start + s.count) for s in seqs])
    ctx, _ = session.context_for(seqs)
    out = part.forward(ctx, torch.cat([x for _, _, x in pieces]).contiguous().to(DEV),
                       ScheduleEntry(0, 0))
    if out.dim() == 3:
        out = out.sum(0)
    out = out.float().clone()
    session.cache.commit([(s.slot, s.start + s.count) for s in seqs])
    return out


# -- row-wise kernels -------------------------------------------------------------------
@pytest.mark.parametrize("width", [48, 1000, 4096])
@pytest.mark.parametrize("slices", [1, 3])
def test_norm_add_kernel(width, slices):
    from edge_infer_amd.csrc import lib
    torch.manual_seed(width + slices)
    rows = 5
    residual = torch.randn(rows, width, device=DEV)
    delta = torch.randn(slices, rows, width, device=DEV) * 3
    weight = 1 + 0.1 * torch.randn(width, device=DEV)
    expected = residual.double().cpu() + plain.rms_norm(delta.double().cpu().sum(0), weight.cpu(), 1e-3)
    low = torch.empty(rows, width, device=DEV, dtype=torch.bfloat16)
    lib.norm_add(residual, delta if slices > 1 else delta[0], weight, 1e-3, cast_out=low)
    assert_close_f32(residual, expected, "norm_add")
    assert torch.equal(low, residual.to(torch.bfloat16))
    again = residual.clone()
    lib.norm_add(again, delta[0].to(torch.bfloat16), weight, 1e-3)
    expected = residual.double().cpu() + plain.rms_norm(delta[0].to(torch.bfloat16).cpu(), weight.cpu(), 1e-3)
    assert_close_f32(again, expected, "norm_add of a bfloat16 delta")


def test_activation_kernels():
    from edge_infer_amd.csrc import lib
    x = torch.linspace(-6, 6, 1001, device=DEV).reshape(7, 143).contiguous()
    z = x.double().cpu()
    forms = {"relu2": torch.relu(z) ** 2, "relu": torch.relu(z), "silu": z / (1 + torch.exp(-z)),
             "gelu_tanh": 0.5 * z * (1 + torch.tanh((2 / torch.pi) ** 0.5 * (z + 0.044715 * z ** 3)))}
    for kind, expected in forms.items():
        out = torch.empty_like(x)
        lib.activation(x, out, kind)
        assert_close_f32(out, expected, kind)
    halves = torch.stack([x * 0.25, x * 0.75])
    out = torch.empty(7, 143, device=DEV, dtype=torch.bfloat16)
    lib.activation(halves, out, "relu2")
    assert torch.equal(out, (torch.relu(halves[0] + halves[1]) ** 2).to(torch.bfloat16))
    with pytest.raises(lib.KernelError, match="unknown kind"):
        lib.activation(x, torch.empty_like(x), "swish")


# -- attention ----------------------------------------------------------------------------
def attention_spec(**kw):
    from edge_infer_amd.config.specs import AttentionSpec, PositionSpec
    base = dict(n_heads=3, n_kv_heads=3, head_dim=32, value_dim=8, qk_norm=True, qk_norm_eps=EPS,
                qk_norm_scope="projection", qkv_bias=True, scale=1.0, chunk=50,
                distance_slope_range=8.0, sink=True, position=PositionSpec(kind="none"))
    base.update(kw)
    return AttentionSpec(**base)


def plain_attention(params, mixer, x):
    p = {"q": params["layers.0.mixer.q_proj.weight"], "k": params["layers.0.mixer.k_proj.weight"],
         "v": params["layers.0.mixer.v_proj.weight"], "o": params["layers.0.mixer.o_proj.weight"],
         "q.b": params["layers.0.mixer.q_proj.bias"], "k.b": params["layers.0.mixer.k_proj.bias"],
         "v.b": params["layers.0.mixer.v_proj.bias"],
         "q.norm": params["layers.0.mixer.q_norm.weight"],
         "k.norm": params["layers.0.mixer.k_norm.weight"], "sink": params["layers.0.mixer.sink"]}
    m = {"heads": mixer.n_heads, "kv_heads": mixer.n_kv_heads, "dim": mixer.head_dim,
         "vdim": mixer.v_dim, "scale": mixer.scale,
         "mask": None if mixer.chunk is None else {"size": mixer.chunk}}
    return plain.attention_mixer(x, p, m, mixer.qk_norm_eps)


@pytest.mark.parametrize("variant", ["narrow values", "groups of 4", "no chunk", "odd sizes"])
def test_attention_options_alone(variant):
    """Unequal sequences in one step, then a portion appended to each, then single tokens."""
    kw = {"narrow values": {}, "groups of 4": dict(n_heads=8, n_kv_heads=2, head_dim=16, value_dim=40),
          "no chunk": dict(chunk=None, n_heads=2, n_kv_heads=1, scale=0.4),
          "odd sizes": dict(n_heads=2, n_kv_heads=2, head_dim=20, value_dim=7, chunk=33)}[variant]
    mixer = attention_spec(**kw)
    spec = one_layer(mixer)
    params = params_for(spec, 3)
    model, session = session_for(spec, params)
    part = model.layers[0].mixer
    lengths = [140, 9, 66]
    torch.manual_seed(1)
    xs = [torch.randn(n, HIDDEN) for n in lengths]
    expected = [plain_attention(params, mixer, x) for x in xs]
    slots = [session.begin() for _ in lengths]
    first = [n - 6 for n in lengths]
    out = run_part(session, part, [(s, 0, x[:f]) for s, x, f in zip(slots, xs, first)])
    assert_close_f32(out, torch.cat([e[:f] for e, f in zip(expected, first)]), f"{variant}: prompts")
    out = run_part(session, part, [(s, f, x[f:f + 3]) for s, x, f in zip(slots, xs, first)])
    assert_close_f32(out, torch.cat([e[f:f + 3] for e, f in zip(expected, first)]), f"{variant}: portions")
    for t in range(3, 6):
        out = run_part(session, part, [(s, f + t, x[f + t:f + t + 1]) for s, x, f in zip(slots, xs, first)])
        assert_close_f32(out, torch.cat([e[f + t:f + t + 1] for e, f in zip(expected, first)]),
                         f"{variant}: token {t}")


@pytest.mark.parametrize("head_dim, dtype", [(32, "float32"), (64, "bfloat16"), (128, "bfloat16")])
@pytest.mark.parametrize("decoded", [False, True])
@pytest.mark.parametrize("where", ["just outside", "just inside", "far inside", "nowhere"])
def test_a_key_that_stands_out_at_a_chunks_edge(where, decoded, head_dim, dtype):
    """Query and key projections are made equal and read only the first half of an input row
    (the values read the other half), so a key whose row shares that half with the query's
    scores as high as the query's own key and far above every other (32 against a few units).
    Put just outside the query's chunk it must change nothing; just inside (37 positions
    back, which the distance term of the second head hardly lowers), or next to the query, it
    takes up to half the weight for a value of its own.  The query is the last row of a
    prompt, or a token decoded alone.  In bfloat16 with head sizes 64 and 128 the matrix-core
    kernels run (values as wide as the keys; the scale keeps the score that stands out at 32)."""
    value_dim = 8 if dtype == "float32" else head_dim
    mixer = attention_spec(n_heads=2, n_kv_heads=2, head_dim=head_dim, value_dim=value_dim,
                           chunk=50, scale=32.0 / head_dim)
    spec = one_layer(mixer)
    params = params_for(spec, 5)
    half = HIDDEN // 2
    params["layers.0.mixer.q_proj.weight"][:, half:] = 0
    params["layers.0.mixer.v_proj.weight"][:, :half] = 0
    params["layers.0.mixer.k_proj.weight"] = params["layers.0.mixer.q_proj.weight"].clone()
    params["layers.0.mixer.k_proj.bias"] = params["layers.0.mixer.q_proj.bias"].clone()
    params["layers.0.mixer.k_norm.weight"] = params["layers.0.mixer.q_norm.weight"].clone()
    model, session = session_for(spec, params, dtype)
    part = model.layers[0].mixer
    assert part.matrix_cores == (dtype == "bfloat16")
    torch.manual_seed(2)
    query = 137                                   # its chunk is 100..149
    x = torch.randn(query + 1, HIDDEN)
    plainly = plain_attention(params, mixer, x)[query]
    place = {"just outside": 99, "just inside": 100, "far inside": 136, "nowhere": None}[where]
    if place is not None:
        x[place, :half] = x[query, :half]
    expected = plain_attention(params, mixer, x)[query]
    moved = (expected - plainly).abs().max().item() / plainly.abs().max().item()
    assert (moved > 0.1) == (where in ("just inside", "far inside")), moved
    slot = session.begin()
    x = x.to(model.dtype)
    if decoded:
        run_part(session, part, [(slot, 0, x[:query])])
        out = run_part(session, part, [(slot, query, x[query:])])[0]
    else:
        out = run_part(session, part, [(slot, 0, x)])[query]
    if dtype == "float32":
        assert_close_f32(out, expected, f"key {where}")
    else:       # bfloat16 queries, keys and probabilities: a few per cent of the largest output
        error = (out.double().cpu() - expected).abs().max() / expected.abs().max()
        assert error < 0.04, f"key {where}: {error:.3f}"


def test_the_sink_and_the_slopes_count():
    """Leaving the sink out, or the distance term, would move the output by far more than the
    tolerance: the same inputs with those parameters changed give other results, and the part
    follows the oracle in each case."""
    torch.manual_seed(4)
    x = torch.randn(90, HIDDEN)
    results = []
    for sink, slope_range in ((2.0, 8.0), (-30.0, 8.0), (2.0, 64.0)):
        mixer = attention_spec(n_heads=4, n_kv_heads=2, head_dim=16, value_dim=16, chunk=64,
                               distance_slope_range=slope_range, scale=0.25)
        spec = one_layer(mixer)
        params = params_for(spec, 6)
        params["layers.0.mixer.sink"] = torch.full((4,), sink)
        model, session = session_for(spec, params)
        out = run_part(session, model.layers[0].mixer, [(session.begin(), 0, x)])
        if slope_range == 8.0:
            assert_close_f32(out, plain_attention(params, mixer, x), f"sink {sink}")
        results.append(out)
    assert (results[0] - results[1]).abs().max() > 0.05 * results[0].abs().max()
    assert (results[0] - results[2]).abs().max() > 0.05 * results[0].abs().max()


# -- gated delta rule ---------------------------------------------------------------------
def delta_spec(**kw):
    from edge_infer_amd.config.specs import GatedDeltaSpec
    base = dict(n_heads=4, n_kv_heads=2, key_dim=24, value_dim=40, conv_taps=4, out_norm_eps=EPS)
    base.update(kw)
    return GatedDeltaSpec(**base)


def plain_delta(params, mixer, x):
    names = {"q": "q_proj.weight", "k": "k_proj.weight", "v": "v_proj.weight",
             "q.conv": "q_conv.weight", "k.conv": "k_conv.weight", "v.conv": "v_conv.weight",
             "b": "beta_proj.weight", "a": "decay_proj.weight", "A_log": "decay_log_rate",
             "dt_bias": "decay_bias", "g": "gate_proj.weight", "norm": "out_norm.weight",
             "o": "o_proj.weight"}
    p = {short: params["layers.0.mixer." + long] for short, long in names.items()}
    m = {"heads": mixer.n_heads, "kv_heads": mixer.n_kv_heads, "dim": mixer.key_dim,
         "vdim": mixer.value_dim, "conv": mixer.conv_taps}
    return plain.delta_mixer(x, p, m, mixer.out_norm_eps)


@pytest.mark.parametrize("variant", ["base", "one tap", "wide keys", "odd sizes", "many taps",
                                     "ten taps", "keys of 256"])
def test_delta_rule_alone(variant):
    """Two sequences: whole prompts of unequal lengths, then portions of 2, 1 and 5 rows, then
    single tokens; the state and the convolution's tail carry over every cut."""
    kw = {"base": {}, "one tap": dict(conv_taps=1, n_heads=2, n_kv_heads=2, key_dim=8, value_dim=8),
          "wide keys": dict(key_dim=144, value_dim=12, n_heads=2, n_kv_heads=1),
          "odd sizes": dict(key_dim=13, value_dim=5, n_heads=3, n_kv_heads=1, conv_taps=2),
          "many taps": dict(conv_taps=7, key_dim=64, value_dim=64, n_heads=2, n_kv_heads=2),
          "ten taps": dict(conv_taps=10, key_dim=16, value_dim=24, n_heads=2, n_kv_heads=1),
          "keys of 256": dict(key_dim=256, value_dim=8, n_heads=1, n_kv_heads=1, conv_taps=3)}[variant]
    mixer = delta_spec(**kw)
    spec = one_layer(mixer)
    params = params_for(spec, 8)
    model, session = session_for(spec, params)
    part = model.layers[0].mixer
    lengths = [83, 21]
    torch.manual_seed(3)
    xs = [torch.randn(n, HIDDEN) for n in lengths]
    expected = [plain_delta(params, mixer, x) for x in xs]
    slots = [session.begin() for _ in lengths]
    at = [n - 12 for n in lengths]
    out = run_part(session, part, [(s, 0, x[:a]) for s, x, a in zip(slots, xs, at)])
    assert_close_f32(out, torch.cat([e[:a] for e, a in zip(expected, at)]), f"{variant}: prompts")
    for take in (2, 1, 5, 1, 1, 2):
        out = run_part(session, part, [(s, a, x[a:a + take]) for s, x, a in zip(slots, xs, at)])
        assert_close_f32(out, torch.cat([e[a:a + take] for e, a in zip(expected, at)]),
                         f"{variant}: {take} rows at {at}")
        at = [a + take for a in at]
    assert at == lengths


def test_delta_rule_from_the_first_token_and_in_a_slot_used_again():
    """Single tokens from position 0 (the convolution sees zeros before the start), then the
    slot is given back and taken again: the new sequence starts from an empty state."""
    mixer = delta_spec()
    spec = one_layer(mixer)
    params = params_for(spec, 9)
    model, session = session_for(spec, params, max_seqs=1)
    part = model.layers[0].mixer
    torch.manual_seed(5)
    for trial in range(2):
        x = torch.randn(9, HIDDEN)
        expected = plain_delta(params, mixer, x)
        slot = session.begin()
        assert slot == 0
        rows = [run_part(session, part, [(slot, t, x[t:t + 1])]) for t in range(9)]
        assert_close_f32(torch.cat(rows), expected, f"trial {trial}")
        session.end(slot)


def test_delta_rule_keeps_what_was_written_long_ago():
    """With almost no decay, what the third token wrote is still read 150 tokens later (every
    later write takes a little of it away, which is the rule's nature): the output at the end
    differs by far more than the tolerance between two inputs that differ in row 2 alone."""
    mixer = delta_spec(n_heads=2, n_kv_heads=2, key_dim=32, value_dim=16)
    spec = one_layer(mixer)
    params = params_for(spec, 10)
    params["layers.0.mixer.decay_log_rate"] = torch.full((2,), -9.0)
    model, session = session_for(spec, params)
    part = model.layers[0].mixer
    torch.manual_seed(6)
    x = torch.randn(153, HIDDEN)
    other = x.clone()
    other[2] = torch.randn(HIDDEN)
    ends = []
    for rows in (x, other):
        expected = plain_delta(params, mixer, rows)
        slot = session.begin()
        run_part(session, part, [(slot, 0, rows[:70])])
        out = run_part(session, part, [(slot, 70, rows[70:])])
        assert_close_f32(out, expected[70:], "far write")
        ends.append(expected[-1])
        session.end(slot)
    assert (ends[0] - ends[1]).abs().max() > 0.01 * ends[0].abs().max()


# -- feed-forward and block --------------------------------------------------------------
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("with_ffn", [True, False])
def test_block_norms_its_sublayers_outputs(dtype, with_ffn):
    """x + norm1(mixer(x)), then x + norm2(ff(x)), on a model of one layer; a layer without a
    feed-forward has no second norm."""
    from edge_infer_amd.config.specs import DenseMLPSpec
    mixer = delta_spec(n_heads=2, n_kv_heads=1, key_dim=16, value_dim=16, conv_taps=3)
    spec = one_layer(mixer, DenseMLPSpec(intermediate_size=72) if with_ffn else None)
    params = params_for(spec, 11)
    assert ("layers.0.norm2.weight" in params) == with_ffn
    model, session = session_for(spec, params, dtype)
    tokens = [3, 30, 7, 7, 12, 0, 19, 4]
    x = params["embed.weight"][tokens].double()
    p = "layers.0."
    x = x + plain.rms_norm(plain_delta(params, mixer, x), params[p + "norm1.weight"], EPS)
    if with_ffn:
        ff = plain.dense_feed_forward(x, {"up": params[p + "ffn.up_proj.weight"],
                                          "down": params[p + "ffn.down_proj.weight"]})
        x = x + plain.rms_norm(ff, params[p + "norm2.weight"], EPS)
    expected = plain.linear(plain.rms_norm(x, params["final_norm.weight"], EPS), params["head.weight"])
    slot = session.begin()
    logits = session.step([(slot, tokens[:5], list(range(5)))])
    logits = torch.cat([logits, session.step([(slot, tokens[5:], [0, 1, 2])])])
    if dtype == "float32":
        assert_close_f32(logits, expected, "block")
    else:
        error = (logits.double().cpu() - expected).abs().max() / expected.abs().max()
        assert error < 0.03, error
