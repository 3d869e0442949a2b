"""The mechanisms of the Zadenex layers alone, each against its plain function: the row-wise
kernels (the fused norm-add-norm, the two streams side by side, the stream made anew, the
gated gelu, the scaled embedding), the per-head kernels (one matrix a head, the rotation of
neighbouring pairs, queries mixed over heads), attention whose scores are mixed over heads
with keys made to stand out just inside and just outside the window, latent attention with a
far key made to stand out and a sink that weighs, and the matrix memory in portions, token by
token, in batches and with slots used again."""
import math

import pytest
import torch

import plain_zadenex as plain
from helpers import assert_close_bf16, assert_close_f32

pytestmark = pytest.mark.gpu
DEV = "cuda"
HIDDEN, VOCAB, EPS = 48, 31, 1e-5


def one_layer(mixer, ffn=None, scale=1.0):
    from edge_infer_amd.config.specs import LayerSpec, ModelSpec, NormSpec, default_schedule
    norm = NormSpec(eps=EPS)
    return ModelSpec(architecture="test", vocab_size=VOCAB, hidden_size=HIDDEN,
                     layers=(LayerSpec(block="sandwich", norm=norm, mixer=mixer, feed_forward=ffn,
                                       residual_scale=scale),),
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
        elif param.init == "near_identity":
            value = torch.eye(*shape) + 0.3 * torch.randn(shape, generator=g)
        elif len(shape) == 2:
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


def mixer_tensors(params):
    pre = "layers.0.mixer."
    return {k[len(pre):]: v for k, v in params.items() if k.startswith(pre)}


def in_cuts(session, part, x, cuts, slot=None):
    """The rows of `x` through the part in steps of the given sizes, as one sequence."""
    own = slot is None
    slot = session.begin() if own else slot
    rows, at = [], 0
    for take in cuts:
        rows.append(run_part(session, part, [(slot, at, x[at:at + take])]))
        at += take
    assert at == x.shape[0]
    if own:
        session.end(slot)
    return torch.cat(rows)


# -- row-wise kernels -------------------------------------------------------------------
@pytest.mark.parametrize("width", [48, 1000, 4100])
@pytest.mark.parametrize("slices", [1, 3])
def test_norm_add_norm_kernel(width, slices):
    from edge_infer_amd.csrc import lib
    torch.manual_seed(width + slices)
    rows = 5
    residual = torch.randn(rows, width, device=DEV)
    delta = torch.randn(slices, rows, width, device=DEV) * 3
    after = 0.3 * (1 + 0.1 * torch.randn(width, device=DEV))
    ahead = 1 + 0.1 * torch.randn(width, device=DEV)
    stream = residual.double().cpu() + plain.rms_norm(delta.double().cpu().sum(0), after.cpu(), 1e-3)
    out = torch.empty(rows, width, device=DEV)
    lib.norm_add_norm(residual, delta if slices > 1 else delta[0], after, ahead, 1e-3, out)
    assert_close_f32(residual, stream, "norm_add_norm: the stream")
    assert_close_f32(out, plain.rms_norm(stream, ahead.cpu(), 1e-3), "norm_add_norm: the normed rows")
    low = torch.empty(rows, width, device=DEV, dtype=torch.bfloat16)
    again = residual.clone()
    lib.norm_add_norm(again, delta[0].to(torch.bfloat16), after, ahead, 1e-3, low)
    stream = residual.double().cpu() + plain.rms_norm(delta[0].to(torch.bfloat16).cpu(), after.cpu(), 1e-3)
    assert_close_f32(again, stream, "norm_add_norm of a bfloat16 delta")
    assert_close_bf16(low, plain.rms_norm(stream, ahead.cpu(), 1e-3), "bfloat16 rows",
                      rms_rel=4e-3, max_rel=8e-3)


def test_streams_side_by_side_and_the_stream_made_anew():
    from edge_infer_amd.csrc import lib
    torch.manual_seed(2)
    a, b = torch.randn(7, 40, device=DEV), torch.randn(7, 40, device=DEV)
    for dtype in (torch.float32, torch.bfloat16):
        both = torch.empty(7, 80, device=DEV, dtype=dtype)
        lib.concat_cast(a, b, both)
        assert torch.equal(both, torch.cat([a, b], dim=1).to(dtype))
    slices = torch.randn(3, 7, 40, device=DEV)
    vector = torch.randn(40, device=DEV)
    out = torch.full((7, 40), 9.0, device=DEV)
    lib.set_rows(slices, out, vector)
    assert_close_f32(out, slices.double().cpu().sum(0) + vector.double().cpu(), "set_rows")
    low = slices[0].to(torch.bfloat16)
    lib.set_rows(low, out)
    assert torch.equal(out, low.float())


def test_gated_gelu_and_scaled_embedding():
    from edge_infer_amd.csrc import lib
    torch.manual_seed(3)
    gate_up = torch.randn(2, 6, 64, device=DEV) * 2
    out = torch.empty(6, 32, device=DEV)
    lib.swiglu(gate_up, out, 0, "gelu_tanh")
    both = gate_up.double().cpu().sum(0)
    assert_close_f32(out, plain.gelu_tanh(both[:, :32]) * both[:, 32:], "gated gelu")
    strips = torch.empty(6, 32, device=DEV)
    lib.swiglu(gate_up, strips, 16, "gelu_tanh")
    g = torch.cat([both[:, 0:16], both[:, 32:48]], dim=1)
    u = torch.cat([both[:, 16:32], both[:, 48:64]], dim=1)
    assert_close_f32(strips, plain.gelu_tanh(g) * u, "gated gelu in strips")
    with pytest.raises(lib.KernelError, match="unknown gate activation"):
        lib.swiglu(gate_up, out, 0, "swish")
    table = torch.randn(11, 24, device=DEV).to(torch.bfloat16)
    tokens = torch.tensor([3, 0, 10, 3], device=DEV, dtype=torch.int32)
    rows = torch.empty(4, 24, device=DEV)
    lib.embed_gather(tokens, table, rows, 2.5)
    assert torch.equal(rows, table.float()[tokens.long()] * 2.5)


# -- per-head kernels ----------------------------------------------------------------------
@pytest.mark.parametrize("rows, heads, k, j", [(1, 3, 16, 40), (37, 5, 130, 7), (300, 2, 8, 300)])
def test_one_matrix_a_head(rows, heads, k, j):
    from edge_infer_amd.csrc import lib
    torch.manual_seed(rows)
    x_head, y_head = k + 5, j + 3           # a head's part lies inside a wider row
    x = torch.randn(rows, heads * x_head, device=DEV)
    m = (torch.randn(heads, k, j, device=DEV) / k ** 0.5)
    y = torch.zeros(rows, heads * y_head, device=DEV)
    lib.head_matmul(x, m, y, heads, x_head=x_head, x_first=2, y_head=y_head, y_first=1)
    xs = x.double().cpu().reshape(rows, heads, x_head)[:, :, 2:2 + k]
    want = torch.einsum("nhk,hkj->nhj", xs, m.double().cpu())
    got = y.reshape(rows, heads, y_head)
    assert_close_f32(got[:, :, 1:1 + j], want, "head_matmul")
    assert torch.count_nonzero(got[:, :, 0]) == 0 and torch.count_nonzero(got[:, :, 1 + j:]) == 0
    # float32 slices in, bfloat16 matrices and rows out
    halves = torch.stack([x * 0.25, x * 0.75])
    low = torch.zeros(rows, heads * y_head, device=DEV, dtype=torch.bfloat16)
    lib.head_matmul(halves, m.to(torch.bfloat16), low, heads, x_head=x_head, x_first=2,
                    y_head=y_head, y_first=1)
    want = torch.einsum("nhk,hkj->nhj", xs, m.to(torch.bfloat16).double().cpu())
    assert_close_bf16(low.reshape(rows, heads, y_head)[:, :, 1:1 + j], want, "head_matmul bfloat16",
                      rms_rel=4e-3, max_rel=8e-3)


def test_rotation_of_neighbouring_pairs():
    from edge_infer_amd.csrc import lib
    from edge_infer_amd.config.specs import PositionSpec
    from edge_infer_amd.parts.rope import RotaryFrequencies
    torch.manual_seed(4)
    heads, rot, head = 3, 6, 11
    freq = RotaryFrequencies(PositionSpec(kind="rope_pairs", theta=500.0, dim=rot), DEV).frequencies
    positions = torch.tensor([0, 1, 63, 64, 5000, 123456], device=DEV, dtype=torch.int32)
    x = torch.randn(6, heads * head, device=DEV)
    y = torch.zeros(6, heads * rot, device=DEV)
    lib.rotate_pairs(x, freq, positions, y, heads, rot, x_head=head, x_first=4, y_head=rot, y_first=0)
    part = x.double().cpu().reshape(6, heads, head)[:, :, 4:4 + rot]
    want = plain.rotate_neighbours(part, positions.cpu(), 500.0, rot)
    # the angle of position 123456 is a float32 product: 2^-24 of it is what the cosine may be off
    err = (y.double().cpu().reshape(6, heads, rot) - want).abs().amax(dim=(1, 2))
    assert (err[:4] < 1e-6).all() and err[4] < 1e-3 and err[5] < 2e-2, err


# -- attention with scores mixed over heads ----------------------------------------------
def talking_spec(**kw):
    from edge_infer_amd.config.specs import AttentionSpec, PositionSpec
    base = dict(n_heads=6, n_kv_heads=2, head_dim=16, value_dim=8, qk_norm=False, qkv_bias=True,
                o_bias=True, scale=0.3, window=21, unit_sink=True, talking_heads=True,
                position=PositionSpec(kind="none"))
    base.update(kw)
    return AttentionSpec(**base)


def plain_talking(params, mixer, x):
    t = mixer_tensors(params)
    p = {"q": t["q_proj.weight"], "q.b": t["q_proj.bias"], "k": t["k_proj.weight"],
         "k.b": t["k_proj.bias"], "v": t["v_proj.weight"], "v.b": t["v_proj.bias"],
         "talk": t["talk"], "o": t["o_proj.weight"], "o.b": t["o_proj.bias"]}
    m = {"heads": mixer.n_heads, "kv_heads": mixer.n_kv_heads, "dim": mixer.head_dim,
         "vdim": mixer.v_dim, "scale": mixer.scale,
         "mask": None if mixer.window is None else {"size": mixer.window}}
    return plain.talking_attention_mixer(x, p, m)


@pytest.mark.parametrize("mixer", [
    talking_spec(), talking_spec(n_heads=4, n_kv_heads=4, head_dim=24, value_dim=40, window=64),
    talking_spec(n_heads=8, n_kv_heads=1, head_dim=8, value_dim=8, window=65),
    talking_spec(n_heads=2, n_kv_heads=2, head_dim=64, value_dim=64, window=None),
    talking_spec(n_heads=20, n_kv_heads=5, head_dim=16, value_dim=4, window=1),
    talking_spec(n_heads=3, n_kv_heads=1, head_dim=40, value_dim=3, window=130),
    # sizes that the matrix-core kernel for wide keys takes in bfloat16: groups of 3, 4 and 1
    talking_spec(n_heads=6, n_kv_heads=2, head_dim=16, value_dim=16, window=21),
    talking_spec(n_heads=16, n_kv_heads=4, head_dim=32, value_dim=48, window=70),
    talking_spec(n_heads=5, n_kv_heads=5, head_dim=32, value_dim=32, window=None)])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_talking_attention_alone(mixer, dtype):
    """Whole, in portions and token by token, over the window's edge and two page borders."""
    spec = one_layer(mixer)
    params = params_for(spec, seed=7)
    model, session = session_for(spec, params, dtype)
    part = model.layers[0].mixer
    torch.manual_seed(5)
    x = torch.randn(150, HIDDEN).to(torch.bfloat16).float()
    want = plain_talking(params, mixer, x.double())
    feed = x.to(model.dtype)
    for cuts in ([150], [60, 2, 3, 64, 21], [100] + [1] * 50):
        got = in_cuts(session, part, feed, cuts)
        if dtype == "float32":
            assert_close_f32(got, want, f"talking attention {cuts[:3]}")
        else:
            assert_close_bf16(got, want, f"talking attention {cuts[:3]}", rms_rel=2e-2, max_rel=4e-2)
    session.cache.check()


@pytest.mark.parametrize("window", [5, 64, 65, 100])
def test_keys_that_stand_out_at_the_windows_edge(window):
    """The key just outside the window of the last position is made to dominate (its input is
    a multiple of the query's, and the keys are made with the queries' matrix, so its score is
    a large positive number): the engine must not see it.  Then the key just inside."""
    mixer = talking_spec(n_heads=2, n_kv_heads=2, head_dim=16, value_dim=8, window=window, scale=0.5)
    spec = one_layer(mixer)
    params = params_for(spec, seed=9)
    pre = "layers.0.mixer."
    params[pre + "k_proj.weight"] = params[pre + "q_proj.weight"].clone()
    params[pre + "q_proj.bias"].zero_()
    params[pre + "k_proj.bias"].zero_()
    params[pre + "talk"] = torch.eye(2)
    model, session = session_for(spec, params)
    part = model.layers[0].mixer
    torch.manual_seed(6)
    T = 180
    base = (0.3 * torch.randn(T, HIDDEN)).to(torch.bfloat16).float()
    for offset, seen in ((window, False), (window - 1, True)):
        x = base.clone()
        x[T - 1 - offset] = 4.0 * x[T - 1] / 0.3
        x[T - 1] = x[T - 1] / 0.3
        x = x.to(torch.bfloat16).float()
        want = plain_talking(params, mixer, x.double())
        calm = x.clone()
        calm[T - 1 - offset] = base[T - 1 - offset]
        quiet = plain_talking(params, mixer, calm.double())
        moved = (want[-1] - quiet[-1]).abs().max().item() / want[-1].abs().max().item()
        assert (moved > 0.1) == seen, f"the test's key does not stand out as meant ({moved:.2e})"
        for cuts in ([T], [T - 1, 1], [T - offset - 1, 1, offset], [T - 30] + [1] * 30):
            got = in_cuts(session, part, x, cuts)
            assert_close_f32(got, want, f"window {window}, key at distance {offset}, cuts {cuts[:3]}")


# -- latent attention -----------------------------------------------------------------------
def latent_spec(**kw):
    from edge_infer_amd.config.specs import LatentAttentionSpec, PositionSpec
    base = dict(n_heads=3, head_dim=16, rot_dim=8, value_dim=24, kv_rank=40, q_rank=24, scale=0.25,
                norm_eps=EPS, sink=True, output_gate=True)
    base.update(kw)
    base["position"] = PositionSpec(kind="rope_pairs", theta=base.pop("theta", 10000.0),
                                    dim=base["rot_dim"])
    return LatentAttentionSpec(**base)


def plain_latent(params, mixer, x):
    t = mixer_tensors(params)
    p = {"dq": t["q_down.weight"], "dq.norm": t["q_down_norm.weight"], "uq": t["q_up.weight"],
         "dkv": t["kv_down.weight"], "dkv.norm": t["kv_down_norm.weight"], "uk": t["k_up.weight"],
         "uv": t["v_up.weight"], "sink": t["sink"], "g": t["gate_proj.weight"],
         "o": t["o_proj.weight"]}
    m = {"heads": mixer.n_heads, "dim": mixer.head_dim, "rot_dim": mixer.rot_dim,
         "vdim": mixer.value_dim, "kv_rank": mixer.kv_rank, "scale": mixer.scale,
         "rot": {"base": mixer.position.theta, "dims": mixer.rot_dim}}
    return plain.latent_attention_mixer(x, p, m, EPS)


@pytest.mark.parametrize("mixer", [
    latent_spec(), latent_spec(n_heads=1, head_dim=32, rot_dim=16, value_dim=40, kv_rank=24, q_rank=56),
    latent_spec(n_heads=20, head_dim=8, rot_dim=2, value_dim=8, kv_rank=72, q_rank=16, theta=500.0),
    latent_spec(n_heads=5, head_dim=24, rot_dim=32, value_dim=12, kv_rank=264, q_rank=40, scale=0.1),
    # cache rows that the matrix-core kernel for wide keys takes in bfloat16; 3, 20 and 70 heads
    latent_spec(kv_rank=48, rot_dim=16),
    latent_spec(n_heads=20, head_dim=8, rot_dim=32, value_dim=8, kv_rank=96, q_rank=16),
    latent_spec(n_heads=70, head_dim=8, rot_dim=32, value_dim=4, kv_rank=32, q_rank=32)])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_latent_attention_alone(mixer, dtype):
    spec = one_layer(mixer)
    params = params_for(spec, seed=11)
    params["layers.0.mixer.sink"][0] = 3.0          # a sink that outweighs the first keys
    model, session = session_for(spec, params, dtype)
    part = model.layers[0].mixer
    assert part.wide == (dtype == "bfloat16" and mixer.cache_width % 32 == 0 and mixer.kv_rank % 16 == 0)
    torch.manual_seed(8)
    x = torch.randn(150, HIDDEN).to(torch.bfloat16).float()
    want = plain_latent(params, mixer, x.double())
    feed = x.to(model.dtype)
    for cuts in ([150], [60, 2, 3, 64, 21], [100] + [1] * 50):
        got = in_cuts(session, part, feed, cuts)
        if dtype == "float32":
            assert_close_f32(got, want, f"latent attention {cuts[:3]}")
        else:
            assert_close_bf16(got, want, f"latent attention {cuts[:3]}", rms_rel=2e-2, max_rel=5e-2)
    session.cache.check()


def test_a_far_key_among_hundreds_and_the_sink():
    """Position 3 of 700 repeats the last position's input, the rotation is slow and the scale
    large, so that key takes a weight that shows; with the sink left out, or the far key, the
    oracle's own output moves by much more than the tolerance."""
    mixer = latent_spec(n_heads=2, head_dim=16, rot_dim=4, value_dim=16, kv_rank=32, q_rank=32,
                        scale=0.6, theta=1e8)
    spec = one_layer(mixer)
    params = params_for(spec, seed=13)
    pre = "layers.0.mixer."
    # keys made with the queries' matrices: a position's key is aligned with its own query
    rank, d, r = 32, 16, 4
    params[pre + "kv_down.weight"][:rank] = params[pre + "q_down.weight"]
    params[pre + "kv_down_norm.weight"] = params[pre + "q_down_norm.weight"].clone()
    up = params[pre + "q_up.weight"].reshape(2, d + r, rank)[:, :d]
    params[pre + "k_up.weight"] = up.reshape(2 * d, rank).clone()
    params[pre + "sink"] = torch.tensor([10.0, 10.0])
    model, session = session_for(spec, params, max_tokens=1024)
    part = model.layers[0].mixer
    torch.manual_seed(10)
    T = 700
    x = torch.randn(T, HIDDEN).to(torch.bfloat16).float()
    x[3] = x[T - 1]
    want = plain_latent(params, mixer, x.double())
    other = x.clone()
    other[3] = x[4]
    moved = (plain_latent(params, mixer, other.double())[-1] - want[-1]).abs().max() / want[-1].abs().max()
    assert moved > 0.05, f"the far key does not show ({moved:.2e})"
    no_sink = dict(params)
    no_sink[pre + "sink"] = torch.tensor([-30.0, -30.0])
    moved = (plain_latent(no_sink, mixer, x.double())[-1] - want[-1]).abs().max() / want[-1].abs().max()
    assert moved > 0.05, f"the sink does not show ({moved:.2e})"
    for cuts in ([T], [T - 1, 1], [2, 2, 300, T - 304 - 40] + [1] * 40):
        got = in_cuts(session, part, x, cuts)
        assert_close_f32(got, want, f"far key, cuts {cuts[:4]}")


# -- matrix memory --------------------------------------------------------------------------
def memory_spec(**kw):
    from edge_infer_amd.config.specs import MatrixMemorySpec
    base = dict(n_heads=3, key_dim=24, value_dim=16, gate_cap=10.0, out_norm_eps=EPS)
    base.update(kw)
    return MatrixMemorySpec(**base)


def plain_memory(params, mixer, x):
    t = mixer_tensors(params)
    p = {"q": t["q_proj.weight"], "k": t["k_proj.weight"], "v": t["v_proj.weight"],
         "i": t["in_gate.weight"], "i.b": t["in_gate.bias"], "f": t["forget_gate.weight"],
         "f.b": t["forget_gate.bias"], "g": t["gate_proj.weight"], "norm": t["out_norm.weight"],
         "o": t["o_proj.weight"]}
    m = {"heads": mixer.n_heads, "dim": mixer.key_dim, "vdim": mixer.value_dim,
         "gate_cap": mixer.gate_cap}
    return plain.mlstm_mixer(x, p, m, EPS)


@pytest.mark.parametrize("mixer", [
    memory_spec(), memory_spec(n_heads=1, key_dim=100, value_dim=70, gate_cap=15.0),
    memory_spec(n_heads=2, key_dim=256, value_dim=8, gate_cap=2.0),
    memory_spec(n_heads=4, key_dim=7, value_dim=130, gate_cap=30.0),
    memory_spec(n_heads=2, key_dim=8, value_dim=1)])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_matrix_memory_alone(mixer, dtype):
    """Whole, in portions down to two tokens and one (tiles of 16 tokens are cut everywhere),
    and token by token: the state is carried."""
    spec = one_layer(mixer)
    params = params_for(spec, seed=15)
    params["layers.0.mixer.in_gate.weight"] *= 6.0       # log input gates that reach the cap
    model, session = session_for(spec, params, dtype)
    part = model.layers[0].mixer
    torch.manual_seed(12)
    x = torch.randn(120, HIDDEN).to(torch.bfloat16).float()
    want = plain_memory(params, mixer, x.double())
    feed = x.to(model.dtype)
    for cuts in ([120], [2, 2, 1, 16, 17, 31, 51], [70] + [1] * 50):
        got = in_cuts(session, part, feed, cuts)
        if dtype == "float32":
            assert_close_f32(got, want, f"matrix memory {cuts[:3]}")
        else:
            assert_close_bf16(got, want, f"matrix memory {cuts[:3]}", rms_rel=2e-2, max_rel=5e-2)


def test_matrix_memory_in_batches_with_slots_used_again():
    """Three sequences of unequal lengths side by side, each equal to itself alone; a slot that
    is taken again starts from a zero state although its rows hold the last owner's."""
    mixer = memory_spec(n_heads=2, key_dim=40, value_dim=24)
    spec = one_layer(mixer)
    params = params_for(spec, seed=17)
    model, session = session_for(spec, params, max_seqs=3)
    part = model.layers[0].mixer
    torch.manual_seed(14)
    xs = [torch.randn(n, HIDDEN).to(torch.bfloat16).float() for n in (50, 1, 33)]
    wants = [plain_memory(params, mixer, x.double()) for x in xs]
    for _ in range(3):          # the same slots again and again
        slots = [session.begin() for _ in xs]
        first = run_part(session, part, [(s, 0, x[:max(1, len(x) - 10)]) for s, x in zip(slots, xs)])
        at = 0
        for x, want in zip(xs, wants):
            n = max(1, len(x) - 10)
            assert_close_f32(first[at:at + n], want[:n], "batched prompt")
            at += n
        for t in range(10):
            live = [(s, len(x) - 10 + t, x[len(x) - 10 + t:len(x) - 9 + t]) for s, x in zip(slots, xs)
                    if len(x) > 10]
            rows = run_part(session, part, live)
            for row, (x, want) in enumerate([(x, w) for x, w in zip(xs, wants) if len(x) > 10]):
                assert_close_f32(rows[row:row + 1], want[len(x) - 10 + t:len(x) - 9 + t], "batched token")
        for s in slots:
            session.end(s)


def test_the_running_maximum_starts_at_zero():
    """A first token whose log input gate is far below zero: with m_0 = 0 the read-out's floor
    e^(-m) is 1, with m_0 = -inf it would be e^(-i), and the output would differ by orders of
    magnitude."""
    mixer = memory_spec(n_heads=1, key_dim=8, value_dim=8, gate_cap=20.0)
    spec = one_layer(mixer)
    params = params_for(spec, seed=19)
    params["layers.0.mixer.in_gate.bias"] = torch.tensor([-12.0])
    params["layers.0.mixer.in_gate.weight"].zero_()
    model, session = session_for(spec, params)
    torch.manual_seed(16)
    x = torch.randn(3, HIDDEN).to(torch.bfloat16).float()
    want = plain_memory(params, mixer, x.double())
    got = in_cuts(session, model.layers[0].mixer, x, [1, 1, 1])
    assert_close_f32(got, want, "first tokens")
    assert math.isfinite(got.abs().max().item())


# -- the block and the loop -------------------------------------------------------------------
def test_sandwich_block_with_a_multiplier_and_the_gated_feed_forward():
    from edge_infer_amd.config.specs import GatedMLPSpec
    import edge_infer_amd as ei
    mixer = memory_spec(n_heads=2, key_dim=16, value_dim=24)
    spec = one_layer(mixer, GatedMLPSpec(intermediate_size=72, activation="gelu_tanh", bias=True),
                     scale=0.35)
    params = params_for(spec, seed=21)
    model, session = session_for(spec, params)
    tokens = [3, 30, 0, 7, 7, 12, 1, 29, 4]
    slot = session.begin()
    got = session.step([(slot, tokens, list(range(len(tokens))))])
    # the oracle's own layer on the same numbers
    names = {"norm1": "l0.norm1", "norm1b": "l0.norm1b", "norm2": "l0.norm2", "norm2b": "l0.norm2b"}
    tensors = {"embed": params["embed.weight"], "final.norm": params["final_norm.weight"],
               "head": params["head.weight"]}
    for part, name in names.items():
        tensors[name] = params[f"layers.0.{part}.weight"]
    t = mixer_tensors(params)
    for ours, theirs in (("q_proj.weight", "q"), ("k_proj.weight", "k"), ("v_proj.weight", "v"),
                         ("in_gate.weight", "i"), ("in_gate.bias", "i.b"), ("forget_gate.weight", "f"),
                         ("forget_gate.bias", "f.b"), ("gate_proj.weight", "g"),
                         ("out_norm.weight", "norm"), ("o_proj.weight", "o")):
        tensors["l0.mix." + theirs] = t[ours]
    for ours, theirs in (("gate_proj", "gate"), ("up_proj", "up"), ("down_proj", "down")):
        tensors[f"l0.mlp.{theirs}"] = params[f"layers.0.ffn.{ours}.weight"]
        tensors[f"l0.mlp.{theirs}.b"] = params[f"layers.0.ffn.{ours}.bias"]
    cfg = {"vocab": VOCAB, "width": HIDDEN, "norm": {"eps": EPS}, "embedding": {"scale": 1.0},
           "residual_mult": 0.35, "loop": None,
           "layers": [{"type": "mlstm", "mixer": {"heads": 2, "dim": 16, "vdim": 24, "gate_cap": 10.0},
                       "mlp": {"kind": "dense", "ff": 72}}]}
    assert_close_f32(got, plain.forward(cfg, tensors, tokens), "one sandwich layer")
