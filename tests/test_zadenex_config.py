"""Zadenex without a GPU: the configuration reader, the checkpoint's names, the schedule of a
loop, what the cache is asked for, pages given back behind a window, and the oracle's own
mechanisms against closed forms."""
import copy
import math

import pytest
import torch

import plain_zadenex as plain
from zadenex_helpers import CONFIGS, sharp_weights, tensor_shapes

NAMES = sorted(CONFIGS)


def config(name):
    from edge_infer_amd.config import ZadenexConfig
    return ZadenexConfig.from_dict(CONFIGS[name])


@pytest.mark.parametrize("name", NAMES)
def test_config_round_trip_and_registry(name, tmp_path):
    import json
    from edge_infer_amd.config import ZadenexConfig, read_config, resolve_architecture
    cfg = config(name)
    assert ZadenexConfig.from_dict(cfg.to_dict()) == cfg
    assert resolve_architecture(CONFIGS[name]).config_class is ZadenexConfig
    (tmp_path / "config.json").write_text(json.dumps(CONFIGS[name]))
    entry, read, _ = read_config(tmp_path)
    assert read == cfg and entry.name == "Zadenex"


@pytest.mark.parametrize("name", NAMES)
def test_spec_takes_every_size_from_the_configuration(name):
    from edge_infer_amd.config.specs import AttentionSpec, LatentAttentionSpec, MatrixMemorySpec
    raw = CONFIGS[name]
    spec = config(name).model_spec()
    assert (spec.vocab_size, spec.hidden_size) == (raw["vocab"], raw["width"])
    assert spec.embedding_scale == raw["embedding"]["scale"]
    assert spec.final_norm.eps == raw["norm"]["eps"] and len(spec.layers) == len(raw["layers"])
    for layer, source in zip(spec.layers, raw["layers"]):
        m, mixer = source["mixer"], layer.mixer
        assert layer.block == "sandwich" and layer.norm.eps == raw["norm"]["eps"]
        assert layer.residual_scale == raw["residual_mult"]
        if source["type"] == "mlstm":
            assert isinstance(mixer, MatrixMemorySpec)
            assert (mixer.n_heads, mixer.key_dim, mixer.value_dim, mixer.gate_cap) == \
                (m["heads"], m["dim"], m["vdim"], m["gate_cap"])
            assert mixer.out_norm_eps == raw["norm"]["eps"] and mixer.bottom_eps == 1e-6
        elif source["type"] == "latent_attention":
            assert isinstance(mixer, LatentAttentionSpec)
            assert (mixer.n_heads, mixer.head_dim, mixer.rot_dim, mixer.value_dim, mixer.kv_rank,
                    mixer.q_rank, mixer.scale) == \
                (m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"], m["q_rank"], m["scale"])
            assert (mixer.position.kind, mixer.position.theta, mixer.position.dim) == \
                ("rope_pairs", m["rot"]["base"], m["rot"]["dims"])
            assert mixer.sink and mixer.output_gate and mixer.norm_eps == raw["norm"]["eps"]
        else:
            assert isinstance(mixer, AttentionSpec)
            assert (mixer.n_heads, mixer.n_kv_heads, mixer.head_dim, mixer.v_dim, mixer.scale) == \
                (m["heads"], m["kv_heads"], m["dim"], m["vdim"], m["scale"])
            assert mixer.window == (m.get("mask") or {}).get("size")
            assert mixer.talking_heads and mixer.unit_sink and not mixer.sink
            assert mixer.qkv_bias is True and mixer.o_bias is True and not mixer.qk_norm
            assert mixer.position.kind == "none" and mixer.chunk is None
        if source["mlp"] is None:
            assert layer.feed_forward is None
        else:
            assert layer.feed_forward.kind == "gated_mlp"
            assert layer.feed_forward.intermediate_size == source["mlp"]["ff"]
            assert layer.feed_forward.activation == "gelu_tanh" and layer.feed_forward.bias is True


@pytest.mark.parametrize("name", NAMES)
def test_schedule_of_the_loop(name):
    """The looped layers run `times` times in a row, every run with a cache entry of its own;
    the oracle's order of runs is the same."""
    spec = config(name).model_spec()
    runs = plain.layer_runs(CONFIGS[name])
    assert [entry.layer for entry in spec.schedule] == [layer for layer, _ in runs]
    assert [entry.cache for entry in spec.schedule] == list(range(len(runs)))
    assert all(entry.writes_cache for entry in spec.schedule)
    from edge_infer_amd.config.specs import pass_starts
    loop = CONFIGS[name]["loop"]
    if loop is None:
        assert spec.loop is None
    else:
        starts = pass_starts(len(spec.layers), spec.loop)
        assert [runs[run] for run in starts] == [(loop["start"], t) for t in range(loop["times"])]


@pytest.mark.parametrize("name", NAMES)
def test_checkpoint_names_and_shapes(name):
    from edge_infer_amd.engine.model import expected_parameters
    cfg = config(name)
    expected = expected_parameters(cfg.model_spec(), cfg.checkpoint_name)
    named = {tensor: (tuple(param.shape), param.optional) for tensor, param in expected.values()}
    shapes = {tensor: shape for tensor, (shape, _) in tensor_shapes(CONFIGS[name]).items()}
    required = {tensor for tensor, (_, optional) in named.items() if not optional}
    assert required <= set(shapes) and set(shapes) <= set(named)
    for tensor in shapes:
        assert named[tensor][0] == tuple(shapes[tensor]), tensor


def test_the_loader_matches_a_written_folder(tmp_path):
    """Tensors by name through the framework's own reader and matcher; a missing and a
    misshapen tensor are both reported."""
    from edge_infer_amd.engine.model import expected_parameters
    from edge_infer_amd.weights import WeightsError, match_parameters, read_tensors
    from zadenex_helpers import write_folder
    cfg = config("A")
    tensors = sharp_weights(CONFIGS["A"], seed=1)
    folder = write_folder(tmp_path / "a", CONFIGS["A"], tensors)
    expected = expected_parameters(cfg.model_spec(), cfg.checkpoint_name)
    params = match_parameters(expected, read_tensors(folder))
    assert torch.equal(params["layers.1.mixer.k_up.weight"], tensors["l1.mix.uk"])
    assert torch.equal(params["loop.step"], tensors["loop.step"])
    broken = dict(tensors)
    del broken["l2.mix.f.b"]
    broken["l0.mix.talk"] = torch.zeros(5, 5, dtype=torch.bfloat16)
    with pytest.raises(WeightsError) as caught:
        match_parameters(expected, broken)
    assert "l2.mix.f.b" in caught.value.missing
    assert [entry[0] for entry in caught.value.wrong_shape] == ["l0.mix.talk"]


@pytest.mark.parametrize("change, message", [
    (lambda c: c["layers"][0]["mixer"].update(extra=1), "does not know"),
    (lambda c: c["layers"][0].update(type="conv"), "must be one of"),
    (lambda c: c["layers"][1]["mixer"]["rot"].update(dims=4), "rot.dims must equal rot_dim"),
    (lambda c: c["loop"].update(stop=9), "loop.start < loop.stop"),
    (lambda c: c.pop("residual_mult"), "lacks 'residual_mult'"),
    (lambda c: c["embedding"].update(scale=-1.0), "positive number"),
    (lambda c: c["layers"][0]["mlp"].update(kind="routed"), "must be 'dense'"),
    (lambda c: c["layers"][0]["mixer"].update(heads=7), "multiple of kv_heads"),
])
def test_what_the_decoder_does_not_know_is_refused(change, message):
    from edge_infer_amd.config.zadenex import ZadenexConfig, ZadenexConfigError
    raw = copy.deepcopy(CONFIGS["A"])
    change(raw)
    with pytest.raises(ZadenexConfigError, match=message):
        ZadenexConfig.from_dict(raw)


def test_cache_requests():
    """Window attention asks for key and value pages with its window; latent attention for
    one row of kv_rank + rot_dim a position and no value pages; the matrix memory for a state
    row with two versions.  Runs of a looped layer have entries of their own."""
    from edge_infer_amd.cache.storage import CacheLayout
    from edge_infer_amd.parts.base import KVRequest, StateRequest
    layout = CacheLayout(config("A").model_spec())
    requests = [request for request, _ in layout.kv_groups]
    assert KVRequest(n_kv_heads=3, head_dim=16, window=20, value_dim=24) in requests
    assert KVRequest(n_kv_heads=1, head_dim=48, value_dim=0) in requests
    assert KVRequest(n_kv_heads=1, head_dim=18, value_dim=0) in requests
    by_request = {request: entries for request, entries in layout.kv_groups}
    assert by_request[KVRequest(n_kv_heads=1, head_dim=48, value_dim=0)] == [1, 3, 5]   # three passes
    (state, entries), = layout.state_groups
    assert state == StateRequest(shape=(3 * 412,), two_versions=True)      # 16 * 24 + 24 + 1, padded to 4
    assert entries == [2, 4, 6]


def test_pages_behind_a_window_go_back():
    from edge_infer_amd.cache.allocator import PagePool, SequencePages
    pool = PagePool(8)
    pages = SequencePages(pool, 2, window=65)
    pages.open(0)
    pages.grow(0, 200)
    assert pool.n_free == 4
    pages.trim(0, 128)          # the query at 128 sees keys 64 .. 128
    assert pages.row(0)[0] == -1 and pages.row(0)[1] >= 0 and pool.n_free == 5
    pages.trim(0, 129)          # the query at 129 sees keys 65 .. 129: page 1 still holds 65
    assert pages.row(0)[1] >= 0
    pages.trim(0, 192)
    assert pages.row(0)[1] == -1 and pages.row(0)[2] >= 0


# -- the oracle's mechanisms against closed forms ----------------------------------------
def test_oracle_rotation_is_a_complex_multiplication():
    x = torch.randn(5, 3, 10, dtype=torch.float64)
    positions = torch.tensor([0, 1, 7, 100, 3000])
    out = plain.rotate_neighbours(x, positions, 500.0, 6)
    assert torch.equal(out[..., 6:], x[..., 6:]) and torch.equal(out[0], x[0])
    z = torch.complex(x[..., 0:6:2], x[..., 1:6:2])
    for i in range(3):
        angle = positions.double() * 500.0 ** (-2.0 * i / 6)
        turned = z[..., i] * torch.polar(torch.ones(5, dtype=torch.float64), angle)[:, None]
        assert torch.allclose(out[..., 2 * i], turned.real) and torch.allclose(out[..., 2 * i + 1], turned.imag)


def test_oracle_matrix_memory_against_the_unrolled_sum():
    """Without the running maximum: S_t = sum_s exp(i_s + sum_{s < r <= t} f_r) k_s v_s^T, and
    the stabilised recurrence gives the same read-out."""
    torch.manual_seed(0)
    T, d, e = 9, 4, 3
    q, k, v = (torch.randn(T, n, dtype=torch.float64) for n in (d, d, e))
    log_in = torch.randn(T, dtype=torch.float64) * 3
    log_forget = -torch.rand(T, dtype=torch.float64)
    got = plain.matrix_memory(q, k, v, log_in, log_forget)
    for t in range(T):
        weight = torch.stack([torch.exp(log_in[s] + log_forget[s + 1:t + 1].sum()) for s in range(t + 1)])
        top = (weight[:, None] * v[:t + 1] * (k[:t + 1] @ q[t])[:, None]).sum(0)
        n_dot_q = (weight * (k[:t + 1] @ q[t])).sum()
        # m_t as the recurrence defines it, from zero
        m = torch.zeros((), dtype=torch.float64)
        for s in range(t + 1):
            m = torch.maximum(log_forget[s] + m, log_in[s])
        bottom = torch.maximum(n_dot_q.abs() * torch.exp(-m), torch.exp(-m)) + 1e-6
        assert torch.allclose(got[t], top * torch.exp(-m) / bottom, rtol=1e-9, atol=1e-12)


def test_oracle_window_attention_sees_exactly_its_window():
    """Changing the token just outside the window leaves a position's mixer output as it was;
    changing the one just inside does not."""
    torch.manual_seed(1)
    m = {"heads": 4, "kv_heads": 2, "dim": 8, "vdim": 6, "scale": 0.4, "mask": {"size": 5}}
    w = 16
    p = {"q": torch.randn(32, w), "q.b": torch.randn(32), "k": torch.randn(16, w), "k.b": torch.randn(16),
         "v": torch.randn(12, w), "v.b": torch.randn(12), "talk": torch.eye(4) + 0.3 * torch.randn(4, 4),
         "o": torch.randn(w, 24), "o.b": torch.randn(w)}
    h = torch.randn(12, w, dtype=torch.float64)
    base = plain.talking_attention_mixer(h, p, m)[11]
    outside, inside = h.clone(), h.clone()
    outside[6] += 1.0          # 11 - 6 = 5: not seen
    inside[7] += 1.0           # 11 - 7 = 4: seen
    assert torch.allclose(plain.talking_attention_mixer(outside, p, m)[11], base)
    assert not torch.allclose(plain.talking_attention_mixer(inside, p, m)[11], base)


def test_oracle_softmax_with_one_in_the_denominator():
    """One key, talk = identity: the weight is e^s / (1 + e^s)."""
    m = {"heads": 1, "kv_heads": 1, "dim": 2, "vdim": 1, "scale": 1.0, "mask": {"size": 4}}
    p = {"q": torch.tensor([[1.0], [0.0]]), "q.b": torch.zeros(2), "k": torch.tensor([[2.0], [0.0]]),
         "k.b": torch.zeros(2), "v": torch.tensor([[1.0]]), "v.b": torch.zeros(1),
         "talk": torch.ones(1, 1), "o": torch.ones(1, 1), "o.b": torch.zeros(1)}
    h = torch.tensor([[1.5]], dtype=torch.float64)
    s = 1.5 * 3.0
    want = 1.5 * math.exp(s) / (1.0 + math.exp(s))
    assert abs(plain.talking_attention_mixer(h, p, m).item() - want) < 1e-12


def test_oracle_forward_uses_the_loop_and_the_multiplier():
    """times = 1 with an identity loop matrix on x and a zero step is the model without a loop;
    the stream after every run is kept."""
    raw = copy.deepcopy(CONFIGS["D"])
    tensors = sharp_weights(raw, seed=3)
    w = raw["width"]
    tensors["loop.in"] = torch.cat([torch.eye(w), torch.zeros(w, w)], dim=1).to(torch.bfloat16)
    tensors["loop.step"] = torch.zeros(1, w, dtype=torch.bfloat16)
    request = [3, 1, 4, 1, 5, 9, 2, 6]
    looped, kept = plain.forward(raw, tensors, request, keep_layers=True)
    plain_cfg = dict(raw, loop=None)
    assert torch.allclose(looped, plain.forward(plain_cfg, tensors, request), rtol=1e-12, atol=1e-12)
    assert kept.shape == (2, len(request), w)
