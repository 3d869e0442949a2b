"""Tirurax without a GPU: the configuration reader, the checkpoint's names, what the cache
is asked for, pages given back behind a chunk, and the oracle's own mechanisms against
closed forms."""
import copy
import math

import pytest
import torch

import plain_tirurax as plain
from tirurax_helpers import CONFIGS, sharp_weights, tensor_shapes


def config(name):
    from edge_infer_amd.config import TiruraxConfig
    return TiruraxConfig.from_dict(CONFIGS[name])


@pytest.mark.parametrize("name", ["A", "B"])
def test_config_round_trip_and_registry(name, tmp_path):
    import json
    from edge_infer_amd.config import TiruraxConfig, read_config, resolve_architecture
    cfg = config(name)
    assert TiruraxConfig.from_dict(cfg.to_dict()) == cfg
    assert resolve_architecture(CONFIGS[name]).config_class is TiruraxConfig
    (tmp_path / "config.json").write_text(json.dumps(CONFIGS[name]))
    entry, read, _ = read_config(tmp_path)
    assert read == cfg and entry.name == "Tirurax"


@pytest.mark.parametrize("name", ["A", "B"])
def test_spec_takes_every_size_from_the_configuration(name):
    from edge_infer_amd.config.specs import AttentionSpec, GatedDeltaSpec
    raw = CONFIGS[name]
    spec = config(name).model_spec()
    assert (spec.vocab_size, spec.hidden_size) == (raw["vocab"], raw["width"])
    assert spec.final_norm.eps == raw["norm"]["eps"] and len(spec.layers) == len(raw["layers"])
    for layer, source in zip(spec.layers, raw["layers"]):
        m, mixer = source["mixer"], layer.mixer
        assert layer.block == "outnorm" and layer.norm.eps == raw["norm"]["eps"]
        if source["type"] == "delta":
            assert isinstance(mixer, GatedDeltaSpec)
            assert (mixer.n_heads, mixer.n_kv_heads, mixer.key_dim, mixer.value_dim, mixer.conv_taps) \
                == (m["heads"], m["kv_heads"], m["dim"], m["vdim"], m["conv"])
            assert mixer.out_norm_eps == raw["norm"]["eps"] and mixer.unit_eps == 1e-6
        else:
            assert isinstance(mixer, AttentionSpec)
            assert (mixer.n_heads, mixer.n_kv_heads, mixer.head_dim, mixer.v_dim, mixer.scale) \
                == (m["heads"], m["kv_heads"], m["dim"], m["vdim"], m["scale"])
            assert mixer.chunk == (m.get("mask") or {}).get("size")
            assert mixer.qk_norm_scope == "projection" and mixer.sink and mixer.qkv_bias is True
            assert mixer.distance_slope_range == 8.0 and mixer.position.kind == "none"
        if source["mlp"] is None:
            assert layer.feed_forward is None
        else:
            assert layer.feed_forward.intermediate_size == source["mlp"]["ff"]
            assert layer.feed_forward.activation == "relu2"


@pytest.mark.parametrize("name", ["A", "B"])
def test_checkpoint_names_and_shapes(name):
    from edge_infer_amd.engine.model import expected_parameters
    cfg = config(name)
    expected = expected_parameters(cfg.model_spec(), cfg.checkpoint_name)
    required = {ckpt: tuple(param.shape) for ckpt, param in expected.values() if not param.optional}
    assert required == {k: shape for k, (shape, _) in tensor_shapes(CONFIGS[name]).items()}


def test_weights_that_do_not_fit_are_named():
    from edge_infer_amd.engine.model import expected_parameters
    from edge_infer_amd.weights import WeightsError, match_parameters
    cfg = config("A")
    expected = expected_parameters(cfg.model_spec(), cfg.checkpoint_name)
    tensors = sharp_weights(CONFIGS["A"], 0)
    del tensors["l0.mix.sink"]
    tensors["l1.mix.extra"] = torch.zeros(1)
    with pytest.raises(WeightsError) as error:
        match_parameters(expected, tensors)
    assert error.value.missing == ["l0.mix.sink"] and error.value.unexpected == ["l1.mix.extra"]


def test_a_second_norm_without_a_feed_forward_is_taken_and_unused():
    from edge_infer_amd.engine.model import expected_parameters
    from edge_infer_amd.weights import match_parameters
    cfg = config("A")
    expected = expected_parameters(cfg.model_spec(), cfg.checkpoint_name)
    tensors = sharp_weights(CONFIGS["A"], 0)
    assert "l1.norm2" not in tensors                 # layer 1 has no feed-forward
    matched = match_parameters(expected, tensors)
    tensors["l1.norm2"] = torch.ones(CONFIGS["A"]["width"])
    assert len(match_parameters(expected, tensors)) == len(matched) + 1


@pytest.mark.parametrize("change, message", [
    (lambda c: c["layers"][0].update(type="conv"), "type"),
    (lambda c: c["layers"][0]["mixer"].update(window=5), "does not know"),
    (lambda c: c["layers"][0]["mixer"].update(heads=5), "multiple of kv_heads"),
    (lambda c: c["layers"][0]["mlp"].update(kind="gated"), "kind"),
    (lambda c: c["layers"][1]["mixer"].pop("conv"), "lacks 'conv'"),
    (lambda c: c.pop("norm"), "norm"),
    (lambda c: c.update(layers=[]), "at least one layer"),
])
def test_configurations_that_are_refused(change, message):
    from edge_infer_amd.config import TiruraxConfig
    raw = copy.deepcopy(CONFIGS["A"])
    change(raw)
    with pytest.raises(ValueError, match=message):
        TiruraxConfig.from_dict(raw)


def test_cache_requests():
    """A delta layer asks for one float32 row: S of every head, then the convolution's tail;
    an attention layer for pages whose values have their own width and which a chunk lets go."""
    from edge_infer_amd.cache.storage import CacheLayout
    from edge_infer_amd.parts import KVRequest, StateRequest
    layout = CacheLayout(config("A").model_spec())
    kv = [request for request, _ in layout.kv_groups]
    assert kv == [KVRequest(2, 16, None, 24, 24), KVRequest(2, 32, None, None, None)]
    states = [request for request, _ in layout.state_groups]
    # 4 heads x 8 x 16 + 2 taps kept x (2 x 4 x 16 + 4 x 8);  4 x 16 x 24 + 1 x (2 x 24 + 64)
    assert states == [StateRequest((512 + 2 * 160,), two_versions=True),
                      StateRequest((1536 + 112,), two_versions=True)]


def test_pages_behind_a_chunk_go_back():
    from edge_infer_amd.cache.allocator import PagePool, SequencePages
    pool = PagePool(8)
    pages = SequencePages(pool, 1, chunk=100)
    pages.open(0)
    pages.grow(0, 199)
    pages.trim(0, 199)          # the next query, at 199, still sees 100..198: page 0 is dead
    assert pages.row(0)[0] == -1 and pages.row(0)[1] >= 0 and pool.n_free == 8 - 3
    pages.grow(0, 200)
    pages.trim(0, 200)          # the next query starts a block at 200: pages 0..2 are dead
    assert [p >= 0 for p in pages.row(0)] == [False, False, False, True]
    pages.close(0)
    assert pool.n_free == 8
    both = SequencePages(PagePool(8), 1, window=70, chunk=128)
    both.open(0)
    both.grow(0, 300)
    both.trim(0, 300)           # window: from 231; block: from 256
    assert [p >= 0 for p in both.row(0)] == [False, False, False, False, True]


# -- the oracle's mechanisms against closed forms ------------------------------------------
def test_oracle_convolution_and_recurrence():
    x = torch.arange(1.0, 6.0, dtype=torch.float64).reshape(5, 1)
    w = torch.tensor([[0.5, -1.0, 2.0]])          # the last tap is the current token's
    assert plain.short_conv(x, w).flatten().tolist() == [2.0, 3.0, 4.5, 6.0, 7.5]
    # with beta = 1 and no decay, writing v under a unit key and reading with it returns v
    k = torch.tensor([[1.0, 0.0], [0.0, 1.0], [1.0, 0.0]], dtype=torch.float64)
    v = torch.tensor([[3.0], [5.0], [7.0]], dtype=torch.float64)
    one = torch.ones(3, dtype=torch.float64)
    out = plain.delta_recurrence(k, k, v, one, one)
    assert out.flatten().tolist() == [3.0, 5.0, 7.0]       # the third write replaces the first
    # a decay of one half and beta = 0: the state only fades, the read-out halves
    out = plain.delta_recurrence(k[:1].repeat(3, 1), k[:1].repeat(3, 1), v,
                                 torch.tensor([1.0, 0.0, 0.0], dtype=torch.float64), one * 0.5)
    assert out.flatten().tolist() == [3.0, 1.5, 0.75]


def test_oracle_attention_sink_chunk_and_slopes():
    """One head, keys that all score zero: the weights are exp(-slope distance) against
    exp(sink), over the keys of the query's own chunk."""
    T, w = 7, 4
    m = {"heads": 1, "kv_heads": 1, "dim": 2, "vdim": 1, "scale": 1.0, "mask": {"size": 3}}
    zero = torch.zeros
    p = {"q": zero(2, w), "q.b": torch.ones(2), "k": zero(2, w), "k.b": zero(2), "v": zero(1, w),
         "v.b": torch.ones(1), "q.norm": torch.ones(2), "k.norm": torch.ones(2),
         "sink": torch.tensor([0.75]), "o": torch.ones(w, 1)}
    out = plain.attention_mixer(torch.randn(T, w, dtype=torch.float64), p, m, 1e-6)
    slope = 2.0 ** -8
    for i in range(T):
        seen = sum(math.exp(-slope * d) for d in range(i % 3 + 1))
        assert abs(out[i, 0].item() - seen / (seen + math.exp(0.75))) < 1e-12
    assert plain.distance_slopes(4) == [0.25, 0.0625, 0.015625, 0.00390625]
