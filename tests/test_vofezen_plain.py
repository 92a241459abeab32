"""Pins of the plain Vofezen implementation (hand-worked numbers, identities), the configuration
reader, the declared tensors, and the product's rotation frequencies against the plain ones."""
import math

import numpy as np
import pytest

import plain_vofezen as pv
import vofezen_util as vu


def test_frequencies_without_stretching():
    f, amp = pv.rotary_frequencies(8, 10000.0)
    assert amp == 1.0
    np.testing.assert_allclose(f, [1.0, 0.1, 0.01, 0.001], rtol=1e-12)


def test_stretched_frequencies_by_hand():
    # dims 8, base 16, original 64, factor 4: turn(t) = 8 ln(64 / (2 pi t)) / (2 ln 16)
    scaling = {"factor": 4.0, "original": 64, "fast": 4.0, "slow": 1.0}
    turn = lambda t: 8 * math.log(64 / (2 * math.pi * t)) / (2 * math.log(16))
    assert math.floor(turn(4.0)) == 1 and math.ceil(turn(1.0)) == 4
    lo, hi = 1, min(4, 7)
    f, amp = pv.rotary_frequencies(8, 16.0, scaling)
    base = [16.0 ** (-2 * i / 8) for i in range(4)]
    ramp = [0.0, 0.0, 1 / 3, 2 / 3]
    want = [b / 4 * r + b * (1 - r) for b, r in zip(base, ramp)]
    np.testing.assert_allclose(f, want, rtol=1e-12)
    assert amp == pytest.approx(0.1 * math.log(4.0) + 1.0)
    assert (lo, hi) == (1, 4)


def test_product_frequencies_equal_plain_ones():
    from hfee_amd.parts.rotary import rope_amplitude, rope_frequencies
    for dims, base, sc in ((32, 50000.0, (4.0, 1024.0, 32.0, 1.0)), (16, 10000.0, (8.0, 64.0, 16.0, 2.0)),
                           (8, 16.0, (4.0, 64.0, 4.0, 1.0)), (24, 500.0, None), (6, 100.0, (2.0, 4096.0, 1000.0, 0.001))):
        scaling = None if sc is None else dict(zip(("factor", "original", "fast", "slow"), sc))
        f, amp = pv.rotary_frequencies(dims, base, scaling)
        tagged = None if sc is None else ("yarn",) + sc
        np.testing.assert_allclose(rope_frequencies(dims, base, tagged), f, rtol=1e-13)
        assert rope_amplitude(tagged) == pytest.approx(amp, rel=1e-15)


def test_rotation_pairs_and_untouched_dims():
    u = np.arange(12, dtype=np.float64).reshape(1, 2, 6) + 1.0
    out = pv.rotate(u, np.array([3]), np.array([0.5, 0.25]), 2.0, 4)
    for h in range(2):
        for i, fr in enumerate((0.5, 0.25)):
            a, b = u[0, h, i], u[0, h, i + 2]
            c, s = 2.0 * math.cos(3 * fr), 2.0 * math.sin(3 * fr)
            assert out[0, h, i] == pytest.approx(a * c - b * s)
            assert out[0, h, i + 2] == pytest.approx(b * c + a * s)
        np.testing.assert_array_equal(out[0, h, 4:], u[0, h, 4:])
    np.testing.assert_array_equal(pv.rotate(u, np.array([0]), np.array([0.5, 0.25]), 1.0, 4), u)


def test_sink_joins_the_denominator_only():
    scores = np.array([[[1.0, 9.0], [0.5, 2.0]]])          # one head, two tokens; (0, 1) is masked
    values = np.array([[[1.0, 10.0], [3.0, 20.0]]])
    out = pv.causal_softmax_mix(scores, values, sink=np.array([0.7]))
    w00 = math.exp(1.0) / (math.exp(1.0) + math.exp(0.7))
    np.testing.assert_allclose(out[0, 0], w00 * values[0, 0], rtol=1e-12)
    den = math.exp(0.5) + math.exp(2.0) + math.exp(0.7)
    np.testing.assert_allclose(out[0, 1], (math.exp(0.5) * values[0, 0] + math.exp(2.0) * values[0, 1]) / den, rtol=1e-12)
    plain = pv.causal_softmax_mix(scores, values)
    np.testing.assert_allclose(plain[0, 0], values[0, 0], rtol=1e-12)
    far = pv.causal_softmax_mix(scores, values, sink=np.array([-60.0]))
    np.testing.assert_allclose(far, plain, rtol=1e-12)


def test_norms():
    y = np.array([[3.0, -4.0]])
    np.testing.assert_allclose(pv.offset_norm(y, np.array([0.5, -1.0]), 0.0), [[3 / math.sqrt(12.5) * 1.5, 0.0]], atol=1e-15)
    np.testing.assert_allclose(pv.plain_norm(y, np.array([0.5, -1.0]), 3.5),
                               [[3 / 4 * 0.5, 4 / 4 * 1.0]], rtol=1e-12)


def test_feed_forward_squares_relu():
    w = {"up": np.array([[1.0], [-1.0]]), "up.b": np.array([0.5, 0.25]), "down": np.array([[2.0, 3.0]]), "down.b": np.array([-1.0])}
    assert pv.dense_feed_forward(np.array([[1.0]]), w)[0, 0] == pytest.approx(2.0 * 1.5 ** 2 - 1.0)
    assert pv.dense_feed_forward(np.array([[-1.0]]), w)[0, 0] == pytest.approx(3.0 * 1.25 ** 2 - 1.0)


def _model(name, tmp_path, seed=3):
    return pv.PlainVofezen(vu.make_folder(tmp_path / name, vu.CONFIGS[name], seed))


def test_a_token_sees_only_what_came_before(tmp_path):
    m = _model("A", tmp_path)
    tokens = np.random.default_rng(0).integers(0, 211, size=40).tolist()
    whole = m.forward(tokens)
    for cut in (1, 2, 17, 33):
        np.testing.assert_allclose(m.forward(tokens[:cut]), whole[:cut], rtol=1e-9, atol=1e-12)


def test_blending_uses_the_first_blending_layer(tmp_path):
    folder = vu.make_folder(tmp_path / "A", vu.V_A, 5)
    m = pv.PlainVofezen(folder)
    tokens = list(range(3, 30))
    base = m.forward(tokens)
    m2 = pv.PlainVofezen(folder)
    m2.t["l0.mix.vmix"] = np.float64(0.9)       # layer 0 blends nothing, layer 1 is the source: both unused
    m2.t["l1.mix.vmix"] = np.float64(0.1)
    np.testing.assert_array_equal(m2.forward(tokens), base)
    m2.t["l3.mix.vmix"] = m2.t["l3.mix.vmix"] + 0.2
    assert np.abs(m2.forward(tokens) - base).max() > 1e-4


def test_latent_attention_in_absorbed_form(tmp_path):
    """[W_uk^T q_plain | q_rot] against the cached row [c | k_rot], the weighted sum over c, then
    W_uv: the same as scoring and mixing per-head keys and values."""
    m = _model("C", tmp_path)
    cfg = vu.V_C["layers"][1]["mixer"]
    w = m._sub("l1.mix.")
    rng = np.random.default_rng(1)
    T = 9
    h = rng.standard_normal((T, 128))
    pos = np.arange(T)
    want = pv.latent_attention_mixer(h, pos, w, cfg, 1e-5)
    H, Dn, Dr, Dv, R = cfg["heads"], cfg["dim"], cfg["rot_dim"], cfg["vdim"], cfg["kv_rank"]
    q = (pv.plain_norm(h @ w["dq"].T, w["dq.norm"], 1e-5) @ w["uq"].T).reshape(T, H, Dn + Dr)
    dkv = h @ w["dkv"].T
    c = pv.plain_norm(dkv[:, :R], w["dkv.norm"], 1e-5)
    f, amp = pv.rotary_frequencies(Dr, cfg["rot"]["base"])
    key = np.concatenate([c, pv.rotate(dkv[:, R:].reshape(T, 1, Dr), pos, f, amp, Dr)[:, 0]], axis=1)
    uk, uv = w["uk"].reshape(H, Dn, R), w["uv"].reshape(H, Dv, R)
    qa = np.concatenate([np.einsum("thd,hdr->thr", q[..., :Dn], uk), pv.rotate(q[..., Dn:], pos, f, amp, Dr)], axis=-1)
    scores = np.einsum("thk,sk->hts", qa, key) * cfg["scale"]
    mixed = pv.causal_softmax_mix(scores, np.broadcast_to(c, (H, T, R)))
    got = np.einsum("htr,hvr->thv", mixed, uv).reshape(T, H * Dv) @ w["o"].T
    np.testing.assert_allclose(got, want, rtol=1e-9, atol=1e-12)


def test_config_round_trip_and_errors():
    from hfee_amd.config import ConfigError, config_from_dict, model_spec_of
    for cj in vu.CONFIGS.values():
        cfg = config_from_dict(cj)
        assert cfg.to_dict() == cj
        spec = model_spec_of(cfg)
        assert [l.mixer.kind for l in spec.layers] == [{"attention": "kv_attention"}.get(l["type"], l["type"]) for l in cj["layers"]]
    blends = [l.mixer.get("value_blend") for l in model_spec_of(config_from_dict(vu.V_A)).layers]
    assert blends == [None, "source", None, "mix", None, "mix"]
    bad = {"architecture": "Vofezen", "vocab": 10, "width": 8, "norm": {"eps": 1e-5},
           "layers": [vu.with_mlp(vu.attention(3, 2, 8, 8, 4, False), 8)]}
    with pytest.raises(ConfigError, match="multiple"):
        config_from_dict(bad)
    bad["layers"] = [dict(vu.with_mlp(vu.attention(2, 2, 8, 8, 4, False), 8), type="ssm")]
    with pytest.raises(ConfigError, match="unknown mixer type"):
        config_from_dict(bad)
    bad["layers"] = [vu.with_mlp(vu.attention(2, 2, 8, 8, 4, True), 8), vu.with_mlp(vu.attention(2, 1, 8, 8, 4, True), 8)]
    with pytest.raises(ConfigError, match="blend"):
        config_from_dict(bad)
    with pytest.raises(ConfigError, match="missing key 'vocab'"):
        config_from_dict({"architecture": "Vofezen", "width": 8, "norm": {"eps": 0.1}, "layers": [{}]})


def test_declared_tensors(tmp_path):
    from hfee_amd.config import config_from_dict
    from hfee_amd.engine.model import declared_tensors
    specs = {s.name: tuple(s.shape) for s in declared_tensors(config_from_dict(vu.V_A))}
    assert specs["embed"] == (211, 72) and specs["head"] == (211, 72) and specs["final.norm"] == (72,)
    assert specs["l1.mix.q"] == (128, 72) and specs["l1.mix.k"] == (64, 72) and specs["l1.mix.v"] == (32, 72)
    assert specs["l1.mix.o"] == (72, 64) and specs["l1.mix.sink"] == (4,) and specs["l1.mix.vmix"] == ()
    assert specs["l2.mix.dkv"] == (48, 72) and specs["l2.mix.uq"] == (96, 48) and specs["l2.mix.uk"] == (48, 32)
    assert specs["l2.mix.dq.norm"] == (48,) and specs["l2.mix.dkv.norm"] == (32,) and specs["l2.mix.uv"] == (48, 32)
    assert "l2.mlp.up" not in specs and "l2.norm2" not in specs and "l2.norm1b" in specs
    assert specs["l0.mlp.up.b"] == (100,) and specs["l0.mlp.down.b"] == (72,)
    # the folder made for the tests holds exactly these
    got = pv.read_safetensors(vu.make_folder(tmp_path / "A", vu.V_A, 1) + "/model.safetensors")
    assert {k: v.shape for k, v in got.items()} == specs
