"""Vobotar without a GPU: the plain implementation pinned on cases worked out by
hand, configuration errors, and the built model's tensor names, cache groups
and states."""
import copy
import math

import pytest
import torch

from plain import vobotar_plain as VP
from vobotar_util import CONFIGS, RANKS, attention, config, dense, pair, pair2, write_model

F = torch.float64


# ------------------------------------------------------- the plain mechanisms
def test_norm_with_a_weight_stored_around_zero():
    x = torch.tensor([[3.0, 4.0]], dtype=F)
    r = math.sqrt(12.5)
    assert torch.allclose(VP.norm_one_plus(x, torch.tensor([0.0, 1.0], dtype=F), 0.0), torch.tensor([[3 / r, 8 / r]], dtype=F))
    assert torch.allclose(VP.norm_plain(x, torch.tensor([0.0, 1.0], dtype=F), 0.0), torch.tensor([[0.0, 4 / r]], dtype=F))
    # eps stands inside the root
    assert math.isclose(float(VP.norm_plain(x, torch.ones(2, dtype=F), 3.5)[0, 0]), 3 / 4.0)


def test_both_rotations_by_hand():
    x = torch.tensor([[[1.0, 2.0, 3.0, 4.0, 5.0, 6.0]]], dtype=F)       # one token, one head of six
    base, dims, p = 100.0, 4, 3
    a0, a1 = p * 1.0, p * base ** (-2 / 4)
    n = VP.rotate_neighbours(x, [p], dims, base)[0, 0]
    want = [1 * math.cos(a0) - 2 * math.sin(a0), 2 * math.cos(a0) + 1 * math.sin(a0),
            3 * math.cos(a1) - 4 * math.sin(a1), 4 * math.cos(a1) + 3 * math.sin(a1), 5.0, 6.0]
    assert torch.allclose(n, torch.tensor(want, dtype=F))
    h = VP.rotate_halves(x, [p], dims, base)[0, 0]
    want = [1 * math.cos(a0) - 3 * math.sin(a0), 2 * math.cos(a1) - 4 * math.sin(a1),
            3 * math.cos(a0) + 1 * math.sin(a0), 4 * math.cos(a1) + 2 * math.sin(a1), 5.0, 6.0]
    assert torch.allclose(h, torch.tensor(want, dtype=F))


@pytest.mark.parametrize("rotate", [VP.rotate_neighbours, VP.rotate_halves])
def test_rotated_products_depend_on_the_distance_alone(rotate):
    g = torch.Generator().manual_seed(1)
    q, k = torch.randn(1, 1, 8, generator=g, dtype=F), torch.randn(1, 1, 8, generator=g, dtype=F)
    def dot(pq, pk):
        return float((rotate(q, [pq], 6, 50.0) * rotate(k, [pk], 6, 50.0)).sum())
    assert math.isclose(dot(9, 4), dot(105, 100), rel_tol=1e-9)
    assert not math.isclose(dot(9, 4), dot(9, 5), rel_tol=1e-3)


def test_who_sees_whom():
    ok = VP.visible(5, 3)
    assert ok.tolist() == [[True, False, False, False, False], [True, True, False, False, False],
                           [True, True, True, False, False], [False, True, True, True, False],
                           [False, False, True, True, True]]
    assert VP.visible(3, 0).tolist() == [[True, False, False], [True, True, False], [True, True, True]]


def test_softmax_with_a_sink_a_cap_and_a_distance_penalty():
    q = torch.tensor([[[1.0]], [[1.0]]], dtype=F)
    k = torch.tensor([[[2.0]], [[3.0]]], dtype=F)
    v = torch.tensor([[[10.0]], [[20.0]]], dtype=F)
    # the sink stands in the denominator once and has no value
    o = VP.attend(q, k, v, 1.0, sink=torch.tensor([0.5], dtype=F))
    e2, e3, es = math.exp(2), math.exp(3), math.exp(0.5)
    assert math.isclose(float(o[0, 0, 0]), 10 * e2 / (e2 + es))
    assert math.isclose(float(o[1, 0, 0]), (10 * e2 + 20 * e3) / (e2 + e3 + es))
    # a sink of zero: one more 1 in the denominator
    o = VP.attend(q, k, v, 1.0, sink=torch.zeros(1, dtype=F))
    assert math.isclose(float(o[0, 0, 0]), 10 * e2 / (e2 + 1))
    # the cap bends the scaled score; the penalty is taken off afterwards and grows with the distance
    o = VP.attend(q, k, v, 2.0, cap=3.0, slopes=torch.tensor([0.25], dtype=F))
    s0, s1 = 3 * math.tanh(4 / 3) - 0.25, 3 * math.tanh(6 / 3)
    assert math.isclose(float(o[1, 0, 0]), (10 * math.exp(s0) + 20 * math.exp(s1)) / (math.exp(s0) + math.exp(s1)))
    assert VP.distance_slopes(4).tolist() == [2.0 ** -2, 2.0 ** -4, 2.0 ** -6, 2.0 ** -8]


def test_convolution_taps_bias_and_start():
    x = torch.tensor([[1.0], [2.0], [3.0]], dtype=F)
    w = torch.tensor([[100.0, 10.0, 1.0]], dtype=F)       # the last column is the current token's
    y = VP.causal_conv(x, w, torch.tensor([0.5], dtype=F), silu_after=False)
    assert torch.allclose(y, torch.tensor([[1.5], [12.5], [123.5]], dtype=F))


def _time_mix_weights(mu=0.0):
    # one head of two key channels; identity projections
    eye = torch.eye(2, dtype=F)
    w = {"m.mu." + s: torch.full((2,), mu, dtype=F) for s in "rkvgw"}
    w.update({"m.r": eye, "m.k": eye, "m.v": eye, "m.g": eye, "m.o": eye, "m.w1": torch.zeros(1, 2, dtype=F),
              "m.w2": torch.zeros(2, 1, dtype=F), "m.w0": torch.log(torch.tensor([math.log(2.0), math.log(4.0)], dtype=F)),
              "m.u": torch.tensor([[3.0, 0.0]], dtype=F), "m.norm": torch.ones(2, dtype=F)})
    return w


def test_time_mix_two_steps_by_hand():
    """Decays of 1/2 and 1/4, a bonus of 3 on the first key channel.  Step 0: S = 0, so
    o = (u k) . r * v.  Step 1 reads S before its decay; then S <- diag(decay) S + k v^T."""
    w = _time_mix_weights()
    h = torch.tensor([[1.0, 2.0], [2.0, 1.0]], dtype=F)
    y, (S, last) = VP.right_time_mix(h, w, "m.", dict(heads=1, dim=2), 0.0)
    # step 0: o = (3 * 1 * 1) * v = [3, 6]; step 1: S0 = k0 v0^T = [[1, 2], [2, 4]]; o = r . S0 + (3 * 2 * 2) v1 = [4, 8] + [24, 12]
    o = torch.tensor([[3.0, 6.0], [28.0, 20.0]], dtype=F)
    want = o / torch.sqrt((o * o).mean(-1, keepdim=True)) * (h * torch.sigmoid(h))
    assert torch.allclose(y, want)
    # S1 = diag(1/2, 1/4) S0 + k1 v1^T
    assert torch.allclose(S[0], torch.tensor([[0.5 + 4, 1 + 2], [0.5 + 2, 1 + 1]], dtype=F))
    assert torch.equal(last, h[1])


def test_time_mix_blends_with_the_row_before_and_carries_it_between_steps():
    w = _time_mix_weights(mu=0.25)
    g = torch.Generator().manual_seed(0)
    h = torch.randn(5, 2, generator=g, dtype=F)
    whole, _ = VP.right_time_mix(h, w, "m.", dict(heads=1, dim=2), 1e-6)
    a, st = VP.right_time_mix(h[:2], w, "m.", dict(heads=1, dim=2), 1e-6)
    b, _ = VP.right_time_mix(h[2:], w, "m.", dict(heads=1, dim=2), 1e-6, state=st)
    assert torch.allclose(torch.cat([a, b]), whole)
    # the first row blends with zeros
    only, _ = VP.right_time_mix(h[:1], w, "m.", dict(heads=1, dim=2), 1e-6)
    assert torch.allclose(only, whole[:1])


def test_state_space_step_by_hand_and_in_portions():
    m = dict(heads=1, vdim=1, state=2, groups=1, conv=2, norm_groups=1)
    # rows of W_in: z | x | B (2) | C (2) | dt, reading a stream of width 1
    w = {"m.in": torch.tensor([[1.0], [1.0], [1.0], [0.0], [0.0], [1.0], [0.0]], dtype=F),
         "m.conv": torch.tensor([[0.0, 1.0]] * 5, dtype=F), "m.conv.b": torch.zeros(5, dtype=F),
         "m.dt_bias": torch.tensor([0.0], dtype=F), "m.A_log": torch.tensor([0.0], dtype=F), "m.D": torch.tensor([2.0], dtype=F),
         "m.norm": torch.ones(1, dtype=F), "m.o": torch.ones(1, 1, dtype=F)}
    h = torch.tensor([[1.0], [3.0]], dtype=F)
    y, (S, tail) = VP.right_state_space(h, w, "m.", m, 0.0)
    sl = lambda z: z / (1 + math.exp(-z))
    dt = math.log(2.0)                                      # softplus(0)
    x0, x1 = sl(1.0), sl(3.0)
    # B = (silu(h), 0), C = (0, silu(h)): the state's second row stays empty, so y = D x
    s0 = dt * x0 * x0
    s1 = math.exp(-dt) * s0 + dt * x1 * x1
    assert math.isclose(float(S[0, 0, 0]), s1) and float(S[0, 1, 0]) == 0.0
    pre = torch.tensor([2 * x0 * sl(1.0), 2 * x1 * sl(3.0)], dtype=F)
    assert torch.allclose(y[:, 0], pre / pre.abs())
    assert torch.allclose(tail, torch.tensor([[3.0, 3.0, 0.0, 0.0, 3.0]], dtype=F))    # the last input of x, B, C
    g = torch.Generator().manual_seed(3)
    m2 = dict(heads=2, vdim=3, state=4, groups=1, conv=3, norm_groups=2)
    inner, ch = 6, 6 + 8
    w2 = {"m.in": torch.randn(inner + ch + 2, 5, generator=g, dtype=F), "m.conv": torch.randn(ch, 3, generator=g, dtype=F),
          "m.conv.b": torch.randn(ch, generator=g, dtype=F), "m.dt_bias": torch.randn(2, generator=g, dtype=F),
          "m.A_log": torch.randn(2, generator=g, dtype=F), "m.D": torch.randn(2, generator=g, dtype=F),
          "m.norm": torch.randn(inner, generator=g, dtype=F), "m.o": torch.randn(5, inner, generator=g, dtype=F)}
    hh = torch.randn(7, 5, generator=g, dtype=F)
    whole, _ = VP.right_state_space(hh, w2, "m.", m2, 1e-6)
    a, st = VP.right_state_space(hh[:1], w2, "m.", m2, 1e-6)
    b, st = VP.right_state_space(hh[1:3], w2, "m.", m2, 1e-6, state=st)
    c, _ = VP.right_state_space(hh[3:], w2, "m.", m2, 1e-6, state=st)
    assert torch.allclose(torch.cat([a, b, c]), whole)


def test_the_layer_norms_what_a_branch_gives_and_not_what_it_reads():
    """One attention layer without feed-forward or side input: the stream after the layer is the
    embedding plus the normed mixer output; scaling the mixer's output projection changes nothing."""
    cfg = config(11, 8, [attention(1, 1, 4, 4, 0.5)], scale=2.0)
    g = torch.Generator().manual_seed(5)
    w = {"embed": torch.randn(11, 8, generator=g, dtype=F), "final.norm": torch.zeros(8, dtype=F), "l0.norm1": torch.zeros(8, dtype=F)}
    for n, s in (("q", (4, 8)), ("k", (4, 8)), ("v", (4, 8)), ("g", (4, 8)), ("o", (8, 4))):
        w["l0.mix." + n] = torch.randn(s, generator=g, dtype=F)
    w["l0.mix.q.norm"] = w["l0.mix.k.norm"] = torch.ones(4, dtype=F)
    _, layers = VP.forward(cfg, w, [3, 5, 7], return_layers=True)
    x0 = w["embed"][[3, 5, 7]] * 2.0
    added = layers[0] - x0
    assert torch.allclose((added * added).mean(-1), torch.ones(3, dtype=F), atol=1e-4)
    w2 = dict(w)
    w2["l0.mix.o"] = w["l0.mix.o"] * 7.0
    _, layers2 = VP.forward(cfg, w2, [3, 5, 7], return_layers=True)
    assert torch.allclose(layers, layers2, atol=1e-5)


def test_blended_values_come_from_the_first_blending_layer(tmp_path):
    """With three blending layers the third takes the first layer's values, not the second's: making
    the second layer's own value projection zero leaves what the third blends in untouched."""
    cfg = config(31, 16, [attention(2, 1, 4, 6, 0.5, v_mix=True), attention(2, 1, 4, 6, 0.5, v_mix=True),
                          attention(2, 1, 4, 6, 0.5, v_mix=True)])
    g = torch.Generator().manual_seed(2)
    shapes = {"q": (8, 16), "k": (4, 16), "v": (6, 16), "g": (12, 16), "o": (16, 12)}
    w = {"embed": torch.randn(31, 16, generator=g, dtype=F), "final.norm": torch.zeros(16, dtype=F)}
    for i in range(3):
        w[f"l{i}.norm1"] = torch.zeros(16, dtype=F)
        for n, s in shapes.items():
            w[f"l{i}.mix.{n}"] = torch.randn(s, generator=g, dtype=F)
        w[f"l{i}.mix.q.norm"] = w[f"l{i}.mix.k.norm"] = torch.ones(4, dtype=F)
        w[f"l{i}.mix.vmix"] = torch.tensor(1.0, dtype=F)            # all of the first layer's values
    toks = [1, 2, 3, 4]
    base = VP.forward(cfg, w, toks)
    w2 = dict(w)
    w2["l2.mix.v"] = torch.zeros(6, 16, dtype=F)                    # unused at a blend of 1
    assert torch.allclose(VP.forward(cfg, w2, toks), base)
    w3 = dict(w)
    w3["l0.mix.vmix"] = torch.tensor(0.3, dtype=F)                  # the first layer's own number is never read
    assert torch.allclose(VP.forward(cfg, w3, toks), base)
    w4 = dict(w)
    w4["l0.mix.v"] = w["l0.mix.v"] * 2.0                            # and its values reach the last layer
    assert not torch.allclose(VP.forward(cfg, w4, toks), base)


# ------------------------------------------------------------- configuration
def test_configuration_errors_name_the_missing_key():
    from lyapunov_engine_amd.config import ConfigError, VobotarConfig

    good = CONFIGS["A"]
    VobotarConfig.from_dict(good)
    for path, key in ((("embedding",), "scale"), (("norm",), "eps"), (("layers", 0, "mixer"), "scale"),
                      (("layers", 1, "mixer", "left"), "kv_heads"), (("layers", 1, "mixer", "right"), "dim"),
                      (("layers", 3, "mixer", "right"), "norm_groups"), (("layers", 3, "mixer"), "left_scale"),
                      (("layers", 0, "mixer", "rot"), "base"), (("layers", 0, "mlp"), "ff"), ((), "width")):
        bad = copy.deepcopy(good)
        d = bad
        for p in path:
            d = d[p]
        del d[key]
        with pytest.raises(ConfigError, match=key):
            VobotarConfig.from_dict(bad)
    bad = copy.deepcopy(good)
    bad["layers"][0]["type"] = "something"
    with pytest.raises(ConfigError, match="something"):
        VobotarConfig.from_dict(bad)
    bad = copy.deepcopy(good)
    bad["layers"][1]["mixer"]["left"]["heads"] = 3
    with pytest.raises(ConfigError, match="split"):
        VobotarConfig.from_dict(bad)
    again = VobotarConfig.from_dict(VobotarConfig.from_dict(good).to_dict())
    assert again == VobotarConfig.from_dict(good)


def test_optional_constants_may_be_absent():
    from lyapunov_engine_amd.config.registry import architecture_of
    from lyapunov_engine_amd.models.decoder import build_model

    cfg = CONFIGS["B"]
    arch = architecture_of(cfg)
    model = build_model(arch.to_spec(arch.config_class.from_dict(cfg)))
    names = set(model.expected_tensors())
    assert "side.embed" not in names and not any(".side." in n for n in names)
    assert "l1.norm2" not in names and "l1.mlp.gate" not in names
    assert model.layers[1].mixer.position is None and model.layers[1].mixer.cap == 0.0
    assert model.layers[2].mixer.left.window == 0


# ------------------------------------------------------------------ the model
def test_built_model_names_groups_and_states(tmp_path):
    from lyapunov_engine_amd.config.registry import architecture_of
    from lyapunov_engine_amd.models.decoder import build_model

    cfg = CONFIGS["A"]
    arch = architecture_of(cfg)
    model = build_model(arch.to_spec(arch.config_class.from_dict(cfg)))
    names = model.expected_tensors()
    for n in ("embed", "side.embed", "final.norm", "l0.norm1", "l0.mix.q.norm", "l0.mix.g", "l1.mix.left.q.b", "l1.mix.left.sink",
              "l1.mix.right.mu.w", "l1.mix.right.u", "l1.mix.right.w2", "l2.mix.vmix", "l3.mix.left.v.b", "l3.mix.left.k.norm",
              "l3.mix.right.conv.b", "l3.mix.right.A_log", "l4.side.gate", "l4.side.norm", "l0.mlp.down"):
        assert n in names, n
    for n in ("l0.mix.vmix", "l1.mix.left.v", "l2.norm2", "head"):
        assert n not in names, n
    assert model.ignorable("l0.mix.vmix") and model.ignorable("l2.norm2") and not model.ignorable("l2.mix.vmix")
    assert names["side.embed"][0] == (203, 25) and names["l1.mix.left.g"][0] == (4, 72) and names["l0.mix.g"][0] == (36, 72)
    assert names["l3.mix.left.q.norm"][0] == (36,) and names["l0.mix.q.norm"][0] == (10,)
    assert names["l3.mix.right.in"][0] == (24 + 24 + 24 + 3, 72)
    # every layer's branch takes its own stretch of the shared side table
    cols = [model.layers[i].side.weight_specs()[2].sources[0].columns for i in range(5)]
    assert cols == [(0, 5), (5, 10), (10, 15), (15, 20), (20, 25)]
    layout = model.cache_layout()
    # full attention with values of 12 twice (keys of 10 and of 8 differ), windows of 21 and of 13, one more full layer
    assert [(g.spec.window, g.buffers) for g in layout.groups] == [(0, (0,)), (21, (1,)), (0, (2,)), (13, (3,)), (0, (4,))]
    assert set(layout.states) == {1, 3}
    assert tuple(layout.states[1].shape) == (3, 10, 10) and tuple(layout.states[3].shape) == (3, 8, 12)
    assert set(layout.part_states) == {(1, "mixer.right.shift"), (3, "mixer.right.conv")}
    assert tuple(layout.part_states[(3, "mixer.right.conv")].shape) == (2, 24 + 24)
    # written and read back: shapes fit, the free rank is the file's
    folder = write_model(str(tmp_path / "m"), cfg, seed=1, dtype="float32", rank=RANKS["A"])
    cfg2, tensors = VP.load_folder(folder)
    assert tensors["l1.mix.right.w1"].shape == (5, 72) and tensors["l0.mix.vmix"].shape == ()
    assert VP.forward(cfg2, tensors, [1, 2, 3]).shape == (3, 203)


def test_a_tensor_shared_by_column_ranges_is_claimed_once(tmp_path):
    from lyapunov_engine_amd.config.registry import architecture_of
    from lyapunov_engine_amd.models.decoder import build_model
    from lyapunov_engine_amd.weights.loader import DictSource, WeightError, check_tensors

    cfg = config(19, 16, [attention(1, 1, 4, 4, 0.5), attention(1, 1, 4, 4, 0.5)], side=3)
    arch = architecture_of(cfg)
    model = build_model(arch.to_spec(arch.config_class.from_dict(cfg)))
    shapes = {n: tuple(abs(d) for d in s) for n, (s, _) in model.expected_tensors().items()}
    assert shapes["side.embed"] == (19, 6)
    check_tensors(model, shapes)
    with pytest.raises(WeightError, match="side.embed"):
        check_tensors(model, dict(shapes, **{"side.embed": (19, 5)}))
