"""TEST INFRASTRUCTURE — numpy restatement of the reference's uniform weight
initializers (paths under /root/reference/lib/deep-learning/):

  initialize_weights_with_glorot_uniform   v1/ops/initializers/glorot.cpp:225-359
  Initialization__Uniform                  v1/ops/initializers/uniform.cpp:26-90
  weights_initialize_uniform               v1/learner/model.cpp:5087-5096
  layer_initialize_const_bias              v1/learner/model.cpp:5031-5042
  Clear__Parameter__Normalized_Unit        v1/learner/model.cpp:3959-4025
  Dist::Real                               ops/distributions/real.cpp (std::mt19937 +
                                           std::uniform_real_distribution<float>)

The random stream: std::mt19937 seeded with `seed` is numpy's MT19937 after
init_genrand(seed) (RandomState(seed).randint over the full 32-bit range returns
the raw words).  libstdc++'s uniform_real_distribution<float>(a, b) takes one
word per draw: u = float(word) / 2^32 (1.0 replaced by the float below it), and
returns u * (b - a) + a, which the compiler fuses into one multiply-add.

Pinned by tests/golden/init.npz, written by the compiled reference
(tests/test_oracle_init.py).  Only tests may import this module.
"""
import numpy as np

f32 = np.float32

RELU, LEAKY_RELU, PARAMETRIC_RELU, SELU, TANH, TANH_STEPWISE = 16, 14, 15, 17, 23, 24


def uniform_stream(seed, n):
    """n draws of std::uniform_real_distribution<float>(0, 1)(std::mt19937(seed))."""
    words = np.random.RandomState(seed).randint(0, 2 ** 32, size=n, dtype=np.uint64)
    u = words.astype(f32) / f32(2.0 ** 32)
    u[u >= f32(1)] = np.nextafter(f32(1), f32(0))
    return u


def gain_scale(act):
    """Initialization__Gain__Scale, glorot.cpp:27-66."""
    if act == LEAKY_RELU:
        return np.sqrt(f32(2) / (f32(1) + np.power(f32(0.01), f32(2))), dtype=f32)
    if act == PARAMETRIC_RELU:
        return np.sqrt(f32(2) / (f32(1) + np.power(f32(0.25), f32(2))), dtype=f32)
    if act == RELU:
        return np.sqrt(f32(2), dtype=f32)
    if act in (TANH, TANH_STEPWISE):
        return f32(5) / f32(3)
    return f32(1)


def uniform_variance(n_inp, n_out, act):
    """Initialization__Uniform__Variance (glorot.cpp:91-111) on the class of `act`
    (train.cpp:312-363): rectifiers and SELU use the fan-in alone."""
    if act in (RELU, LEAKY_RELU, PARAMETRIC_RELU, SELU):
        return np.sqrt(f32(6) / f32(n_inp), dtype=f32)
    return np.sqrt(f32(6) / f32(n_inp + n_out), dtype=f32)


def _structure(layers):
    """Per entry: (is_fc, n_inp, n_out, in_block, block_first, block_last, residual index)."""
    n = len(layers)
    out = [None] * n
    width = {0: layers[0][1]}
    feed = 0
    l = 1
    while l < n:
        if layers[l][0] == "RES":
            D, r, cur = layers[l][1], l, feed
            for d in range(1, D + 1):
                i = r + d
                out[i] = dict(fc=True, n_inp=width[cur], n_out=layers[i][1], in_block=True, first=d == 1, last=d == D, res=r)
                width[i] = layers[i][1]
                cur = i
            width[r] = max(width[feed], width[r + D])
            out[r] = dict(fc=False, n_out=width[r])
            feed = r
            l = r + D + 1
        else:
            out[l] = dict(fc=True, n_inp=width[feed], n_out=layers[l][1], in_block=False, first=False, last=False, res=None)
            width[l] = layers[l][1]
            feed = l
            l += 1
    return out


def glorot_bounds(layers, acts):
    """{layer: bound} for the fully-connected entries.  acts[l] = ACTIVATION value
    (18, the sigmoid default, where not given)."""
    S = _structure(layers)
    n = len(layers)
    act = lambda l: acts.get(l, 18)
    bounds = {}
    for l in range(1, n):
        s = S[l]
        if not s["fc"]:
            continue
        n_inp = s["n_inp"]
        if l + 1 == n:
            n_out = n_inp
        elif s["in_block"] and s["last"]:
            n_out = S[s["res"]]["n_out"]
        elif not S[l + 1]["fc"]:
            n_out = (S[l + 1]["n_out"] + S[l + 2]["n_out"]) // 2
        else:
            n_out = S[l + 1]["n_out"]
        # a block's first layer has no activation unit of its own: the read lands on
        # the first unit of the next layer that has some (glorot.cpp:273)
        g = l
        while g + 1 < n and (not S[g]["fc"] or S[g]["first"]):
            g += 1
        bounds[l] = f32(gain_scale(act(g)) * uniform_variance(n_inp, n_out, act(l)))
    return bounds


def _fill(layers, seed, bias, bound_of, info):
    """info(l) -> dict(w0, w1, bias, n_out); returns {'weights': {l: w}, ...} as a
    flat parameter vector is the caller's business (it knows the layout)."""
    S = _structure(layers)
    fcs = [l for l in range(1, len(layers)) if S[l]["fc"]]
    total = sum(S[l]["n_inp"] * S[l]["n_out"] for l in fcs)
    u = uniform_stream(seed, total)
    k = 0
    out = {}
    for l in fcs:
        m = S[l]["n_inp"] * S[l]["n_out"]
        lo, hi = bound_of(l)
        # u * (b - a) + a is one fused multiply-add in the reference as built (GCC contracts it
        # when the target has FMA, which its -march=native release build and the x86-64-v3 build
        # used for the golden vectors both have): the 48-bit product is exact in float64, and the
        # sum is rounded to float32 from there
        out[l] = (u[k:k + m].astype(np.float64) * np.float64(f32(f32(hi) - f32(lo))) + np.float64(f32(lo))).astype(f32)
        k += m
    return out


def initialize(layers, acts, seed, bias, info, P, n_units, lower=None, upper=None):
    """The whole parameter vector after initialize_weights_with_glorot_uniform(bias)
    (lower/upper None) or Initialization__Uniform(bias, lower, upper), with the
    generator seeded first.  info(l) gives the layout of entry l (w0, w1, bias,
    n_out, gamma): scales are 1, shifts 0."""
    if lower is None:
        b = glorot_bounds(layers, acts)
        W = _fill(layers, seed, bias, lambda l: (-b[l], b[l]), info)
    else:
        W = _fill(layers, seed, bias, lambda l: (lower, upper), info)
    p = np.zeros(P, f32)
    for l, w in W.items():
        i = info(l)
        assert i["w1"] - i["w0"] == w.size
        p[i["w0"]:i["w1"]] = w
        p[i["bias"]:i["bias"] + i["n_out"]] = f32(bias)
    g0 = info(0)["gamma"]
    p[g0:g0 + n_units] = 1
    p[g0 + n_units:g0 + 2 * n_units] = 0
    return p


# ---- dropout masks: Model::Dropout_Bernoulli, v1/learner/bernoulli_st.cpp:27-100 ------------------
class BernoulliStream:
    """Dist::Bernoulli (ops/distributions/bernoulli.cpp): std::bernoulli_distribution over a std::mt19937
    of its own.  libstdc++ draws u = generate_canonical<double, 53>: two 32-bit words, (w0 + w1 * 2^32) / 2^64
    in double, and keeps the unit when u < p (p the float probability widened to double)."""

    def __init__(self, seed):
        self.rs = np.random.RandomState(seed)

    def draw(self, n, p):
        w = self.rs.randint(0, 2 ** 32, size=2 * n, dtype=np.uint64).astype(np.float64)
        u = (w[0::2] + w[1::2] * 2.0 ** 32) / 2.0 ** 64
        u[u >= 1.0] = np.nextafter(1.0, 0.0)
        return (u < np.float64(f32(p))).astype(np.uint8)


def dropout_bernoulli(stream, units, dropout, masks):
    """One call of Dropout_Bernoulli: `dropout` maps a layer to (kind, keep), `units` to its number of units,
    `masks` holds the current masks and is updated in place.  Only the plain Bernoulli layers are resampled,
    in layer order; a keep probability of 0 clears the mask without drawing (bernoulli_st.cpp:39-100)."""
    for l in sorted(dropout):
        kind, keep = dropout[l]
        if kind != "BERNOULLI":
            continue
        masks[l] = stream.draw(units[l], keep) if f32(keep) != 0 else np.zeros(units[l], np.uint8)
    return masks
