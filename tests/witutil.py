"""Seeded synthetic inputs of the witness generator tests: activations at scale 2^16 with unit
variance, weights with the variance of a trained layer (1/fan_in), norm weights near one."""
import numpy as np

# the files the reference's generator writes per layer (zzllama/llama/model.py:236-249, :479-586,
# :646-693, :762-773), as "<directory>/<name>"
TENSOR_NAMES = (
    ["W/" + n for n in ("Q", "K", "V", "O", "gate", "up", "down", "NormFirst", "NormSecond")]
    + ["Q/" + n for n in ("input", "rmsFirst", "rmswFirst", "normOutFirst", "xq", "xk", "xv", "scores", "max", "exp_input",
                          "exp_output", "exp_sum", "softmax_output", "softmax_lookup_query", "qkv", "atten_out", "skip",
                          "rmsSecond", "rmswSecond", "normOutSecond", "ffn_input", "up_out", "gate_out", "silu_out", "upSilu",
                          "down_out", "output")]
    + ["R/" + n for n in ("rmswFirst", "normOutFirst", "xq", "xk", "xv", "scores", "qkv", "atten_out", "rmswSecond",
                          "normOutSecond", "up_out", "gate_out", "upSilu", "down_out")])


def layer_inputs(T, D, F, seed):
    rng = np.random.default_rng(seed)

    def gauss(shape, sigma):
        return np.rint(rng.normal(0.0, sigma, shape)).astype(np.int32)

    x = gauss((T, D), 65536.0)
    sd, sf = 65536.0 / np.sqrt(D), 65536.0 / np.sqrt(F)
    weights = {"Q": gauss((D, D), sd), "K": gauss((D, D), sd), "V": gauss((D, D), sd), "O": gauss((D, D), sd),
               "gate": gauss((F, D), sd), "up": gauss((F, D), sd), "down": gauss((D, F), sf),
               "NormFirst": 65536 + gauss((D,), 2000.0), "NormSecond": 65536 + gauss((D,), 2000.0)}
    return x, weights
