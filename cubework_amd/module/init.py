"""Initializer factories with the reference's call convention
`initializer(tensor, fan_in=None, fan_out=None)` where the fans are the GLOBAL
layer sizes, never the shard sizes (cubework/module/init.py:8-140). They are
thin wrappers over torch.nn.init; the bounds/standard deviations are:

  kaiming_uniform_(a, mode, nonlinearity): U(+-sqrt(3) * gain / sqrt(fan))      (init.py:43-63)
  kaiming_normal_ : N(0, gain / sqrt(fan))                                       (init.py:66-85)
  xavier_uniform_(a, scale, gain): U(+-a * gain * sqrt(scale / (fan_in[+fan_out])))  (init.py:88-101)
  xavier_normal_(scale, gain): N(0, gain * sqrt(scale / (fan_in[+fan_out])))     (init.py:104-116)
  lecun_uniform_: U(+-sqrt(3 / fan_in)); lecun_normal_: truncated N with std sqrt(1/fan_in)/0.8796...
"""
import math
import warnings

import torch.nn as nn


def _simple(fn, *args):
    def initializer(tensor, fan_in=None, fan_out=None):
        return fn(tensor, *args)
    return initializer


def zeros_():
    return _simple(nn.init.zeros_)


def ones_():
    return _simple(nn.init.ones_)


def uniform_(a: float = 0.0, b: float = 1.0):
    return _simple(nn.init.uniform_, a, b)


def normal_(mean: float = 0.0, std: float = 1.0):
    return _simple(nn.init.normal_, mean, std)


def trunc_normal_(mean: float = 0.0, std: float = 1.0, a: float = -2.0, b: float = 2.0):
    return _simple(nn.init.trunc_normal_, mean, std, a, b)


def _pick_fan(mode, fan_in, fan_out):
    if mode == "fan_in":
        assert fan_in is not None, "Fan_in is not provided."
        return fan_in
    if mode == "fan_out":
        assert fan_out is not None, "Fan_out is not provided."
        return fan_out
    raise ValueError(f"Invalid initialization mode '{mode}'")


def _kaiming(a, mode, nonlinearity, uniform):
    def initializer(tensor, fan_in=None, fan_out=None):
        if 0 in tensor.shape:
            warnings.warn("Initializing zero-element tensors is a no-op")
            return tensor
        std = nn.init.calculate_gain(nonlinearity, a) / math.sqrt(_pick_fan(mode, fan_in, fan_out))
        if uniform:
            bound = math.sqrt(3.0) * std
            return nn.init.uniform_(tensor, -bound, bound)
        return nn.init.normal_(tensor, 0, std)
    return initializer


def kaiming_uniform_(a=0, mode="fan_in", nonlinearity="leaky_relu"):
    return _kaiming(a, mode, nonlinearity, True)


def kaiming_normal_(a=0, mode="fan_in", nonlinearity="leaky_relu"):
    return _kaiming(a, mode, nonlinearity, False)


def _xavier_std(scale, gain, fan_in, fan_out):
    assert fan_in is not None, "Fan_in is not provided."
    fan = fan_in + (fan_out if fan_out is not None else 0)
    return gain * math.sqrt(scale / float(fan))


def xavier_uniform_(a: float = math.sqrt(3.0), scale: float = 2.0, gain: float = 1.0):
    def initializer(tensor, fan_in=None, fan_out=None):
        bound = a * _xavier_std(scale, gain, fan_in, fan_out)
        return nn.init.uniform_(tensor, -bound, bound)
    return initializer


def xavier_normal_(scale: float = 2.0, gain: float = 1.0):
    def initializer(tensor, fan_in=None, fan_out=None):
        return nn.init.normal_(tensor, 0.0, _xavier_std(scale, gain, fan_in, fan_out))
    return initializer


def lecun_uniform_():
    def initializer(tensor, fan_in=None, fan_out=None):
        assert fan_in is not None, "Fan_in is not provided."
        bound = math.sqrt(3.0 / fan_in)
        return nn.init.uniform_(tensor, -bound, bound)
    return initializer


def lecun_normal_():
    def initializer(tensor, fan_in=None, fan_out=None):
        assert fan_in is not None, "Fan_in is not provided."
        return nn.init.trunc_normal_(tensor, std=math.sqrt(1.0 / fan_in) / 0.87962566103423978)
    return initializer
