"""Rotary position tables: the frequency of every pair of columns, from a mixer's constants."""

import math

import torch


def rotary_table(dims, base, scaling=None, device=None):
    """``(inv_freq float32 [dims / 2], factor for cos and sin)``: ``f_i = base^(-2i / dims)``.

    With ``scaling = {factor, original, fast, slow}`` (the interpolation by wavelength known as
    YaRN): pairs that turn more than ``fast`` times within ``original`` positions keep ``f_i``,
    pairs that turn fewer than ``slow`` times get ``f_i / factor``, a linear ramp over the pair
    index between the two; cos and sin are multiplied by ``0.1 ln(factor) + 1``.  Computed in
    float64 on the host, once, when the weights are loaded."""
    dims, base = int(dims), float(base)
    if dims % 2 or dims < 0:
        raise ValueError(f"{dims} turning columns: an even number is needed")
    f = [base ** (-2.0 * i / dims) for i in range(dims // 2)]
    mult = 1.0
    if scaling:
        factor, original = float(scaling["factor"]), float(scaling["original"])

        def pair_of(turns):
            return dims * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(base))

        lo = max(math.floor(pair_of(float(scaling["fast"]))), 0)
        hi = min(math.ceil(pair_of(float(scaling["slow"]))), dims - 1)
        for i, fi in enumerate(f):
            ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
            f[i] = fi / factor * ramp + fi * (1.0 - ramp)
        mult = 0.1 * math.log(factor) + 1.0
    return torch.tensor(f, dtype=torch.float64).float().to(device), mult
