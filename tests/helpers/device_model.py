"""Runs a model spec on the device decoder (through the C ABI) the same way run_sequences drives the oracle."""
import numpy as np


def device_decoder(cai, spec, **kw):
    return cai.Decoder(spec, **kw)


def run_sequences_device(dec, seqs):
    out = []
    for s in seqs:
        dec.reset()
        out.append([dec.step(t, p)[1][0] for p, t in enumerate(s)])
    return np.array(out, np.float32)
