"""Pins the CPU oracle against the known answers recorded from the reference's
own C code (tests/golden/reference_kat.json).  CPU only."""
import numpy as np

import oracle
from helpers import check_digest, kat_conv_inputs, kat_pool_inputs, load_kat

KAT = load_kat()


def _conv_case(cfg):
    inp, weight, bias, go = kat_conv_inputs(cfg)
    geo = (cfg["kH"], cfg["kW"], cfg["pH"], cfg["pW"], cfg["sH"], cfg["sW"])
    out, finput = oracle.conv_updateOutput(inp, weight, bias, *geo)
    gi, fgi = oracle.conv_updateGradInput(go, weight, inp.shape, *geo)
    gw = np.zeros_like(weight)
    gb = np.zeros_like(bias)
    oracle.conv_accGradParameters(go, finput, gw, gb, cfg["scale"])
    return dict(finput=finput, output=out, fgradInput=fgi, gradInput=gi, gradWeight=gw, gradBias=gb)


def test_conv_stride1_padded_matches_reference_vectors():
    cfg = KAT["conv_stride1"]
    got = _conv_case(cfg)
    for name in ("finput", "output", "fgradInput", "gradInput", "gradWeight", "gradBias"):
        check_digest(got[name], cfg[name])


def test_conv_strided_asymmetric_pad_matches_reference_vectors():
    cfg = KAT["conv_strided"]
    got = _conv_case(cfg)
    for name in ("output", "gradInput", "gradWeight"):
        check_digest(got[name], cfg[name])


def test_maxpool_overlapping_ties_match_reference_vectors():
    cfg = KAT["maxpool_overlap_ties"]
    inp, go = kat_pool_inputs(cfg)
    out, ind = oracle.maxpool_updateOutput(inp, cfg["kH"], cfg["kW"], cfg["dH"], cfg["dW"])
    assert np.all(out == cfg["output_all"])
    assert ind[0].ravel().tolist() == [float(v) for v in cfg["indices_y"]]
    assert ind[1].ravel().tolist() == [float(v) for v in cfg["indices_x"]]
    gi = oracle.maxpool_updateGradInput(go, ind, inp.shape, cfg["dH"], cfg["dW"])
    assert np.array_equal(gi[0], np.array(cfg["gradInput"], np.float32))
