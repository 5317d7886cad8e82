"""The oracle reproduces its committed golden vectors (regression pin; inputs come from seeds)."""

import os

import numpy as np
import torch

from areno_amd import workloads
from oracle import quant_ref as qr
from tests.golden.make_fixtures import decode_expected

GOLD = np.load(os.path.join(os.path.dirname(__file__), "golden", "oracle_vectors.npz"))


def test_decode_vectors():
    for kv in ("fp32", "bf16", "int8", "fp8"):
        for window in (-1, 40):
            w = workloads.cfg0_tiny(kv, quantize_fn=qr.quantize)
            got = decode_expected(w, window).numpy()
            np.testing.assert_allclose(got, GOLD[f"cfg0_decode_{kv}_w{window}"], rtol=0, atol=1e-6)


def test_quantizer_vectors_bit_exact():
    g = torch.Generator().manual_seed(4242)
    x = (torch.randn(8, 2, 64, generator=g) * torch.tensor([0.01, 1.0, 30.0, 1e-6]).repeat(2).view(8, 1, 1)).bfloat16()
    c8, s8 = qr.quantize_int8(x)
    cf, sf = qr.quantize_fp8(x)
    assert np.array_equal(c8.numpy(), GOLD["quant_int8_codes"]) and np.array_equal(s8.numpy(), GOLD["quant_int8_scales"])
    assert np.array_equal(cf.view(torch.uint8).numpy(), GOLD["quant_fp8_codes"])
    assert np.array_equal(sf.numpy(), GOLD["quant_fp8_scales"])
