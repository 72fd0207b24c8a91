"""The two device probes behind the roofline figures (matrix pipe rate, LDS read rate) run and return sane values."""
import pytest
from pooled_amd.capi import PooledAttn
from helpers import SHAPES

pytestmark = pytest.mark.gpu


def test_mfma_and_lds_probe():
    with PooledAttn(SHAPES["qwen36_moe"], 64, n_layers=1, max_cols=1) as pa:
        for mode in (1, 2):                                             # random operands: 32x32x16 tiles, 16x16x32 tiles
            tf, mhz = pa.mfma_probe(mode, 2000)
            assert 500.0 < tf < 2600.0 and 500.0 < mhz < 3000.0, (mode, tf, mhz)
        for tr in (0, 1):
            for waves in (4, 8):
                bpc = pa.lds_probe(tr, waves, 2000)
                assert 30.0 < bpc <= 260.0, (tr, waves, bpc)       # a CU's LDS delivers at most 256 bytes a clock
