"""mi_matmul_parse_param (host logic of the C ABI, no GPU needed) against the cases the reference documents above
tpu::MatMulOp::parseParam (lib/Dialect/Tpu/Interfaces/Common/MatMul.cpp:17-22) and against the oracle's restatement on
every combination of the transpose flags."""
import pytest

from helpers import pkg

DOCUMENTED = [((5, 6), (6, 7), (5, 7), (1, 5, 6, 7)), ((1, 512, 7, 7), (25088, 4096), (1, 4096), (1, 1, 25088, 4096)),
              ((3, 4, 5, 6), (3, 4, 6, 7), (3, 4, 5, 7), (12, 5, 6, 7)), ((4, 5, 6), (6, 7), (4, 5, 7), (1, 20, 6, 7)),
              ((4, 5, 6), (6,), (4, 5), (1, 20, 6, 1)), ((4096,), (4096, 12884), (12884,), (1, 1, 4096, 12884))]


@pytest.mark.parametrize("a,b,o,expect", DOCUMENTED)
def test_parse_param_documented_cases_and_oracle(orc, a, b, o, expect):
    m = pkg()
    p = m.matmul_parse_param(a, b, o)
    assert (p["batch"], p["M"], p["K"], p["N"]) == expect       # MatMul.cpp:17-22
    assert p == orc.matmul_parse_param(a, b, o)


def test_parse_param_matches_oracle_on_every_flag(orc):
    m = pkg()
    clib = pkg("clib")
    shapes = [((2, 5, 3, 6), (2, 6, 3, 7), (2, 5, 3, 7)), ((2, 3, 5, 6), (2, 6, 3, 7), (2, 3, 5, 7)),
              ((2, 5, 6), (2, 7, 6), (2, 5, 7)), ((2, 3, 5, 6), (6, 7), (2, 3, 5, 7)), ((2, 5, 3, 6), (2, 7, 3, 6), (2, 5, 3, 7))]
    for a, b, o in shapes:
        for rt in (False, True):
            for lt in (False, True):
                for ot in (False, True):
                    for hd in (False, True):
                        for chip, ochip in ((clib.CHIP_BM168X, orc.CHIP_BM1684X), (clib.CHIP_CV18XX, orc.CHIP_CV18XX),
                                            (clib.CHIP_BM1684, orc.CHIP_OTHER)):
                            kw = dict(right_transpose=rt, left_transpose=lt, output_transpose=ot, hdim_is_batch=hd)
                            try:
                                want = orc.matmul_parse_param(a, b, o, chip=ochip, **kw)
                            except ValueError:  # shapes the reference asserts on: refused here as well
                                with pytest.raises(clib.BackendError):
                                    m.matmul_parse_param(a, b, o, chip=chip, **kw)
                                continue
                            assert m.matmul_parse_param(a, b, o, chip=chip, **kw) == want, (a, b, o, kw, chip)


def test_parse_param_tells_bm1684_from_the_bm1684x_family():
    """MatMul.cpp:63-72: under hdim_is_batch a transposed right operand (B0, K, B1, N) gives K = shape[-3],
    N = shape[-1]; only the BM1684X / BM1690 families swap the two."""
    m = pkg()
    clib = pkg("clib")
    a, b, o = (2, 5, 3, 6), (2, 6, 3, 7), (2, 5, 3, 7)
    kw = dict(right_transpose=True, hdim_is_batch=True)
    plain = m.matmul_parse_param(a, b, o, chip=clib.CHIP_BM1684, **kw)
    swapped = m.matmul_parse_param(a, b, o, chip=clib.CHIP_BM168X, **kw)
    assert (plain["K"], plain["N"]) == (6, 7) and (swapped["K"], swapped["N"]) == (7, 6)
