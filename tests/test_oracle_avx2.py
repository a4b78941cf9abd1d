"""The AVX2 restatement of the TNN GEMM (oracle/ftnn_oracle_avx2.c, the benchmark's CPU baseline where the compiled
reference is absent) against the scalar oracle and, where present, the compiled reference: bit-identical.  CPU only."""
import numpy as np
import pytest

from fastertnn_amd import synth, TNN
from oracle.ftnn_oracle import OracleAvx2, aligned_copy

pytestmark = pytest.mark.skipif(not OracleAvx2.available(), reason="no AVX2 on this CPU")


def operands(oracle, m, n, k, seed):
    a = oracle.pack_gemm_operand(synth.ternary(seed, (m, k)))
    b = oracle.pack_gemm_operand(synth.ternary(seed + 1, (n, k)))
    return aligned_copy(a), aligned_copy(b)


@pytest.mark.parametrize("m,n,k", [(1, 1, 256), (3, 5, 256), (4, 7, 512), (9, 16, 1024), (64, 33, 4096), (256, 256, 4096)])
@pytest.mark.parametrize("alpha", [0.5, 1.0])
def test_avx2_gemm_equals_the_scalar_oracle(oracle, m, n, k, alpha):
    a, b = operands(oracle, m, n, k, seed=900 + m + n)
    got = OracleAvx2().mm(TNN, a, b, m, 1, 1, n, k // 64, alpha)
    want = oracle.mm(TNN, a, b, m, 1, 1, n, k // 64, alpha)
    assert got.tobytes() == want.tobytes()


def test_avx2_gemm_nchw_store_and_word_counts_that_round_up(oracle):
    """a conv-shaped result (OH * OW > 1, rows no multiple of 4) and K words that the row layout rounds up to 4"""
    rng = np.random.default_rng(5)
    n, oh, ow, kn, k = 2, 3, 3, 5, 6          # 18 rows, 6 -> 8 words per plane
    kw = 8
    def rows(count):
        r = rng.integers(0, 2 ** 63, size=(count, kw // 4, 2, 4), dtype=np.int64)
        r[:, :, 0, :] &= ~r[:, :, 1, :]       # no lane both negative and zero
        r[:, -1, 0, 2:] = 0                   # the two pad words: sign 0, zero all-ones
        r[:, -1, 1, 2:] = -1
        return aligned_copy(r.reshape(-1))
    a, b = rows(n * oh * ow), rows(kn)
    got = OracleAvx2().mm(TNN, a, b, n, oh, ow, kn, k, 0.5)
    want = oracle.mm(TNN, a, b, n, oh, ow, kn, k, 0.5)
    assert got.tobytes() == want.tobytes()


def test_avx2_gemm_equals_the_compiled_reference(oracle, reference):
    a, b = operands(oracle, 130, 96, 2048, seed=77)
    got = OracleAvx2().mm(TNN, a, b, 130, 1, 1, 96, 32, 0.5)
    want = reference.mm(TNN, a, b, 130, 1, 1, 96, 32, 0.5)
    assert got.tobytes() == np.ascontiguousarray(want).tobytes()
