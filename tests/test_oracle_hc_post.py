"""Pins the oracle's hyper-connection combine (crates/v4flash-kernels/kernels/hc_post.hip:15-34,
40-64, 66-98, 100-141) without retyping its loop: the closed form as a float64 einsum, cases that
reduce to a copy or a scale, and a mixing matrix that is not symmetric, so that reading
comb[src + dst * n_hc] for comb[dst + src * n_hc] fails.  CPU only."""
import numpy as np
import pytest

from oracle import ref


def _inputs(b, n_hc, n_embd, seed):
    rng = np.random.default_rng(seed)
    block = rng.standard_normal((b, n_embd)).astype(np.float32)
    res = rng.standard_normal((b, n_hc, n_embd)).astype(np.float32)
    post = rng.uniform(0.2, 1.5, (b, n_hc)).astype(np.float32)
    comb = rng.standard_normal((b, n_hc, n_hc)).astype(np.float32)   # memory order [src][dst]
    return block, res, post, comb


@pytest.mark.parametrize("b,n_hc,n_embd", [(1, 4, 64), (3, 4, 256), (2, 1, 32), (5, 7, 20), (2, 8, 128)])
def test_closed_form_in_float64(b, n_hc, n_embd):
    block, res, post, comb = _inputs(b, n_hc, n_embd, 7 * b + n_hc)
    got = ref.hc_post(block, res, post, comb)
    # out[t, dst, :] = block[t] post[t, dst] + sum_src comb_mem[t, src, dst] res[t, src, :]
    want = (block.astype(np.float64)[:, None, :] * post.astype(np.float64)[:, :, None]
            + np.einsum("tsd,tse->tde", comb.astype(np.float64), res.astype(np.float64)))
    assert got.shape == want.shape
    scale = np.abs(want).max()
    assert np.abs(got - want).max() < 4e-7 * n_hc * scale
    # the transposed reading of the mixing matrix is far away, so the bound above tells them apart
    wrong = (block.astype(np.float64)[:, None, :] * post.astype(np.float64)[:, :, None]
             + np.einsum("tds,tse->tde", comb.astype(np.float64), res.astype(np.float64)))
    if n_hc > 1:
        assert np.abs(got - wrong).max() > 1e-2 * scale


def test_cases_that_reduce_to_a_copy_a_scale_and_a_permutation():
    b, n_hc, n_embd = 2, 4, 48
    block, res, post, comb = _inputs(b, n_hc, n_embd, 3)
    eye = np.broadcast_to(np.eye(n_hc, dtype=np.float32), (b, n_hc, n_hc)).copy()
    # post = 0, comb = identity: the residual streams come back bit for bit
    assert np.array_equal(ref.hc_post(block, res, np.zeros_like(post), eye), res)
    # comb = 0: every stream is the block output times its post factor (one rounding each)
    got = ref.hc_post(block, res, post, np.zeros_like(comb))
    assert np.array_equal(got, block[:, None, :] * post[:, :, None])
    # a one-hot comb in memory position [src=1][dst=2] routes stream 1 into output stream 2 only
    one = np.zeros_like(comb)
    one[:, 1, 2] = 1.0
    got = ref.hc_post(block, res, np.zeros_like(post), one)
    want = np.zeros_like(res)
    want[:, 2, :] = res[:, 1, :]
    assert np.array_equal(got, want)


def test_addends_and_the_packed_split_row():
    b, n_hc, n_embd, n_w = 3, 4, 64, 5
    block, res, post, comb = _inputs(b, n_hc, n_embd, 11)
    rng = np.random.default_rng(12)
    a1 = rng.standard_normal((b, n_embd)).astype(np.float32)
    a2 = rng.standard_normal((b, n_embd)).astype(np.float32)
    # (block_out + add1) + add2 in f32, in that order (hc_post.hip:100-141)
    summed = (block + a1) + a2
    assert np.array_equal(ref.hc_post(block, res, post, comb, a1, a2), ref.hc_post(summed, res, post, comb))
    assert np.array_equal(ref.hc_post(block, res, post, comb, a1), ref.hc_post(block + a1, res, post, comb))
    # post and comb read from split[b, n_w + n_hc + n_hc^2] (hc_post.hip:66-98)
    split = np.concatenate([rng.standard_normal((b, n_w)).astype(np.float32), post,
                            comb.reshape(b, n_hc * n_hc)], axis=1)
    assert np.array_equal(ref.hc_post_from_split(block, res, split, n_w), ref.hc_post(block, res, post, comb))
