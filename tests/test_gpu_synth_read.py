"""The streaming-read kernels the benchmark measures ceilings with (libdsx_synth.so) read exactly the
bytes they are said to read: the words they fold together are checked against numpy."""
import numpy as np
import pytest

torch = pytest.importorskip("torch")

from deepstrix_amd import synth

pytestmark = pytest.mark.gpu


def _xor_words(a: np.ndarray) -> int:
    return int(np.bitwise_xor.reduce(a.view(np.uint32).ravel()))


def test_plain_read_folds_every_word_once():
    rng = np.random.default_rng(5)
    host = rng.integers(0, 256, 3 * 1024 * 1024 + 48, dtype=np.uint8)
    src = torch.from_numpy(host).cuda()
    for wgs in (7, 64, 0):
        sink = torch.zeros(4 * 4096, dtype=torch.int32, device="cuda")
        synth.read_dev(sink, src, wgs)
        torch.cuda.synchronize()
        assert _xor_words(sink.cpu().numpy()) == _xor_words(host), wgs


@pytest.mark.parametrize("n_sb", [1, 3, 4, 8, 28])
def test_tile_reads_fold_the_tiles_they_name(n_sb):
    """Memory order: every byte of the first n_tiles tiles once.  Operand order: every nibble byte
    once and the scale bytes once per lane group (four times: they cancel)."""
    n_tiles, row_bytes = 24, n_sb * 136
    rng = np.random.default_rng(n_sb)
    host = rng.integers(0, 256, (n_tiles + 2) * 16 * row_bytes, dtype=np.uint8)   # two tiles that must stay unread
    src = torch.from_numpy(host).cuda()
    region = host[: n_tiles * 16 * row_bytes].reshape(n_tiles * 16, n_sb, 136)
    want_all = _xor_words(np.ascontiguousarray(region))
    want_nibbles = _xor_words(np.ascontiguousarray(region[:, :, :128]))
    for operand, want in ((False, want_all), (True, want_nibbles)):
        sink = torch.zeros(4 * n_tiles, dtype=torch.int32, device="cuda")
        synth.read_tiles_dev(sink, src, n_tiles, n_sb, operand)
        torch.cuda.synchronize()
        assert _xor_words(sink.cpu().numpy()) == want, (n_sb, operand)
