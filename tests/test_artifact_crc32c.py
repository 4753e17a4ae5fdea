"""CRC32C against the literals both sides of the reference pin
(modelexpress_common/src/artifact_manifest.rs:382-384, tests/test_artifact_manifest.py:53-67)."""

import zlib

import pytest

from modelexpress_amd.artifact_manifest import build_checksums, crc32c


def test_pinned_vectors(mxp):
    _pinned_vectors()


@pytest.mark.gpu
def test_pinned_vectors_on_the_gpu_box(mxp):
    """The same literals where the GPU tests run: the host there takes the SSE4.2 ``crc32`` path."""
    _pinned_vectors()


def _pinned_vectors():
    assert crc32c(b"xyz") == "25236885"
    assert crc32c(b"abcd") == "92c80a31"
    assert crc32c(b"ef") == "6bb2dff5"
    assert crc32c(b"abcdef") == "53bceff1"
    assert crc32c(b"123456789") == "e3069283"  # the standard CRC-32C check value
    assert crc32c(b"") == "00000000"
    # append semantics: continuing a finished CRC equals one pass
    assert crc32c(b"ef", seed=int(crc32c(b"abcd"), 16)) == crc32c(b"abcdef")
    blob = bytes(range(256)) * 41 + b"tail"
    assert crc32c(blob[100:], seed=int(crc32c(blob[:100]), 16)) == crc32c(blob)
    assert crc32c(blob) != format(zlib.crc32(blob), "08x")  # not the zlib polynomial


def test_manifest_chunks_and_files(mxp, tmp_path):
    nested = tmp_path / "nested"
    nested.mkdir()
    (nested / "b.bin").write_bytes(b"abcdef")
    (tmp_path / "a.txt").write_bytes(b"xyz")
    (tmp_path / "empty").write_bytes(b"")
    files, chunks = build_checksums(str(tmp_path), 4)
    assert [f.path for f in files] == [(tmp_path / "a.txt").resolve().as_posix(), (tmp_path / "empty").resolve().as_posix(),
                                       (nested / "b.bin").resolve().as_posix()]
    assert [f.checksum for f in files] == ["25236885", "00000000", "53bceff1"]
    assert [(c.chunk_index, c.file_index, c.file_offset, c.length, c.checksum) for c in chunks] == [
        (0, 0, 0, 3, "25236885"), (1, 2, 0, 4, "92c80a31"), (2, 2, 4, 2, "6bb2dff5")]
    big = tmp_path / "big.bin"
    data = bytes((i * 7 + 3) & 0xFF for i in range(5 * (1 << 20) + 17))
    big.write_bytes(data)
    files, chunks = build_checksums(str(tmp_path), 1 << 20)
    bf = [f for f in files if f.path.endswith("big.bin")][0]
    assert bf.checksum == crc32c(data)
    bc = [c for c in chunks if c.file_index == bf.file_index]
    assert len(bc) == 6 and bc[-1].length == 17 and bc[2].checksum == crc32c(data[2 << 20:3 << 20])
