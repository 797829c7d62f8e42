"""Host restatement, in numpy uint32 arithmetic, of the counter-based hash behind the kernels' dropout masks
(dropout_key / dropout_word / dropout_keep in triton-diff-attn_amd/csrc/common.hpp).  Test infrastructure:
the GPU test compares the library's mask dump with it bit for bit, the CPU tests check the hash's statistics."""
import numpy as np

_U = np.uint32


def _mul(a, c):
    return (a.astype(np.uint64) * np.uint64(c)).astype(_U)


def dropout_key(seed, stream_unit):
    """(k1, k2) of a 64-bit seed and a stream_unit = 2 * (batch*head unit) + softmax stream."""
    lo, hi = _U(seed & 0xFFFFFFFF), _U((seed >> 32) & 0xFFFFFFFF)
    su = np.asarray(stream_unit, dtype=_U)
    with np.errstate(over="ignore"):
        a = np.zeros_like(su) + (lo ^ _U(0x9E3779B9))
        a = _mul(a, 0x85EBCA6B); a ^= a >> _U(13)
        a = a + hi
        a = _mul(a, 0xC2B2AE35); a ^= a >> _U(16)
        a = a + su
        a = _mul(a, 0x27D4EB2F); a ^= a >> _U(15)
        a = _mul(a, 0x165667B1); a ^= a >> _U(13)
        b = a ^ _U(0x68E31DA4)
        b = _mul(b, 0xB5297A4D); b ^= b >> _U(15)
        b = b + (hi ^ _mul(su, 0x9E3779B1))
        b = _mul(b, 0x1B56C4E9); b ^= b >> _U(16)
    return a, b


def dropout_word(key, half_n, qh, kh):
    k1, k2 = key
    with np.errstate(over="ignore"):
        h = (np.asarray(qh, dtype=_U) * _U(half_n) + np.asarray(kh, dtype=_U)) ^ k1
        h = _mul(h, 0x9E3779B1); h ^= h >> _U(15)
        h = h + k2
        h = _mul(h, 0xC2B2AE3D); h ^= h >> _U(13)
        h = _mul(h, 0x27D4EB2F); h ^= h >> _U(16)
    return h


def words(seed, unit, stream, N):
    """The [N/2, N/2] hash words of one softmax stream of one (batch, head) unit."""
    qh, kh = np.meshgrid(np.arange(N // 2, dtype=_U), np.arange(N // 2, dtype=_U), indexing="ij")
    return dropout_word(dropout_key(seed, 2 * unit + stream), N // 2, qh, kh)


def keep_mask(seed, unit, stream, N, p):
    """Boolean [N, N] keep decisions: pair (q, k) owns byte 2*(q&1) + (k&1) of the word of its 2x2 block."""
    thr = int(p * 256.0 + 0.5)
    w = words(seed, unit, stream, N)
    out = np.empty((N, N), dtype=bool)
    for dq in (0, 1):
        for dk in (0, 1):
            byte = (w >> _U(8 * (2 * dq + dk))) & _U(0xFF)
            out[dq::2, dk::2] = byte >= thr
    return out
