"""Host restatement of the 2-bit packed ternary weight layout.

The reference stores no quantised weights (mmfreelm/ops/fusedbitnet.py:456
re-quantises the latent matrix on every forward); the layout is this build's.
A weight [N, K] is padded to Np = ceil32(N), Kp = ceil128(K) with code 0 and cut
into blocks of 32 output rows x 128 inputs.  A block is 64 lanes x 4 dwords
(1 KiB); dword s of lane l = (half = l // 32, row = l % 32) holds the 16 inputs
    k = kb*128 + s*32 + half*16 + i,   i = 0..15,
input i stored as the 2-bit field (t + 1) at bit 8*(i % 4) + 2*(i // 4), so that
(dword >> 2j) & 0x03030303 is four byte-wide codes for i = 4j .. 4j+3.
Blocks are ordered [Np/32][Kp/128].
"""
import numpy as np


def packed_shape(n, k):
    npad, kpad = -(-n // 32) * 32, -(-k // 128) * 128
    return npad, kpad, (npad // 32) * (kpad // 128) * 256   # dwords


def pack_ternary(t):
    """t: int8 array [N, K] in {-1,0,1} -> uint32 array of packed_shape(N,K)[2] dwords."""
    t = np.asarray(t, dtype=np.int8)
    n, k = t.shape
    npad, kpad, _ = packed_shape(n, k)
    c = np.ones((npad, kpad), dtype=np.uint32)
    c[:n, :k] = (t.astype(np.int32) + 1).astype(np.uint32)
    # [nb, row, kb, s, half, i]
    c = c.reshape(npad // 32, 32, kpad // 128, 4, 2, 16)
    i = np.arange(16)
    shift = (8 * (i % 4) + 2 * (i // 4)).astype(np.uint32)
    dw = np.bitwise_or.reduce(c << shift, axis=-1)       # [nb, row, kb, s, half]
    dw = dw.transpose(0, 2, 4, 1, 3)                     # [nb, kb, half, row, s]
    return np.ascontiguousarray(dw).reshape(-1).astype(np.uint32)


def unpack_ternary(p, n, k):
    npad, kpad, nd = packed_shape(n, k)
    p = np.asarray(p, dtype=np.uint32).reshape(npad // 32, kpad // 128, 2, 32, 4)
    i = np.arange(16)
    shift = (8 * (i % 4) + 2 * (i // 4)).astype(np.uint32)
    c = (p[..., None] >> shift) & 3                      # [nb, kb, half, row, s, i]
    c = c.transpose(0, 3, 1, 4, 2, 5).reshape(npad, kpad)
    return (c.astype(np.int32) - 1).astype(np.int8)[:n, :k]
