"""Register images of the gfx950 matrix instructions, built from logical matrices.

This is the Python statement of the layouts documented in clpeak_amd/csrc/mfma_common.h;
tests/test_gpu_layouts.py feeds these images to single instructions (mi355_mfma_raw) and
compares with exact integer matrix products, which is what pins the layouts."""
import numpy as np


def pack_codes(codes, bits):
    """codes[..., K] -> bytes[..., K*bits/8], little-endian bit order along K."""
    codes = np.asarray(codes, dtype=np.uint32)
    if bits == 16:
        return codes.astype("<u2").view(np.uint8).reshape(codes.shape[:-1] + (-1,))
    if bits == 8:
        return codes.astype(np.uint8)
    b = ((codes[..., None] >> np.arange(bits, dtype=np.uint32)) & 1).astype(np.uint8)
    return np.packbits(b.reshape(codes.shape[:-1] + (-1,)), axis=-1, bitorder="little")


def operand_regs(rows_bytes, rows_mod, dwords):
    """rows_bytes[R][row_bytes] -> regs[64][dwords] (uint32): lane l holds chunk l // rows_mod
    of row l % rows_mod, where a row is split into 64 // rows_mod equal chunks."""
    R, rb = rows_bytes.shape
    assert R == rows_mod
    chunks = 64 // rows_mod
    cb = rb // chunks
    regs = np.zeros((64, dwords * 4), dtype=np.uint8)
    for l in range(64):
        regs[l, :cb] = rows_bytes[l % rows_mod, (l // rows_mod) * cb:(l // rows_mod + 1) * cb]
    return regs.view("<u4").reshape(64, dwords)


def split_k_regs(rows_bytes):
    """rows_bytes[16][128] -> regs[64][8]: lane l holds bytes [16g, 16g+16) and
    [64+16g, 64+16g+16) of row l % 16, g = l // 16 (two half-K operands back to back).
    This is the B operand of every SMFMAC and both operands of the 8-bit f8f6f4 MFMA."""
    assert rows_bytes.shape == (16, 128)
    regs = np.zeros((64, 32), dtype=np.uint8)
    for l in range(64):
        g = l // 16
        regs[l, :16] = rows_bytes[l % 16, 16 * g:16 * g + 16]
        regs[l, 16:] = rows_bytes[l % 16, 64 + 16 * g:64 + 16 * g + 16]
    return regs.view("<u4").reshape(64, 8)


def c_regs_from_matrix(Cm):
    """C[M][N] (4-byte elements) -> regs[64][16]."""
    M, N = Cm.shape
    regs = np.zeros((64, 16), dtype=np.uint32)
    v = Cm.view(np.uint32)
    for l in range(64):
        if M == 16:
            for r in range(4):
                regs[l, r] = v[4 * (l // 16) + r, l % 16]
        else:
            for r in range(16):
                regs[l, r] = v[8 * (r // 4) + 4 * (l // 32) + r % 4, l % 32]
    return regs


def matrix_from_d_regs(regs, M, N, dtype):
    out = np.zeros((M, N), dtype=np.uint32)
    for l in range(64):
        if M == 16:
            for r in range(4):
                out[4 * (l // 16) + r, l % 16] = regs[l, r]
        else:
            for r in range(16):
                out[8 * (r // 4) + 4 * (l // 32) + r % 4, l % 32] = regs[l, r]
    return out.view(dtype)


def scale_regs(scales, byte):
    """scales[16][4] E8M0 bytes -> regs[64]: lane l carries scales[l % 16][l // 16] in `byte`;
    the other bytes get a decoy (a different exponent) so a wrong byte selection shows."""
    regs = np.zeros(64, dtype=np.uint32)
    for l in range(64):
        s = int(scales[l % 16, l // 16])
        word = 0
        for b in range(4):
            word |= (s if b == byte else ((s + 3 + b) & 0x7f) | 0x40) << (8 * b)
        regs[l] = word
    return regs


def sparse_index_regs(meta, groups_per_lane, half):
    """meta[16][K/4] -> regs[64]: lane l packs the nibbles of groups
    [(l//16)*gpl, (l//16+1)*gpl) from bit 0 (or from bit 16 when half == 1; 16-bit kinds
    use 16 index bits and ABID names the half)."""
    regs = np.zeros(64, dtype=np.uint32)
    for l in range(64):
        word = 0
        for g in range(groups_per_lane):
            word |= (int(meta[l % 16, (l // 16) * groups_per_lane + g]) & 0xf) << (4 * g)
        if groups_per_lane == 4:
            decoy = (~word) & 0xffff
            word = (word << 16 | decoy) if half == 1 else (decoy << 16 | word)
        regs[l] = word
    return regs
