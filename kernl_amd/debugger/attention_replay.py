"""Replay of one key-tile step of the streaming attention kernel (csrc/attention.hip) on the host.

Staging, the K fragment reads, the transposing V reads, both MFMA phases and the final register-to-feature mapping are
walked lane by lane with the kernel's own address functions; the results are compared with plain matrix products.
What a replay proves: every byte of the K and V tiles is staged exactly once, every lane's operand fragments hold the
elements the instruction layouts call for, the key order of P and of Vᵀ agree, each lane ends with 16 consecutive
output features of its query row, and (in the LDS model's terms) no read pattern has bank conflicts.
"""
from dataclasses import dataclass

import numpy as np

from kernl_amd.debugger.index_lib import index_lib
from kernl_amd.debugger.lds import AccessStats, Lds
from kernl_amd.debugger.wave_ops import mfma32, transposing_read_b64

BN = 64  # keys per tile


@dataclass
class TileReplay:
    scores_t: np.ndarray      # [4 waves, 64 lanes, 2 blocks, 16]: Sᵀ registers
    out_regs: np.ndarray      # [4 waves, 64 lanes, D / 32, 16]: Oᵀ registers
    reads: AccessStats
    writes: AccessStats


def stage_tiles(lds: Lds, k_tile: np.ndarray, v_tile: np.ndarray, stage_base: int = 0) -> None:
    """The 16-byte chunks of a K and a V tile [64, D] (float16) go to LDS the way the tile loads put them there:
    thread tid's i-th load writes position tid + 256 i; a wave's load writes 1 KB of consecutive LDS."""
    ix = index_lib()
    D = k_tile.shape[1]
    k_bytes = BN * D * 2
    loads = BN * (D // 8) // 256
    kb, vb = k_tile.astype(np.float16), v_tile.astype(np.float16)
    for i in range(loads):
        for wave in range(4):
            k_addr, k_data, v_addr, v_data = [], [], [], []
            for lane in range(64):
                qd = wave * 64 + lane + 256 * i
                row = ix.attention(D, "stage_row", qd)
                kc, vc = ix.attention(D, "k_stage_chunk", qd), ix.attention(D, "v_stage_chunk", qd)
                k_addr.append(stage_base + qd * 16)
                k_data.append(kb[row, kc * 8:kc * 8 + 8].tobytes())
                v_addr.append(stage_base + k_bytes + qd * 16)
                v_data.append(vb[row, vc * 8:vc * 8 + 8].tobytes())
            lds.wave_write(k_addr, k_data, 16, "stage K")
            lds.wave_write(v_addr, v_data, 16, "stage V")


def replay_tile(q_rows: np.ndarray, k_tile: np.ndarray, v_tile: np.ndarray) -> TileReplay:
    """q_rows [128, D], k_tile / v_tile [64, D], float16 values.  P is taken to be Sᵀ rounded to float16 (the softmax
    in between is lane-local arithmetic, not addressing)."""
    ix = index_lib()
    D = q_rows.shape[1]
    assert q_rows.shape == (128, D) and k_tile.shape == (BN, D) and v_tile.shape == (BN, D) and D in (64, 128)
    krow, vp = D * 2, D * 2
    k_bytes = BN * krow
    lds = Lds(k_bytes + BN * vp)
    stage_tiles(lds, k_tile, v_tile)
    if not (lds.once_written(0, k_bytes + BN * vp)):
        raise AssertionError("staging does not write every byte of the K and V tiles exactly once")

    ks_steps, blocks, dblocks = D // 16, BN // 32, D // 32
    q16 = q_rows.astype(np.float16)
    scores = np.zeros((4, 64, blocks, 16))
    outs = np.zeros((4, 64, dblocks, 16))
    for wave in range(4):
        # ---- Sᵀ = K Qᵀ: K fragments from LDS ("A" side), Q fragments from registers ("B" side)
        s_acc = np.zeros((blocks, 64, 16))
        for nb in range(blocks):
            for ks in range(ks_steps):
                addrs = [nb * 32 * krow + ix.attention(D, "k_frag_offset", lane % 32, lane // 32, ks) for lane in range(64)]
                raw = lds.wave_read(addrs, 16, "K fragment")
                a = np.stack([np.frombuffer(r, dtype=np.float16).astype(np.float64) for r in raw])
                b = np.stack([q16[wave * 32 + lane % 32, 16 * ks + 8 * (lane // 32):16 * ks + 8 * (lane // 32) + 8].astype(np.float64)
                              for lane in range(64)])
                s_acc[nb] = mfma32(a, b, s_acc[nb])
        # ---- Oᵀ += Vᵀ Pᵀ: P from the score registers, Vᵀ through the transposing read
        p16 = s_acc.astype(np.float16).astype(np.float64)
        o_acc = np.zeros((dblocks, 64, 16))
        for ps in range(BN // 16):
            nb, half8 = ps >> 1, (ps & 1) * 8
            b = p16[nb][:, half8:half8 + 8]
            for d in range(dblocks):
                base = [k_bytes + 16 * ps * vp + ix.attention(D, "v_frag_offset", lane, d) for lane in range(64)]
                lo = transposing_read_b64(lds, base, "V fragment")
                hi = transposing_read_b64(lds, [x + 8 * vp for x in base], "V fragment")
                a = np.stack([np.concatenate([lo[lane], hi[lane]]).view(np.float16).astype(np.float64) for lane in range(64)])
                o_acc[d] = mfma32(a, b, o_acc[d])
        scores[wave] = np.transpose(s_acc, (1, 0, 2))
        outs[wave] = np.transpose(o_acc, (1, 0, 2))
    return TileReplay(scores, outs, lds.reads, lds.writes)


def check_tile(q_rows: np.ndarray, k_tile: np.ndarray, v_tile: np.ndarray, atol: float = 1e-6) -> TileReplay:
    """Replays the tile and compares every register with the matrix products it should hold."""
    D = q_rows.shape[1]
    r = replay_tile(q_rows, k_tile, v_tile)
    q, k, v = (t.astype(np.float16).astype(np.float64) for t in (q_rows, k_tile, v_tile))
    s_t = k @ q.T                                             # [64 keys, 128 rows]
    p = s_t.astype(np.float16).astype(np.float64)
    o = p.T @ v                                               # [128 rows, D]
    for wave in range(4):
        for lane in range(64):
            lr, lh = lane % 32, lane // 32
            m = wave * 32 + lr
            for nb in range(BN // 32):
                for e in range(16):
                    key = 32 * nb + 8 * (e // 4) + 4 * lh + e % 4
                    if abs(r.scores_t[wave, lane, nb, e] - s_t[key, m]) > atol * max(1.0, abs(s_t[key, m])):
                        raise AssertionError(f"score register: wave {wave} lane {lane} block {nb} element {e} is not key {key} x row {m}")
            for d in range(D // 32):
                for e in range(16):
                    f = 32 * d + 16 * lh + e
                    if abs(r.out_regs[wave, lane, d, e] - o[m, f]) > atol * max(1.0, abs(o[m, f])):
                        raise AssertionError(f"output register: wave {wave} lane {lane} block {d} element {e} is not row {m} feature {f}")
    return r


def check_mask_tile(mask_rows: np.ndarray) -> Lds:
    """Matrix-mask staging of one wave (head size 64): mask_rows [32 query rows, 64 keys], float32 or a 16-bit dtype.
    Stages the rows through the wave's LDS region as the direct-to-LDS loads do and reads them back as the lanes do;
    lane (lr, lh) must get keys 8 j + 4 lh .. + 3 of its row lr from its j-th read."""
    ix = index_lib()
    es = mask_rows.dtype.itemsize
    assert mask_rows.shape == (32, 64) and es in (2, 4)
    row_bytes = 64 * es
    lds = Lds(32 * row_bytes)
    for i in range(32 * row_bytes // 1024):
        addrs, data = [], []
        for lane in range(64):
            r, c = ix.mask(es, "stage_row", i, lane), ix.mask(es, "stage_chunk", i, lane)
            addrs.append(1024 * i + 16 * lane)
            data.append(mask_rows[r].tobytes()[16 * c:16 * c + 16])
        lds.wave_write(addrs, data, 16, "stage mask")
    if not lds.once_written(0, 32 * row_bytes):
        raise AssertionError("mask staging does not write every byte of the wave's region exactly once")
    width = 4 * es
    for j in range(8):
        addrs = [ix.mask(es, "read_offset", lane % 32, lane // 32, j) for lane in range(64)]
        got = lds.wave_read(addrs, width, "mask read")
        for lane in range(64):
            lr, lh = lane % 32, lane // 32
            want = mask_rows[lr, 8 * j + 4 * lh:8 * j + 4 * lh + 4].tobytes()
            if got[lane] != want:
                raise AssertionError(f"mask read {j} of lane {lane} is not keys {8 * j + 4 * lh}.. of row {lr}")
    return lds
