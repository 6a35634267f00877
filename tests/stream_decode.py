"""NumPy decoder of the streaming KV format (test side restatement of the layout contract):
turns a unit's blob back into per-token K codes per slot, V codes, scale/zp and fp16 rows."""
import numpy as np

TILE = 64
V_TILE_BYTES = (2048, 4096, 8192, 16384)


def field_of(s, k, nf):
    return 2 * s + (k >> 1) + (k & 1) * (nf // 2)


def decode_unit(blob: np.ndarray, u, base: int):
    """blob: uint8 array of the layer's buffer; u: RdkvUnit record (absolute addresses);
    base: device address of blob[0].  Returns dict with K [T, 4*steps] codes, V codes per class
    [n, 128], sz [n_quantized, 2] raw fp16 bits, V16 [n16, 128] raw fp16 bits."""
    dw = blob.view(np.uint32)
    d8, d4, d2 = int(u["d8"]), int(u["d4"]), int(u["d2"])
    R = d8 + d4 + d2
    n_tok = [int(v) for v in u["n_tok"]]
    tiles = [-(-n // TILE) for n in n_tok]
    tstart = np.concatenate([[0], np.cumsum(tiles)])
    steps = d8 + 2 * d4 + 4 * d2
    k_off = (int(u["k_off"]) - base) // 4
    K_cls, V_cls = [], []
    for c in range(4):
        n = n_tok[c]
        Kc = np.zeros((n, 4 * steps), np.uint8)
        for tk in range(n):
            ti, t = tstart[c] + tk // TILE, tk % TILE
            for j in range(R):
                ck = j // 4
                wc = min(4, R - 4 * ck)
                w = int(dw[k_off + ti * TILE * R + 256 * ck + t * wc + j % 4])
                if j < d8:
                    nf, step0 = 4, j
                elif j < d8 + d4:
                    nf, step0 = 8, d8 + 2 * (j - d8)
                else:
                    nf, step0 = 16, d8 + 2 * d4 + 4 * (j - d8 - d4)
                fw = 32 // nf
                for s in range(nf // 4):
                    for k in range(4):
                        f = field_of(s, k, nf)
                        Kc[tk, 4 * (step0 + s) + k] = (w >> (fw * f)) & ((1 << fw) - 1)
        K_cls.append(Kc)
        v_off = (int(u["v_off"][c]) - base) // 4
        per_tile = V_TILE_BYTES[c] // 4
        Vc = np.zeros((n, 128), np.uint16)
        for tk in range(n):
            tl, t = tk // TILE, tk % TILE
            quad, k = t // 4, t % 4
            for ch in range(128):
                l, j = ch % 64, ch // 64
                if c == 3:
                    di = 4 * quad + 2 * j + (k >> 1)
                    w = int(dw[v_off + tl * per_tile + ((di >> 2) * 64 + l) * 4 + (di & 3)])
                    Vc[tk, ch] = (w >> (16 * (k & 1))) & 0xffff
                    continue
                if c == 2:
                    di, s, nf = 2 * quad + j, 0, 4
                elif c == 1:
                    di, s, nf = quad, j, 8
                else:
                    di, s, nf = quad >> 1, 2 * (quad & 1) + j, 16
                fw = 32 // nf
                w = int(dw[v_off + tl * per_tile + ((di >> 2) * 64 + l) * 4 + (di & 3)])
                Vc[tk, ch] = (w >> (fw * field_of(s, k, nf))) & ((1 << fw) - 1)
        V_cls.append(Vc)
    sz_off = (int(u["sz_off"]) - base) // 4
    sz = []
    for c in range(3):
        for tk in range(n_tok[c]):
            w = int(dw[sz_off + (tstart[c] + tk // TILE) * TILE + tk % TILE])
            sz.append((w & 0xffff, w >> 16))
    return dict(K=K_cls, V=V_cls, sz=np.array(sz, np.uint16).reshape(-1, 2))
