"""Independent pure-Python (numpy float32) model of the sampler's definition, for small inputs.

Written from the prose definition, not from the C oracle: quartets aligned to the absolute CSR index;
groups of 64 lanes x 4 quartets; lane totals in (quartet, element) order; wave scan tree (row_shr 1,2,4,8,
row_bcast 15, row_bcast 31); sequential reservoir over group totals with jump acceptance S*u > Sj; inverse
transform inside the accepted group; inverse transform over the wave totals for the workgroup sampler.
"""
import numpy as np

f32 = np.float32
M0, M1 = 0xD2511F53, 0xCD9E8D57


def philox(ctr, key):
    c = list(ctr)
    k = list(key)
    for _ in range(10):
        p0 = M0 * c[0]
        p1 = M1 * c[2]
        c = [((p1 >> 32) ^ c[1] ^ k[0]) & 0xFFFFFFFF, p1 & 0xFFFFFFFF, ((p0 >> 32) ^ c[3] ^ k[1]) & 0xFFFFFFFF,
             p0 & 0xFFFFFFFF]
        k = [(k[0] + 0x9E3779B9) & 0xFFFFFFFF, (k[1] + 0xBB67AE85) & 0xFFFFFFFF]
    return c


def uniform(seed, walker, step, stream, n):
    bits = philox([walker, step, stream, n >> 2], [seed & 0xFFFFFFFF, seed >> 32])[n & 3]
    return f32(bits >> 8) * f32(2.0 ** -24)


def wave_scan(x):
    x = [f32(v) for v in x]
    for off in (1, 2, 4, 8):
        x = [x[l] + x[l - off] if (l % 16) >= off else x[l] for l in range(64)]
    r0, r2 = x[15], x[47]
    x = [x[l] + r0 if 16 <= l < 32 else (x[l] + r2 if 48 <= l < 64 else x[l]) for l in range(64)]
    h = x[31]
    return [x[l] + h if l >= 32 else x[l] for l in range(64)]


def row_scan(x):
    x = [f32(v) for v in x]
    for off in (1, 2, 4, 8):
        x = [x[l] + x[l - off] if l >= off else x[l] for l in range(len(x))]
    return x


def pick_by_prefix(v, prefix, target):
    last = -1
    for i in range(len(v)):
        if v[i] > 0:
            if prefix[i] > target:
                return i
            last = i
    return last


def sample(bias, off, nw, seed, walker, step, U=4):
    """bias: float32 biases of the list; off: absolute CSR offset of its first element (alignment matters)."""
    deg = len(bias)
    if deg == 0:
        return -1
    a0 = off & ~3
    end = off + deg
    nq = (end - a0 + 3) // 4
    G = 64 * U
    ngroups = (nq + G - 1) // G
    W, wsel = [], []
    for wv in range(nw):
        S, Sj, u = f32(0), f32(0), f32(1)
        sel, nd = -1, 0
        for g in range(wv, ngroups, nw):
            x = [[f32(0)] * (4 * U) for _ in range(64)]
            q = []
            for l in range(64):
                s = f32(0)
                for j in range(U):
                    k = g * G + j * 64 + l
                    for e in range(4):
                        a = a0 + 4 * k + e
                        b = f32(bias[a - off]) if (k < nq and off <= a < end) else f32(0)
                        x[l][4 * j + e] = b
                        s = s + b
                q.append(s)
            I = wave_scan(q)
            T = I[63]
            Snew = S + T
            if Snew * u > Sj:
                target = uniform(seed, walker, step, wv, nd) * T
                nd += 1
                lane = pick_by_prefix(q, I, target)
                e = I[lane] - q[lane]
                pre = []
                for i in range(4 * U):
                    e = e + x[lane][i]
                    pre.append(e)
                pick = pick_by_prefix(x[lane], pre, target)
                k = g * G + (pick // 4) * 64 + lane
                sel = a0 + 4 * k + (pick % 4) - off
                Sj = Snew
                u = uniform(seed, walker, step, wv, nd)
                nd += 1
            S = Snew
        W.append(S)
        wsel.append(sel)
    if nw == 1:
        return wsel[0]
    J = row_scan(W)
    target = uniform(seed, walker, step, 0x40000000, 0) * J[nw - 1]
    wv = pick_by_prefix(W, J, target)
    return -1 if wv < 0 else wsel[wv]
