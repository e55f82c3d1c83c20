"""Stage-by-stage CPU restatement of the 16-token chunk pipeline the HIP kernels run.  TEST INFRASTRUCTURE ONLY.

The shipped HIP library splits the chunked operator of ``HRDPLR/hrdplr.py:25-99`` (forward) and ``:149-284``
(backward) into four device stages.  This module spells out the same stages in torch (float64 by default) with
a hand-written backward, so that

* the algebra the kernels implement is checked on the CPU against autograd through the token recurrence
  (``tests/test_chunk_stages.py``) before any of it runs on a GPU, and
* every intermediate buffer a kernel writes can be compared with a named tensor here.

Differences from the reference's chunk form (``HRDPLR/naive.py:107-255``), all mathematically neutral:

* the chunk length is fixed at 16 tokens (the only length for which the reference backward is complete,
  ``HRDPLR/bwd_func.py:299``), ragged tails are padded with zero vectors and zero log-decay;
* rows of a/b inside a chunk are held rank-major (row ``r*16 + i``) instead of token-major (``2*i + r``);
* the decayed scores are factorised around the chunk's 8th token, ``exp(gi_i - gi_j) = exp(gi_i - m) exp(m - gi_j)``
  with ``m = gi[7]``, so every score matrix is one dense product (the reference re-centres per 16-row
  sub-chunk the same way, ``HRDPLR/fwd_triton.py:420-463``);
* ``w`` and ``u`` come from the blocks of ``(I - A_ab)^-1`` exactly as in ``HRDPLR/fwd_triton.py:739-789``.
"""
from typing import Dict, Optional

import torch

C = 16          # tokens per chunk
MID = 7         # index of the token whose cumulative decay centres the factorisation


def _pad_T(x, T_pad):
    if x.shape[1] == T_pad:
        return x
    pad = x.new_zeros(x.shape[0], T_pad - x.shape[1], *x.shape[2:])
    return torch.cat([x, pad], 1)


def _chunks(x, rows):
    # [B, NT*rows, H, D] -> [B, H, NT, rows, D]
    B, TR, H, D = x.shape
    return x.reshape(B, TR // rows, rows, H, D).permute(0, 3, 1, 2, 4)


def prep(q, k, v, a, b, gk, scale, R=2, dtype=torch.float64) -> Dict[str, torch.Tensor]:
    """Per-chunk quantities that do not depend on the state (prep kernel)."""
    B, T, H, K = q.shape
    NT = (T + C - 1) // C
    Tp = NT * C
    q, k, v, gk = (_pad_T(x.to(dtype), Tp) for x in (q, k, v, gk))
    a, b = (_pad_T(x.to(dtype), Tp * R) for x in (a, b))
    q, k, v, gk = (_chunks(x, C) for x in (q, k, v, gk))                  # [B,H,NT,C,D]
    # token-major (2i+r) -> rank-major [B,H,NT,R,C,K]
    a = _chunks(a, C * R).reshape(B, H, NT, C, R, K).transpose(3, 4)
    b = _chunks(b, C * R).reshape(B, H, NT, C, R, K).transpose(3, 4)
    gi = gk.cumsum(-2)
    ge = gi - gk
    m = gi[..., MID:MID + 1, :]
    gl = gi[..., C - 1:C, :]
    qh = scale * q * torch.exp(gi - m)
    kh = k * torch.exp(m - gi)
    ah = a * torch.exp(ge - m)[..., None, :, :]
    bh = b * torch.exp(m - gi)[..., None, :, :]
    qg = scale * q * torch.exp(gi)
    kg = k * torch.exp(gl - gi)
    ag = a * torch.exp(ge)[..., None, :, :]
    bg = b * torch.exp(gl - gi)[..., None, :, :]
    le = torch.tril(torch.ones(C, C, dtype=dtype))                        # j <= i
    lt = torch.tril(torch.ones(C, C, dtype=dtype), -1)                    # j <  i
    Aqk = (qh @ kh.transpose(-1, -2)) * le                                # [B,H,NT,C,C]
    Aqb = (qh[..., None, :, :] @ bh.transpose(-1, -2)) * le               # [B,H,NT,R(s),C,C]
    Aak = (ah @ kh[..., None, :, :].transpose(-1, -2)) * lt               # [B,H,NT,R(r),C,C]
    Aab = (ah[..., :, None, :, :] @ bh[..., None, :, :, :].transpose(-1, -2)) * lt   # [B,H,NT,R(r),R(s),C,C]
    # (I - A_ab)^-1 on the 2C x 2C matrix in rank-major order
    big = Aab.permute(0, 1, 2, 3, 5, 4, 6).reshape(B, H, NT, R * C, R * C)
    eye = torch.eye(R * C, dtype=dtype)
    Tm_big = torch.linalg.inv(eye - big)
    Tm = Tm_big.reshape(B, H, NT, R, C, R, C).permute(0, 1, 2, 3, 5, 4, 6)  # [.., r, s, C, C]
    w = torch.einsum('...rsij,...sjk->...rik', Tm, ag)                     # [B,H,NT,R,C,K]
    M = Aak @ v[..., None, :, :]                                           # [B,H,NT,R,C,V]
    u = torch.einsum('...rsij,...sjv->...riv', Tm, M)
    return dict(q=q, k=k, v=v, a=a, b=b, gk=gk, gi=gi, ge=ge, m=m, gl=gl, qh=qh, kh=kh, ah=ah, bh=bh,
                qg=qg, kg=kg, ag=ag, bg=bg, Aqk=Aqk, Aqb=Aqb, Aak=Aak, Aab=Aab, Tm=Tm, w=w, u=u, M=M)


def scan_fwd(p, h0):
    """Inter-chunk state scan (forward scan kernel): per chunk the entering state h, v_new and o."""
    B, H, NT = p['q'].shape[:3]
    K, V = p['q'].shape[-1], p['v'].shape[-1]
    S = h0.to(p['q'].dtype) if h0 is not None else p['q'].new_zeros(B, H, K, V)
    hs, vns, os_ = [], [], []
    for n in range(NT):
        hs.append(S)
        Sx = S[:, :, None]                                                 # broadcast over rank
        vn = p['w'][:, :, n] @ Sx + p['u'][:, :, n]                        # [B,H,R,C,V]
        o = p['qg'][:, :, n] @ S + p['Aqk'][:, :, n] @ p['v'][:, :, n] + (p['Aqb'][:, :, n] @ vn).sum(2)
        S = torch.exp(p['gl'][:, :, n]).transpose(-1, -2) * S + p['kg'][:, :, n].transpose(-1, -2) @ p['v'][:, :, n] \
            + (p['bg'][:, :, n].transpose(-1, -2) @ vn).sum(2)
        vns.append(vn)
        os_.append(o)
    return dict(h=torch.stack(hs, 2), vn=torch.stack(vns, 2), o=torch.stack(os_, 2), ht=S)


def scan_bwd(p, do, dht):
    """Reverse state-gradient scan (reverse scan kernel): per chunk the gradient dh of the state LEAVING the
    chunk and dvn, the gradient of v_new."""
    B, H, NT = p['q'].shape[:3]
    K, V = p['q'].shape[-1], p['v'].shape[-1]
    dS = dht.to(p['q'].dtype) if dht is not None else p['q'].new_zeros(B, H, K, V)
    dhs, dvns = [None] * NT, [None] * NT
    for n in range(NT - 1, -1, -1):
        dhs[n] = dS
        do_n = do[:, :, n]
        dvn = p['Aqb'][:, :, n].transpose(-1, -2) @ do_n[:, :, None] + p['bg'][:, :, n] @ dS[:, :, None]   # [B,H,R,C,V]
        dS = torch.exp(p['gl'][:, :, n]).transpose(-1, -2) * dS + p['qg'][:, :, n].transpose(-1, -2) @ do_n \
            + (p['w'][:, :, n].transpose(-1, -2) @ dvn).sum(2)
        dvns[n] = dvn
    return dict(dh=torch.stack(dhs, 2), dvn=torch.stack(dvns, 2), dh0=dS)


def bwd_chunk(p, f, r, do, scale):
    """Per-chunk gradient assembly (chunk gradient kernel).  ``f`` = scan_fwd output, ``r`` = scan_bwd output."""
    S, dS, vn, dvn = f['h'], r['dh'], f['vn'], r['dvn']
    v, gi, ge, m, gl = p['v'], p['gi'], p['ge'], p['m'], p['gl']
    T_ = lambda x: x.transpose(-1, -2)
    dtype = v.dtype
    le = torch.tril(torch.ones(C, C, dtype=dtype))
    lt = torch.tril(torch.ones(C, C, dtype=dtype), -1)
    # products whose inner dimension is V
    dqg = do @ T_(S)                                                       # [B,H,NT,C,K]
    dkg = v @ T_(dS)
    dbg = vn @ T_(dS)[:, :, :, None]                                       # [B,H,NT,R,C,K]
    dw = dvn @ T_(S)[:, :, :, None]
    dgl = torch.exp(gl) * T_((S * dS).sum(-1, keepdim=True)) \
        + (dkg * p['kg']).sum(-2, keepdim=True) + (dbg * p['bg']).sum((-2, -3))[..., None, :]
    dAqk = (do @ T_(v)) * le
    dAqb = (do[:, :, :, None] @ T_(vn)) * le                               # [.., s, C, C]
    # WY representation backward:  [w|u] = Tm [ag | Aak v]
    Tm = p['Tm']                                                           # [.., r, s, i, j]
    dag = torch.einsum('...srji,...sjk->...rik', Tm, dw)                   # dR_r = sum_s Tm[s][r]^T dX_s
    dM = torch.einsum('...srji,...sjv->...riv', Tm, dvn)
    dAak = (dM @ T_(v)[:, :, :, None]) * lt                                # [.., r, C, C]
    dAab = (torch.einsum('...rik,...sjk->...rsij', dag, p['w'])
            + torch.einsum('...riv,...sjv->...rsij', dM, p['u'])) * lt
    dv = T_(p['Aqk']) @ do + p['kg'] @ dS + (T_(p['Aak']) @ dM).sum(3)
    # score matrices backward
    qh, kh, ah, bh = p['qh'], p['kh'], p['ah'], p['bh']
    dqh = dAqk @ kh + (dAqb @ bh).sum(3)
    dkh = T_(dAqk) @ qh + (T_(dAak) @ ah).sum(3)
    dah = dAak @ kh[:, :, :, None] + torch.einsum('...rsij,...sjk->...rik', dAab, bh)
    dbh = T_(dAqb) @ qh[:, :, :, None] + torch.einsum('...rsij,...rik->...sjk', dAab, ah)
    e = torch.exp
    dq = scale * (dqh * e(gi - m) + dqg * e(gi))
    dk = dkh * e(m - gi) + dkg * e(gl - gi)
    da = dah * e(ge - m)[:, :, :, None] + dag * e(ge)[:, :, :, None]
    db = dbh * e(m - gi)[:, :, :, None] + dbg * e(gl - gi)[:, :, :, None]
    Dgi = dq * p['q'] - dk * p['k'] - (db * p['b']).sum(3)
    Dge = (da * p['a']).sum(3)
    tot = Dgi + Dge
    rev = tot.flip(-2).cumsum(-2).flip(-2)                                  # inclusive reverse cumsum over tokens
    dgk = rev - Dge + dgl
    return dict(dq=dq, dk=dk, dv=dv, da=da, db=db, dgk=dgk, dqg=dqg, dkg=dkg, dbg=dbg, dw=dw, dgl=dgl,
                dAqk=dAqk, dAqb=dAqb, dAak=dAak, dAab=dAab, dag=dag, dM=dM, dqh=dqh, dkh=dkh, dah=dah, dbh=dbh)


def _unchunk(x, T):
    # [B,H,NT,C,D] -> [B,T,H,D]
    B, H, NT, Cc, D = x.shape
    return x.permute(0, 2, 3, 1, 4).reshape(B, NT * Cc, H, D)[:, :T]


def _unchunk_ab(x, T, R):
    # rank-major [B,H,NT,R,C,K] -> token-major [B,T*R,H,K]
    B, H, NT, R_, Cc, K = x.shape
    return x.permute(0, 2, 4, 3, 1, 5).reshape(B, NT * Cc * R, H, K)[:, :T * R]


def forward(q, k, v, a, b, gk, scale, h0=None, R=2, dtype=torch.float64):
    T = q.shape[1]
    p = prep(q, k, v, a, b, gk, scale, R, dtype)
    f = scan_fwd(p, h0)
    return _unchunk(f['o'], T), f['ht'], p, f


def forward_backward(q, k, v, a, b, gk, scale, h0, do, dht, R=2, dtype=torch.float64):
    """Full hand-written forward + backward; returns (o, ht, grads dict, all stage dicts)."""
    B, T, H, K = q.shape
    o, ht, p, f = forward(q, k, v, a, b, gk, scale, h0, R, dtype)
    NT = p['q'].shape[2]
    do_c = _chunks(_pad_T(do.to(dtype), NT * C), C)
    r = scan_bwd(p, do_c, dht)
    g = bwd_chunk(p, f, r, do_c, scale)
    grads = dict(dq=_unchunk(g['dq'], T), dk=_unchunk(g['dk'], T), dv=_unchunk(g['dv'], T),
                 da=_unchunk_ab(g['da'], T, R), db=_unchunk_ab(g['db'], T, R), dgk=_unchunk(g['dgk'], T),
                 dh0=r['dh0'])
    return o, ht, grads, dict(p=p, f=f, r=r, g=g)
