"""CPU restatement of the CASTLE (causal attention with lookahead keys) hot path.

TEST INFRASTRUCTURE ONLY: imported by tests/, __graft_entry__.smoke() and the
cpu_baseline leg of bench.py.  The product package never imports it.

Every function cites the reference lines it restates
(LKA = lookahead_keys_attention/lookahead_keys_attention.py,
 TRI = lookahead_keys_attention/lookahead_keys_attention_triton.py of the reference).

How each function is pinned (tests/test_oracle_*.py):
  parallel_core      brute-force triple loop from the paper definition, the
                     vu=0 case that must equal torch SDPA(is_causal), the qu=0
                     closed form (A = 1/2 -> cumulative sums), Su[i,i]=0,
                     U[L-1]=0, causality, and equality with decode_core.
  decode_core        equality with parallel_core token by token; t=0 closed form.
  closed_form_grads  torch.autograd of parallel_core in fp64 (and the vu=0 SDPA
                     gradient), so a wrong sign / transposed operand fails.
  blockwise_*        equality with parallel_core / closed_form_grads (these two
                     restate the O(L^2 d) state form the HIP kernels implement
                     and expose its intermediate tensors).
  module_forward     the reference's own test properties (parallel == cached
                     sequential, causality) with default-initialised weights.
  lm_forward         composition of module_forward with library routines (embedding,
                     rms_norm, gelu, cross_entropy): parallel == cached sequential,
                     causality, loss = ln(vocabulary) for zero logits weights, and the
                     wiring cases a missing residual or a misplaced norm would fail: with
                     every attention and feed-forward output projection zeroed the logits
                     are rms_norm(embedding) @ W exactly; with only the feed-forward ones
                     zeroed the hidden state is embedding + sum of the layers' attention
                     outputs, each computed by module_forward on the running state.
  rope               rotary embedding written as a complex multiplication; pinned by its
                     closed-form properties (tests/test_oracle_core.py): position 0 is the
                     identity, norms are kept, R(p) R(q) = R(p + q), the dot product of two
                     rotated rows depends on the position difference only, and pair i at
                     position p turns by exactly p * 10000^(-2i/d) radians.  The reference
                     delegates rotary embedding to `rotary-embedding-torch>=0.8.9`
                     (LKA:13,73,112; pyproject.toml:29), which is absent: agreement with
                     THAT package is parity unpinned; this is the published RoPE formula
                     over interleaved pairs, which is what that package documents.
"""
from __future__ import annotations

import math
from collections import namedtuple

import torch
import torch.nn.functional as F

OracleCache = namedtuple("OracleCache", ("U", "qu_cache", "kc_cache", "vc_cache"))  # LKA:26


# --------------------------------------------------------------------------
# dense parallel core                                                LKA:132-164
# --------------------------------------------------------------------------
def lookahead_gate(qu, ku, scale):
    """A[k, j] = sigmoid(scale * qu_k . ku_j) for j > k, else 0   (LKA:145-146)."""
    L = qu.shape[-2]
    z = torch.matmul(qu * scale, ku.transpose(-1, -2))
    keep = torch.ones(L, L, dtype=torch.bool, device=qu.device).triu(1)
    return torch.sigmoid(z) * keep


def parallel_scores(qc, kc, qu, ku, vu, scale):
    """Masked score matrix S = Sc - silu(Su) with -max above the diagonal (LKA:134-153)."""
    L = qc.shape[-2]
    q = qc * scale
    lower = torch.ones(L, L, dtype=torch.bool, device=qc.device).tril(0)
    T = torch.matmul(q, vu.transpose(-1, -2)) * lower            # LKA:142-143
    A = lookahead_gate(qu, ku, scale)                            # LKA:145-146
    Su = torch.matmul(T, A.transpose(-1, -2))                    # LKA:148
    Sc = torch.matmul(q, kc.transpose(-1, -2))                   # LKA:150
    S = Sc - F.silu(Su)                                          # LKA:152
    S = S.masked_fill(~lower, -torch.finfo(S.dtype).max)         # LKA:36-37,153
    return S, Su, A, T


def parallel_core(qc, kc, vc, qu, ku, vu, scale, want_U=False):
    """out (and U = A @ vu when want_U) for (..., L, d) operands     (LKA:132-164)."""
    S, _, A, _ = parallel_scores(qc, kc, qu, ku, vu, scale)
    P = S.softmax(dim=-1)                                        # LKA:156
    out = torch.matmul(P, vc)                                    # LKA:159
    if not want_U:
        return out
    return out, torch.matmul(A, vu)                              # LKA:161-163


# --------------------------------------------------------------------------
# rotary position embedding                                      LKA:71-73,106-112
# --------------------------------------------------------------------------
def rope(t, positions, theta=10000.0):
    """Rows of t (..., n, d) rotated by their absolute positions (n,): the pair
    (t[2i], t[2i+1]) is read as the complex number t[2i] + 1j t[2i+1] and multiplied by
    exp(1j * position * theta^(-2i/d)).  LKA:112 applies this to qc, kc, qu, ku, vu with
    offset = number of cached rows."""
    d = t.shape[-1]
    z = torch.view_as_complex(t.double().reshape(*t.shape[:-1], d // 2, 2).contiguous())
    freq = torch.tensor([theta ** (-2.0 * i / d) for i in range(d // 2)], dtype=torch.float64)
    turn = torch.polar(torch.ones(len(positions), d // 2, dtype=torch.float64),
                       positions.double()[:, None] * freq[None, :])
    return torch.view_as_real(z * turn).reshape(t.shape).to(t.dtype)


# --------------------------------------------------------------------------
# cached single-token step                                           LKA:166-203
# --------------------------------------------------------------------------
def decode_core(cache, qc, kc, vc, qu, ku, vu, scale):
    """One cached step.  New-token operands are (..., 1, d); cache is a 4-tuple of
    (..., t, d) tensors or None.  Returns (out (...,1,d), OracleCache)."""
    if cache is None:                                            # LKA:169-171
        empty = qu[..., 0:0, :]
        cache = (empty, empty, empty, empty)
    U_prev, qu_hist, kc_hist, vc_hist = cache
    gate = torch.sigmoid(torch.matmul(qu_hist * scale, ku.transpose(-1, -2)))   # LKA:180-182
    U_now = torch.cat((U_prev + gate * vu, torch.zeros_like(qu)), dim=-2)       # LKA:183-185
    kc_all = torch.cat((kc_hist, kc), dim=-2)                    # LKA:187
    vc_all = torch.cat((vc_hist, vc), dim=-2)                    # LKA:188
    q = qc * scale
    Sc = torch.matmul(q, kc_all.transpose(-1, -2))               # LKA:190
    Su = torch.matmul(q, U_now.transpose(-1, -2))                # LKA:191
    P = (Sc - F.silu(Su)).softmax(dim=-1)                        # LKA:194-197
    out = torch.matmul(P, vc_all)                                # LKA:200
    return out, OracleCache(U_now, torch.cat((qu_hist, qu), dim=-2), kc_all, vc_all)  # LKA:202-203


# --------------------------------------------------------------------------
# module wrapper (no rotary)                                LKA:42-80, 82-214
# --------------------------------------------------------------------------
def default_init(dim, heads, dim_head, seed, prenorm=False, dtype=torch.float32):
    """Weights the reference module gets from torch.manual_seed(seed) followed by its
    constructor: to_all_qkv (LKA:75) is created before combine_heads (LKA:80); RMSNorm
    (LKA:67) and the rearrange layers draw nothing from the generator."""
    torch.manual_seed(seed)
    inner = heads * dim_head
    w_qkv = torch.nn.Linear(dim, inner * 6, bias=False).weight.detach().clone()
    w_out = torch.nn.Linear(inner, dim, bias=False).weight.detach().clone()
    params = {"to_all_qkv.weight": w_qkv.to(dtype), "combine_heads.weight": w_out.to(dtype)}
    if prenorm:
        params["norm.weight"] = torch.ones(dim, dtype=dtype)
    return params


def split_projection(proj, heads):
    """(B, n, 6*H*d) -> six (B, H, n, d) views in the order qu, ku, vu, qc, kc, vc (LKA:77,104)."""
    B, n, width = proj.shape
    d = width // (6 * heads)
    parts = proj.view(B, n, 6, heads, d).permute(2, 0, 3, 1, 4)
    return tuple(parts[i] for i in range(6))


def module_forward(x, params, heads, cache=None, return_next_cache=None):
    """Functional restatement of Castle.forward (LKA:82-214).  A `rotary_emb.freqs` entry in
    `params` (the state entry of the reference's rotary submodule, LKA:71-73) switches the rotary
    embedding on: qc, kc, qu, ku, vu are rotated by their absolute positions, offset by the number
    of cached rows (LKA:106-112); the rotation is `rope` above, not the third-party module."""
    w_qkv, w_out = params["to_all_qkv.weight"], params["combine_heads.weight"]
    d = w_qkv.shape[0] // (6 * heads)
    scale = d ** -0.5                                            # LKA:63
    n = x.shape[1]
    single = n == 1                                              # LKA:89
    if return_next_cache is None:
        return_next_cache = single                               # LKA:91
    if "norm.weight" in params:                                  # LKA:67,95 (RMSNorm, eps=None)
        x = F.rms_norm(x, (x.shape[-1],), params["norm.weight"])
    qu, ku, vu, qc, kc, vc = split_projection(x @ w_qkv.t(), heads)   # LKA:99-104
    if "rotary_emb.freqs" in params:                             # LKA:106-112
        offset = cache[2].shape[-2] if cache is not None else 0
        pos = torch.arange(offset, offset + n)
        qc, kc, qu, ku, vu = (rope(t, pos) for t in (qc, kc, qu, ku, vu))
    nxt = None
    if not single:
        assert cache is None, "must be inferencing single tokens if receiving cache"   # LKA:117
        if return_next_cache:
            o, U = parallel_core(qc, kc, vc, qu, ku, vu, scale, want_U=True)
            nxt = OracleCache(U, qu, kc, vc)                     # LKA:164
        else:
            o = parallel_core(qc, kc, vc, qu, ku, vu, scale)
    else:
        o, nxt = decode_core(cache, qc, kc, vc, qu, ku, vu, scale)
    B, H = o.shape[0], o.shape[1]
    y = o.permute(0, 2, 1, 3).reshape(B, n, H * d) @ w_out.t()   # LKA:207-209
    return (y, nxt) if return_next_cache else y                  # LKA:211-214


def lm_forward(tokens, params, heads, depth, return_loss=False, cache=None, return_next_cache=False):
    """Functional restatement of the reference's language model around the layer
    (train_triton.py:141-175): embedding, `depth` x [h += castle(h); h += ff(h)]
    with ff = RMSNorm, Linear(4x), GELU, Linear (train_triton.py:103-108), final RMSNorm, logits,
    and the shift-by-one cross entropy (train_triton.py:143-144,172-175).
    params: state-dict style keys of the module tree (token_emb.weight, layers.<i>.0.<castle key>,
    layers.<i>.1.{0,1,3}.weight, final_norm.weight, to_logits.weight)."""
    if return_loss:
        tokens, target = tokens[:, :-1], tokens[:, 1:]
    h = params["token_emb.weight"][tokens]
    nxt = []
    for i in range(depth):
        layer = {k[len(f"layers.{i}.0."):]: v for k, v in params.items() if k.startswith(f"layers.{i}.0.")}
        layer_cache = cache[i] if cache is not None else None
        if return_next_cache:
            y, c = module_forward(h, layer, heads, cache=layer_cache, return_next_cache=True)
            nxt.append(c)
        else:
            y = module_forward(h, layer, heads, cache=layer_cache, return_next_cache=False)
        h = h + y
        f = F.rms_norm(h, (h.shape[-1],), params[f"layers.{i}.1.0.weight"])
        f = F.gelu(f @ params[f"layers.{i}.1.1.weight"].t()) @ params[f"layers.{i}.1.3.weight"].t()
        h = h + f
    logits = F.rms_norm(h, (h.shape[-1],), params["final_norm.weight"]) @ params["to_logits.weight"].t()
    if return_loss:
        return F.cross_entropy(logits.transpose(1, 2), target)
    return (logits, nxt) if return_next_cache else logits


# --------------------------------------------------------------------------
# brute force from the definition (tiny inputs only)
# --------------------------------------------------------------------------
def bruteforce_core(qc, kc, vc, qu, ku, vu, scale):
    """Triple loop over one head, (L, d) operands, python floats.

    Lookahead key of position k as seen from position i (paper fig. 3; recurrent form
    LKA:182-191):  U^i_k = sum_{k<j<=i} sigmoid(scale qu_k.ku_j) vu_j.
    score[i,k] = scale qc_i.kc_k - silu(scale qc_i.U^i_k),  k <= i;  softmax over k.
    Returns out (L,d) and the final lookahead keys U^{L-1} (L,d)."""
    L, d = qc.shape
    f = lambda t: [[float(v) for v in row] for row in t]
    qc_, kc_, vc_, qu_, ku_, vu_ = map(f, (qc, kc, vc, qu, ku, vu))
    dot = lambda a, b: sum(x * y for x, y in zip(a, b))
    sig = lambda z: 1.0 / (1.0 + math.exp(-z))
    out = [[0.0] * d for _ in range(L)]
    U_last = [[0.0] * d for _ in range(L)]
    for i in range(L):
        sc = []
        for k in range(i + 1):
            u = [0.0] * d
            for j in range(k + 1, i + 1):
                g = sig(scale * dot(qu_[k], ku_[j]))
                u = [a + g * b for a, b in zip(u, vu_[j])]
            if i == L - 1:
                U_last[k] = u
            su = scale * dot(qc_[i], u)
            sc.append(scale * dot(qc_[i], kc_[k]) - su * sig(su))
        m = max(sc)
        w = [math.exp(s - m) for s in sc]
        z = sum(w)
        for k in range(i + 1):
            for c in range(d):
                out[i][c] += w[k] / z * vc_[k][c]
    return torch.tensor(out, dtype=torch.float64), torch.tensor(U_last, dtype=torch.float64)


# --------------------------------------------------------------------------
# closed-form gradients of the dense core            (operator contract TRI:508-602)
# --------------------------------------------------------------------------
def closed_form_grads(qc, kc, vc, qu, ku, vu, scale, d_out):
    """Gradients of parallel_core's `out` w.r.t. the six operands, written out by hand
    (the quantities the reference's backward kernel forms at TRI:333-401):
        dVc = P^T dO;  dS = P*(dO Vc^T - rowsum(dO*O));  dSu = -dS*silu'(Su)
        dT = (dSu A)*[j<=i];  dA = (dSu^T T)*[j>k];  dZ = dA*A*(1-A)
        d(s qc) = dS Kc + dT Vu;  dKc = dS^T (s qc);  dVu = dT^T (s qc)
        d(s qu) = dZ Ku;  dKu = dZ^T (s qu);  dQc = s d(s qc);  dQu = s d(s qu)  (TRI:591-592)
    Returns (dqc, dkc, dvc, dqu, dku, dvu)."""
    L = qc.shape[-2]
    S, Su, A, T = parallel_scores(qc, kc, qu, ku, vu, scale)
    lower = torch.ones(L, L, dtype=torch.bool, device=qc.device).tril(0)
    P = S.softmax(dim=-1)
    O = P @ vc
    q, qus = qc * scale, qu * scale
    dVc = P.transpose(-1, -2) @ d_out
    delta = (d_out * O).sum(-1, keepdim=True)
    dS = P * (d_out @ vc.transpose(-1, -2) - delta)
    sg = torch.sigmoid(Su)
    dSu = -dS * sg * (1 + Su * (1 - sg))
    dT = (dSu @ A) * lower
    dA = (dSu.transpose(-1, -2) @ T) * torch.ones(L, L, dtype=torch.bool, device=qc.device).triu(1)
    dZ = dA * A * (1 - A)
    dq = dS @ kc + dT @ vu
    dKc = dS.transpose(-1, -2) @ q
    dVu = dT.transpose(-1, -2) @ q
    dqu = dZ @ ku
    dKu = dZ.transpose(-1, -2) @ qus
    return dq * scale, dKc, dVc, dqu * scale, dKu, dVu


# --------------------------------------------------------------------------
# O(L^2 d) state form with block snapshots (what the HIP kernels implement)
# --------------------------------------------------------------------------
def blockwise_forward(qc, kc, vc, qu, ku, vu, scale, nb):
    """State form of parallel_core for ONE head ((L, d) operands, L a multiple of nb).

    For query block I (rows I*nb .. I*nb+nb-1) and key k < I*nb the snapshot
        snap[I][k] = sum_{k<j<I*nb} A[k,j] vu_j
    is the lookahead key of k as of the start of block I, so that for i in block I
        Su[i,k] = (s qc_i).snap[I][k] + sum_{j in block I, k<j<=i} T[i,j] A[k,j].
    Row blocks are streamed: the gate columns of a block, its scores and its softmax are formed
    and dropped per block, so nothing of size L x L exists and L = 16384 fits a host.
    Returns dict(out, lse, U, snaps=[None, snap_1, ...], T=[T_II per block])."""
    L, d = qc.shape
    assert L % nb == 0
    nblk = L // nb
    q, qus = qc * scale, qu * scale
    state = torch.zeros(L, d, dtype=qc.dtype)
    snaps, Tblocks = [], []
    out = torch.empty_like(qc)
    lse = torch.empty(L, dtype=qc.dtype)
    tri = torch.ones(nb, nb, dtype=torch.bool).tril(0)
    for I in range(nblk):
        r = slice(I * nb, (I + 1) * nb)
        hi = (I + 1) * nb
        snaps.append(state[: I * nb].clone() if I > 0 else None)
        T_II = (q[r] @ vu[r].t()) * tri
        Tblocks.append(T_II)
        A_KI = _gate_columns(qus, ku, I, nb)
        Su = q[r] @ state[:hi].t() + T_II @ A_KI.t()
        Sblk = q[r] @ kc[:hi].t() - F.silu(Su)
        cols = torch.arange(hi)[None, :] <= torch.arange(I * nb, hi)[:, None]
        Sblk = torch.where(cols, Sblk, torch.full_like(Sblk, -float("inf")))
        lse[r] = torch.logsumexp(Sblk, dim=-1)
        out[r] = torch.exp(Sblk - lse[r, None]) @ vc[:hi]
        state[:hi] += A_KI @ vu[r]
    return {"out": out, "lse": lse, "U": state, "snaps": snaps, "T": Tblocks}


def _gate_columns(qus, ku, I, nb):
    """A[:hi, block I] of lookahead_gate: sigmoid(s qu_k . ku_j) for j in block I and k < j, else 0."""
    hi = (I + 1) * nb
    j = torch.arange(I * nb, hi)
    k = torch.arange(hi)
    return torch.sigmoid(qus[:hi] @ ku[I * nb:hi].t()) * (j[None, :] > k[:, None])


def blockwise_backward(qc, kc, vc, qu, ku, vu, scale, nb, d_out):
    """Reverse-state form of closed_form_grads for ONE head (L multiple of nb), row blocks streamed.

    gsnap[I][k] (k < (I+1)*nb) = sum_{i >= (I+1)*nb} dSu[i,k] (s qc_i) is the reverse
    state of key k as of query block I.  Returns dict(grads=(dqc,dkc,dvc,dqu,dku,dvu),
    gsnaps=[...] (only when keep_gsnaps), delta)."""
    return _blockwise_backward(qc, kc, vc, qu, ku, vu, scale, nb, d_out, keep_gsnaps=True)


def _blockwise_backward(qc, kc, vc, qu, ku, vu, scale, nb, d_out, keep_gsnaps):
    L, d = qc.shape
    nblk = L // nb
    fw = blockwise_forward(qc, kc, vc, qu, ku, vu, scale, nb)
    q, qus = qc * scale, qu * scale
    delta = (d_out * fw["out"]).sum(-1)
    dq = torch.zeros_like(qc); dKc = torch.zeros_like(qc); dVc = torch.zeros_like(qc)
    dqu = torch.zeros_like(qc); dKu = torch.zeros_like(qc); dVu = torch.zeros_like(qc)
    G = torch.zeros(L, d, dtype=qc.dtype)
    gsnaps = [None] * nblk
    tri = torch.ones(nb, nb, dtype=torch.bool).tril(0)
    for I in reversed(range(nblk)):
        r = slice(I * nb, (I + 1) * nb)
        hi = (I + 1) * nb
        if keep_gsnaps:
            gsnaps[I] = G[:hi].clone()
        Ub = torch.zeros(hi, d, dtype=qc.dtype)
        if I > 0:
            Ub[: I * nb] = fw["snaps"][I]
            fw["snaps"][I] = None   # consumed: blocks are visited once, from the last to the first
        T_II = fw["T"][I]
        A_KI = _gate_columns(qus, ku, I, nb)
        Su = q[r] @ Ub.t() + T_II @ A_KI.t()
        Sraw = q[r] @ kc[:hi].t() - F.silu(Su)
        cols = torch.arange(hi)[None, :] <= torch.arange(I * nb, hi)[:, None]
        P = torch.where(cols, torch.exp(Sraw - fw["lse"][r, None]), torch.zeros_like(Sraw))
        dS = P * (d_out[r] @ vc[:hi].t() - delta[r, None])
        sg = torch.sigmoid(Su)
        dSu = -dS * sg * (1 + Su * (1 - sg))
        dVc[:hi] += P.t() @ d_out[r]
        dKc[:hi] += dS.t() @ q[r]
        dTI = (dSu @ A_KI) * tri
        dq[r] += dS @ kc[:hi] + dSu @ Ub + dTI @ vu[r]
        dVu[r] += A_KI.t() @ G[:hi] + dTI.t() @ q[r]
        dA = dSu.t() @ T_II + G[:hi] @ vu[r].t()
        dZ = dA * A_KI * (1 - A_KI)          # A_KI already carries the j>k mask
        dqu[:hi] += dZ @ ku[r]
        dKu[r] += dZ.t() @ qus[:hi]
        G[:hi] += dSu.t() @ q[r]
    return {"out": fw["out"], "U": fw["U"], "grads": (dq * scale, dKc, dVc, dqu * scale, dKu, dVu), "gsnaps": gsnaps, "delta": delta}


def blockwise_head(qc, kc, vc, qu, ku, vu, scale, nb, d_out):
    """out, U and the six gradients of ONE head through the streamed state forms, keeping no
    reverse-state snapshots: the checker for full-length heads (L = 16384) that the dense
    functions cannot reach."""
    bw = _blockwise_backward(qc, kc, vc, qu, ku, vu, scale, nb, d_out, keep_gsnaps=False)
    return bw["out"], bw["U"], bw["grads"]
