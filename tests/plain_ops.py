"""Plain torch versions of every HIP kernel, with the kernels' own signatures.

Two uses, both in tests only: (1) the reference each kernel is compared with on the GPU;
(2) patched over `minfer_amd.kernels.ops` (`install`), they let the CPU-only tests drive
the real engine, cache and generation loop where no GPU exists.  The product never imports
this file.  Arithmetic is float64 inside, rounded once to the output type.
"""
from __future__ import annotations

import math

import torch

PAGE = 64


def embed(table, ids, out):
    out.copy_(table[ids.long()].to(torch.float32))


def rmsnorm(x, weight, eps, out, row_idx=None, cols=None):
    src = x if row_idx is None else x[row_idx.long()]
    if cols is not None:
        src = src[:, :cols]
    s = src.double()
    y = s * (1.0 / torch.sqrt((s * s).mean(dim=-1, keepdim=True) + eps))
    if weight is not None:
        y = y * weight.double()
    out.copy_(y.to(out.dtype))


def rmsnorm_reference(x, weight, eps):
    """The norm alone, float64, unrounded."""
    s = x.double()
    return s * (1.0 / torch.sqrt((s * s).mean(dim=-1, keepdim=True) + eps)) * weight.double()


def gather_rows(x, idx, out):
    out.copy_(x[idx.long()])


def swiglu(gate_up, out):
    nf = gate_up.shape[1] // 2
    g, u = gate_up[:, :nf].double(), gate_up[:, nf:].double()
    out.copy_((g / (1.0 + torch.exp(-g)) * u).to(out.dtype))


def convert(src, dst):
    dst.copy_(src.to(dst.dtype))


def fill_normal(out, seed, std, round_bf16=True):
    """The library's own host fill: the numbers are defined by csrc/random_normal.h, on both sides."""
    from minfer_amd.kernels import ops
    ops.fill_normal_host(out, seed, std, round_bf16)


def rope_table(n_pos, half, theta, freq_scale, device):
    i = torch.arange(half, dtype=torch.float64)
    freq = freq_scale / torch.pow(torch.tensor(float(theta), dtype=torch.float64), 2.0 * i / (2 * half))
    ang = torch.arange(n_pos, dtype=torch.float64)[:, None] * freq[None, :]
    return torch.cos(ang).float().to(device), torch.sin(ang).float().to(device)


def rope_kvwrite(qkv, cos, sin, positions, seq_of_tok, page_table, q_out, kcache, vcache,
                 n_heads, n_kv_heads, head_dim, write_kv=True):
    t = positions.numel()
    half = head_dim // 2
    x = qkv.double().view(t, n_heads + 2 * n_kv_heads, head_dim)
    if cos is None:                      # nothing is rotated: q is rounded, k and v are stored
        c, s = torch.ones(t, 1, half, dtype=torch.float64), torch.zeros(t, 1, half, dtype=torch.float64)
    else:
        c = cos[positions.long()].double()[:, None, :]
        s = sin[positions.long()].double()[:, None, :]

    def rot(v):
        v0, v1 = v[..., :half], v[..., half:]
        return torch.cat([v0 * c - v1 * s, v0 * s + v1 * c], dim=-1)
    q_out.copy_(rot(x[:, :n_heads]).reshape(t, n_heads * head_dim).to(q_out.dtype))
    if not write_kv:
        return
    k = rot(x[:, n_heads:n_heads + n_kv_heads]).to(kcache.dtype)
    v = x[:, n_heads + n_kv_heads:].to(vcache.dtype)
    pos = positions.long()
    page = page_table.long()[seq_of_tok.long(), pos // PAGE]
    assert (page >= 0).all(), "token written to a page that was not reserved"
    kcache[page, :, pos % PAGE, :] = k
    if v_transposed(vcache):
        vcache[page, :, (pos % PAGE) // 32, :, pos % 32] = v
    else:
        vcache[page, :, pos % PAGE, :] = v


def rope_inplace(qkv, cos, sin, positions, n_rot_heads, n_heads_total, head_dim):
    t, half = positions.numel(), head_dim // 2
    x = qkv.view(t, n_heads_total, head_dim)
    c = cos[positions.long()].double()[:, None, :]
    s = sin[positions.long()].double()[:, None, :]
    v = x[:, :n_rot_heads].double()
    v0, v1 = v[..., :half], v[..., half:]
    x[:, :n_rot_heads] = torch.cat([v0 * c - v1 * s, v0 * s + v1 * c], dim=-1).float()


def linear(x, weight, bias, out, accumulate=False, variant=0, tiled=None, xielu=False):
    y = x.double() @ weight.double().t()
    if xielu:                            # the activation's constants ride behind the biases
        n = weight.shape[0]
        y = y + bias[:n].double()
        a_pos, a_neg = float(bias[n]), float(bias[n + 1])
        pos = a_pos * y * y + 0.5 * y
        neg = a_neg * (torch.expm1(torch.clamp(y, max=0.0)) - y) + 0.5 * y
        out.copy_(torch.where(y > 0, pos, neg).to(out.dtype))
        return
    if bias is not None:
        y = y + bias.double()
    if accumulate:
        y = y + out.double()
    out.copy_(y.to(out.dtype))


def interleave_gate_up(gate, up):
    """The layout the fused kernel reads, built row by row."""
    nf, k = gate.shape
    groups = (nf + 31) // 32
    out = torch.zeros(groups * 64, k, dtype=gate.dtype)
    for i in range(nf):
        out[(i // 32) * 64 + i % 32] = gate[i]
        out[(i // 32) * 64 + 32 + i % 32] = up[i]
    return out


def linear_swiglu(x, weight, out, variant=0, tiled=None):
    nf = out.shape[1]
    idx = torch.arange(nf)
    g = x.double() @ weight.double()[(idx // 32) * 64 + idx % 32].t()
    u = x.double() @ weight.double()[(idx // 32) * 64 + 32 + idx % 32].t()
    out.copy_((g / (1.0 + torch.exp(-g)) * u).to(out.dtype))


def linear_normed(x, norm_weight, eps, row_idx, weight, bias, out, accumulate=False, swiglu=False, tiled=None):
    """The stand-in has no folded kernel: the caller norms and multiplies in two steps."""
    return False


def linear_fused(x, weight, bias, out, accumulate=False, tiled=None, swiglu=False, scale_in=None, norm_out=None):
    """The stand-in folds no norm around a product: the caller runs the norm as a step of its own."""
    return False


def linear_normed_reference(x, norm_weight, eps, row_idx, weight, bias, swiglu=False):
    """What the folded kernel computes, in float64, with its one rounding of the activations:
    bf16(x * g) goes to the matrix cores and 1 / sqrt(mean(x^2) + eps) is applied to the sums."""
    rows = x if row_idx is None else x[row_idx.long()]
    a = (rows.float() * norm_weight.float()).to(torch.bfloat16).double()
    inv = 1.0 / torch.sqrt((rows.double() ** 2).mean(dim=1, keepdim=True) + eps)
    y = a @ weight.double().t() * inv
    if bias is not None:
        y = y + bias.double()
    return y


def v_transposed(vcache):
    """A bfloat16 cache keeps a page of V as [kv_heads][2][head_dim][32] (key j is element j % 32
    of half j / 32), a 32-bit one as [kv_heads][64][head_dim] (the product's `v_page_shape`)."""
    return vcache.dtype == torch.bfloat16


def v_rows(vcache, page, off):
    """[n][kv_heads][head_dim] rows of V at (page[i], off[i])."""
    return vcache[page, :, off // 32, :, off % 32] if v_transposed(vcache) else vcache[page, :, off, :]


def gather_cache_rows(cache, page_table_row, length, is_v=False):
    """[length][kv_heads][head_dim] rows 0..length-1 of one sequence."""
    pos = torch.arange(length)
    page = page_table_row.long()[pos // PAGE]
    return v_rows(cache, page, pos % PAGE) if is_v else cache[page, :, pos % PAGE, :]


def attn_tokens(q, kcache, vcache, page_table, positions, seq_of_tok, out, n_heads, n_kv_heads,
                head_dim, scale, window, max_len):
    t = positions.numel()
    g = n_heads // n_kv_heads
    qh = q.double().view(t, n_heads, head_dim)
    res = torch.zeros(t, n_heads, head_dim, dtype=torch.float64)
    for i in range(t):
        p = int(positions[i])
        lo = max(0, p - window + 1) if window else 0
        row = page_table[int(seq_of_tok[i])]
        pos = torch.arange(lo, p + 1)
        page = row.long()[pos // PAGE]
        assert (page >= 0).all(), "attention reads a page that was given back"
        k = kcache[page, :, pos % PAGE, :].double()      # [n][nk][hd]
        v = v_rows(vcache, page, pos % PAGE).double()
        for h in range(n_heads):
            s = (k[:, h // g, :] @ qh[i, h]) * scale
            res[i, h] = torch.softmax(s, dim=0) @ v[:, h // g, :]
    out.copy_(res.view(t, n_heads * head_dim).to(out.dtype))


def attn_decode_rope(qkv, cos, sin, kcache, vcache, page_table, positions, seq_of_tok, out, n_heads,
                     n_kv_heads, head_dim, scale, window, max_len, write_kv=True):
    q = torch.empty(positions.numel(), n_heads * head_dim, dtype=out.dtype)
    rope_kvwrite(qkv, cos, sin, positions, seq_of_tok, page_table, q, kcache, vcache, n_heads, n_kv_heads,
                 head_dim, write_kv)
    attn_tokens(q, kcache, vcache, page_table, positions, seq_of_tok, out, n_heads, n_kv_heads, head_dim, scale,
                window, max_len)


def attn_prefill(q, kcache, vcache, page_table, ctx, out, n_heads, n_kv_heads, head_dim, scale, window):
    attn_tokens(q, kcache, vcache, page_table, ctx.positions, ctx.seq_of_tok, out, n_heads, n_kv_heads,
                head_dim, scale, window, ctx.max_len)


# ------------------------------------------------------------------ norm in groups, xIELU, pair rotation
def group_rmsnorm(x, weight, eps, groups, out, row_idx=None, add=False, cast_out=None):
    src = (x if row_idx is None else x[row_idx.long()]).double()
    d = src.shape[-1]
    parts = src.view(src.shape[0], groups, d // groups)
    y = (parts / torch.sqrt((parts * parts).mean(dim=-1, keepdim=True) + eps)).reshape(src.shape)
    if weight is not None:
        y = y * weight.double()
    if add:
        y = y + out.double()
    out.copy_(y.to(out.dtype))
    if cast_out is not None:
        cast_out.copy_(out.to(cast_out.dtype))


def xielu(x, out, a_pos, a_neg):
    z = x.double()
    pos = a_pos * z * z + 0.5 * z
    neg = a_neg * (torch.expm1(torch.clamp(z, max=0.0)) - z) + 0.5 * z
    out.copy_(torch.where(z > 0, pos, neg).to(out.dtype))


def rope_table_freqs(n_pos, freqs, magnitude, device):
    f = torch.tensor([float(v) for v in freqs], dtype=torch.float64)
    ang = torch.arange(n_pos, dtype=torch.float64)[:, None] * f[None, :]
    return (torch.cos(ang) * magnitude).float().to(device), (torch.sin(ang) * magnitude).float().to(device)


def _rotate_pairs(v, c, s):
    """v [..., n]: the first 2 * c.shape[-1] values in pairs (2i, 2i+1); c, s broadcast over v's leading axes."""
    rd = 2 * c.shape[-1]
    out = v.clone()
    a, b = v[..., 0:rd:2], v[..., 1:rd:2]
    out[..., 0:rd:2] = a * c - b * s
    out[..., 1:rd:2] = b * c + a * s
    return out


def rope_pairs_inplace(qkv, cos, sin, positions, n_rot_heads, n_heads_total, head_dim):
    t = positions.numel()
    x = qkv.double().view(t, n_heads_total, head_dim)
    c, s = cos[positions.long()].double()[:, None, :], sin[positions.long()].double()[:, None, :]
    x[:, :n_rot_heads] = _rotate_pairs(x[:, :n_rot_heads], c, s)
    qkv.copy_(x.view(t, -1).to(qkv.dtype))


# ------------------------------------------------------------------ recurrence
def mingru_scan(zug, cu_seqlens, slot_ids, state, out, chunks=None):
    w = zug.shape[1] // 3
    z = torch.sigmoid(zug[:, :w].double())
    u = zug[:, w:2 * w].double()
    cand = torch.where(u >= 0, u + 0.5, torch.sigmoid(u))
    g = zug[:, 2 * w:].double()
    for b in range(slot_ids.numel()):
        slot = int(slot_ids[b])
        s = state[slot].double()
        for t in range(int(cu_seqlens[b]), int(cu_seqlens[b + 1])):
            s = (1.0 - z[t]) * s + z[t] * cand[t]
            s = s.float().double()                       # the state is carried in 32-bit
            out[t] = (s * g[t] * torch.sigmoid(g[t])).to(out.dtype)
        state[slot] = s.float()


# ------------------------------------------------------------------ latent attention
def latent_prep(proj, off_dkv, off_gate, latent_weight, eps, cos, sin, positions, seq_of_tok, page_table, cache,
                q_plain, q_abs, gate, n_heads, dim, rot_dim, rank, write_cache=True, q_rows=None):
    t = positions.numel()
    p = proj.double()
    c_t, s_t = cos[positions.long()].double(), sin[positions.long()].double()
    q = (p if q_rows is None else q_rows.double())[:, :n_heads * (dim + rot_dim)].reshape(t, n_heads, dim + rot_dim)
    q_plain.copy_(q[:, :, :dim].to(q_plain.dtype))
    q_abs[:, :, rank:] = _rotate_pairs(q[:, :, dim:], c_t[:, None, :], s_t[:, None, :]).to(q_abs.dtype)
    gate.copy_(torch.sigmoid(p[:, off_gate:off_gate + gate[0].numel()]).float().view(gate.shape))
    if not write_cache:
        return
    c = p[:, off_dkv:off_dkv + rank]
    c = c / torch.sqrt((c * c).mean(dim=-1, keepdim=True) + eps) * latent_weight.double()
    k_rot = _rotate_pairs(p[:, off_dkv + rank:off_dkv + rank + rot_dim], c_t, s_t)
    rows = torch.cat([c, k_rot], dim=-1).to(cache.dtype)
    flat = cache.view(-1, PAGE, rank + rot_dim)
    for i in range(t):
        pos = int(positions[i])
        page = int(page_table[int(seq_of_tok[i]), pos // PAGE])
        assert page >= 0
        flat[page, pos % PAGE] = rows[i]


def headwise_linear(x, n_in, wt, out, n_out, gate=None):
    y = torch.einsum("thi,hio->tho", x[:, :, :n_in].double(), wt.double())
    if gate is not None:
        y = y * (gate.double()[:, :, None] if gate.dim() == 2 else gate.double())
    out[:, :, :n_out] = y.to(out.dtype)


def headwise_mfma_takes(dtype, n_in, in_stride):
    return dtype == torch.bfloat16 and n_in % 8 == 0 and in_stride % 8 == 0


def headwise_linear_mfma(x, n_in, wo, out, n_out, gate=None):
    headwise_linear(x, n_in, wo.transpose(1, 2), out, n_out, gate)


def latent_attn(q_abs, cache, page_table, positions, seq_of_tok, out, rank, scale, window, max_len, ctx=None):
    t, heads, dk = q_abs.shape
    flat = cache.view(-1, PAGE, dk)
    for i in range(t):
        p = int(positions[i])
        lo = max(0, p - window + 1) if window else 0
        pos = torch.arange(lo, p + 1)
        page = page_table[int(seq_of_tok[i])].long()[pos // PAGE]
        assert (page >= 0).all(), "attention reads a page that was given back"
        rows = flat[page, pos % PAGE].double()           # [n][dk]
        s = (q_abs[i].double() @ rows.t()) * scale       # [heads][n]
        out[i] = (torch.softmax(s, dim=-1) @ rows[:, :rank]).to(out.dtype)


# ------------------------------------------------------------------ position rows, gelu, weighted sums
def embed_pos(table, pos_table, ids, positions, out):
    out.copy_((table[ids.long()].double() + pos_table[positions.long()].double()).to(torch.float32))


def gelu_tanh(x, out):
    z = x.double()
    out.copy_((0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))).to(out.dtype))


def softcap(x, cap):
    x.copy_((cap * torch.tanh(x.double() / cap)).float())


def weighted_sum(buffers, weights, out, row_idx=None, n_indexed=0):
    acc = torch.zeros(out.shape, dtype=torch.float64)
    for j, b in enumerate(buffers):
        rows = b[row_idx.long()] if j < n_indexed else b
        acc += float(weights[j]) * rows.double()
    out.copy_(acc.to(torch.float32))


# ------------------------------------------------------------------ linear attention with decay
LA_CHUNK = 64
LA_CHUNKED_MAX_DIM = 128


def lightning_scan(proj, cu_seqlens, slot_ids, decays, state, out, n_heads, dim, v_dim, chunks=None):
    H, D, V = n_heads, dim, v_dim
    p = proj.double()
    silu = lambda z: z * torch.sigmoid(z)
    t_all = p.shape[0]
    q = silu(p[:, :H * D]).view(t_all, H, D)
    k = silu(p[:, H * D:2 * H * D]).view(t_all, H, D)
    v = silu(p[:, 2 * H * D:2 * H * D + H * V]).view(t_all, H, V)
    for b in range(slot_ids.numel()):
        slot = int(slot_ids[b])
        S = state[slot].double()
        for t in range(int(cu_seqlens[b]), int(cu_seqlens[b + 1])):
            S = decays.double()[:, None, None] * S + k[t][:, :, None] * v[t][:, None, :]
            S = S.float().double()                       # the state is carried in 32-bit
            out[t] = torch.einsum("hdv,hd->hv", S, q[t]).reshape(-1).float()
        state[slot] = S.float()


def gated_rmsnorm(o, proj, gate_offset, weight, eps, out):
    x = o.double()
    n = x.shape[1]
    g = proj[:, gate_offset:gate_offset + n].double()
    y = x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps) * weight.double() * torch.sigmoid(g)
    out.copy_(y.to(out.dtype))


# ------------------------------------------------------------------ capped attention with a convolution in front
CONV_MAX_TAPS = 16


def _rotate_half(v, c, s):
    half = c.shape[-1]
    a, b = v[..., :half], v[..., half:2 * half]
    return torch.cat([a * c - b * s, b * c + a * s, v[..., 2 * half:]], dim=-1)


def rope_half_inplace(rows, cos, sin, positions, n_rot_heads, n_heads_total, head_dim):
    t = positions.numel()
    x = rows.double().view(t, n_heads_total, head_dim).clone()
    c, s = cos[positions.long()].double()[:, None, :], sin[positions.long()].double()[:, None, :]
    x[:, :n_rot_heads] = _rotate_half(x[:, :n_rot_heads], c, s)
    rows.copy_(x.view(t, -1).to(rows.dtype))


def _store_v(vcache, page, in_page, g, row):
    """One value row of kv head g into a page of either layout."""
    if vcache.dtype == torch.bfloat16:               # [pages][kv][2][V][32]
        vcache[page, g, in_page // 32, :, in_page % 32] = row.to(vcache.dtype)
    else:
        vcache[page, g, in_page] = row.to(vcache.dtype)


def _load_v(vcache, pages, in_page, g):
    if vcache.dtype == torch.bfloat16:
        return vcache[pages, g, in_page // 32, :, in_page % 32].double()
    return vcache[pages, g, in_page].double()


def qkv_conv_prep(qkv, conv_w, conv_state, cu_seqlens, seq_of_tok, slot_ids, positions, cos, sin, blend, v_first, v_own,
                  page_table, q_out, kcache, vcache, n_heads, n_kv_heads, dim, v_dim, write_cache=True):
    t_all, C = qkv.shape
    u = qkv.double()
    y = u.clone()
    taps = 1 if conv_w is None else conv_w.shape[1]
    if conv_w is not None:
        w = conv_w.double()
        for b in range(slot_ids.numel()):
            r0, r1 = int(cu_seqlens[b]), int(cu_seqlens[b + 1])
            slot = int(slot_ids[b])
            before = conv_state[slot].double() if taps > 1 else torch.zeros((0, C), dtype=torch.float64)
            full = torch.cat([before, u[r0:r1]], dim=0)
            acc = torch.zeros((r1 - r0, C), dtype=torch.float64)
            for j in range(taps):
                acc += w[:, j] * full[j:j + (r1 - r0)]
            y[r0:r1] = acc
            if write_cache and taps > 1:
                conv_state[slot] = full[full.shape[0] - (taps - 1):].float()
    nq, nk = n_heads * dim, n_kv_heads * dim
    q = y[:, :nq].view(t_all, n_heads, dim)
    k = y[:, nq:nq + nk].view(t_all, n_kv_heads, dim)
    v = y[:, nq + nk:].view(t_all, n_kv_heads, v_dim)
    if cos is not None:
        c, s = cos[positions.long()].double()[:, None, :], sin[positions.long()].double()[:, None, :]
        q, k = _rotate_half(q, c, s), _rotate_half(k, c, s)
    if v_own is not None:
        v_own.copy_(v.reshape(t_all, -1).float())
    if v_first is not None:
        v = (1.0 - blend) * v + blend * v_first.double().view(t_all, n_kv_heads, v_dim)
    q_out.copy_(q.reshape(t_all, nq).to(q_out.dtype))
    if not write_cache:
        return
    for i in range(t_all):
        pos = int(positions[i])
        page = int(page_table[int(seq_of_tok[i]), pos // PAGE])
        assert page >= 0
        kcache[page, :, pos % PAGE] = k[i].to(kcache.dtype)
        for g in range(n_kv_heads):
            _store_v(vcache, page, pos % PAGE, g, v[i, g])


def capped_attn(q, kcache, vcache, page_table, positions, seq_of_tok, temp, out, n_heads, n_kv_heads, dim, v_dim,
                scale, cap, window, max_len, chunk=0, far=None, keep_first=0, bias=None):
    t_all = positions.numel()
    group = n_heads // n_kv_heads
    qq = q.double().view(t_all, n_heads, dim)
    for i in range(t_all):
        p = int(positions[i])
        lo = max(0, p - window + 1) if window else 0
        if chunk:
            lo = max(lo, p // chunk * chunk)
        pos = torch.arange(lo, p + 1)
        if window and keep_first:
            pos = torch.cat([torch.arange(0, min(keep_first, lo)), pos])
        pages = page_table[int(seq_of_tok[i])].long()[pos // PAGE]
        assert (pages >= 0).all(), "attention reads a page that was given back"
        for h in range(n_heads):
            g = h // group
            keys = kcache[pages, g, pos % PAGE].double()
            vals = torch.stack([_load_v(vcache, int(pg), int(ip), g) for pg, ip in zip(pages, pos % PAGE)])
            s = (keys @ qq[i, h]) * scale * float(temp[h])
            if cap:
                s = cap * torch.tanh(s / cap)
            if far is not None:
                s = s - float(far[0][h]) * torch.log1p(float(far[1][h]) * (p - pos).double())
            if bias is not None:
                s = s + bias[h].double()[torch.clamp(p - pos, max=bias.shape[1] - 1)]
            out[i, h * v_dim:(h + 1) * v_dim] = (torch.softmax(s, dim=0) @ vals).to(out.dtype)


def capped_mfma_takes(dtype, dim, v_dim):
    return dtype == torch.bfloat16 and dim % 16 == 0 and v_dim % 16 == 0 and 16 <= dim <= 256 and 16 <= v_dim <= 256


def capped_attn_prefill(q, kcache, vcache, page_table, ctx, temp, out, n_heads, n_kv_heads, dim, v_dim, scale, cap, window,
                        chunk=0, far=None, keep_first=0, bias=None):
    capped_attn(q, kcache, vcache, page_table, ctx.positions, ctx.seq_of_tok, temp, out, n_heads, n_kv_heads, dim, v_dim,
                scale, cap, window, ctx.max_len, chunk=chunk, far=far, keep_first=keep_first, bias=bias)


# ------------------------------------------------------------------ rows added into rows, the gated recurrence,
# normed and pair-rotated queries and keys
def add_rows(h, x):
    h.add_(x)


GR_CHUNK = 64


def gr_chunks(host_new):
    return torch.zeros(0, dtype=torch.int32), 0


def gated_scan(proj, lower, cu_seqlens, slot_ids, state, out, n_heads, dim, v_dim, chunks=None):
    H, D, V = n_heads, dim, v_dim
    p = proj.double()
    low = lower.double().view(H, D)
    for b in range(slot_ids.numel()):
        r0, r1 = int(cu_seqlens[b]), int(cu_seqlens[b + 1])
        slot = int(slot_ids[b])
        S = state[slot].double()
        for t in range(r0, r1):
            z = p[t, :H * D].view(H, D)
            q = z * torch.sigmoid(z)
            a = low + (1.0 - low) * torch.sigmoid(p[t, H * D:2 * H * D].view(H, D))
            v = p[t, 2 * H * D:].view(H, V)
            S = a[:, :, None] * S + (1.0 - a)[:, :, None] * v[:, None, :]
            out[t] = torch.einsum("hdv,hd->hv", S, q).reshape(-1).float()
        state[slot] = S.float()


def head_rmsnorm(o, weight, eps, out, n_heads, scale=1.0):
    rows, n = o.shape
    x = o.double().view(rows, n_heads, n // n_heads)
    y = x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps) * scale
    if weight is not None:
        y = y * weight.double()
    out.copy_(y.reshape(rows, n).to(out.dtype))


def qk_norm_prep(qkv, q_gain, k_gain, eps, normed, seq_of_tok, positions, rot_tables, value_tables, v_from_k, page_table,
                 q_out, kcache, vcache, n_heads, n_kv_heads, dim, v_dim, write_cache=True, halves=False, q_only=False):
    t_all = positions.numel()
    y = qkv.double()
    nq, nk = n_heads * dim, n_kv_heads * dim
    q = y[:, :nq].view(t_all, n_heads, dim)
    if q_only:           # no keys and values of its own: pad with zeros that nobody stores
        y = torch.cat([y, torch.zeros(t_all, nk + n_kv_heads * v_dim, dtype=torch.float64)], dim=1)
        write_cache = False
    k = y[:, nq:nq + nk].view(t_all, n_kv_heads, dim)
    v = k.clone() if v_from_k else y[:, nq + nk:].view(t_all, n_kv_heads, v_dim)
    if normed:
        q = q / torch.sqrt((q * q).mean(dim=-1, keepdim=True) + eps)
        k = k / torch.sqrt((k * k).mean(dim=-1, keepdim=True) + eps)
    if q_gain is not None:
        q = q * q_gain.double()
    if k_gain is not None:
        k = k * k_gain.double()
    pos = positions.long()
    if rot_tables is not None:
        c, s = rot_tables[0][pos].double()[:, None, :], rot_tables[1][pos].double()[:, None, :]
        turn = _rotate_half_part if halves else _rotate_pairs
        q, k = turn(q, c, s), turn(k, c, s)
    if value_tables is not None:
        v = _rotate_pairs(v, value_tables[0][pos].double()[:, None, :], value_tables[1][pos].double()[:, None, :])
    q_out.copy_(q.reshape(t_all, nq).to(q_out.dtype))
    if not write_cache:
        return
    for i in range(t_all):
        p = int(positions[i])
        page = int(page_table[int(seq_of_tok[i]), p // PAGE])
        assert page >= 0
        kcache[page, :, p % PAGE] = k[i].to(kcache.dtype)
        for g in range(n_kv_heads):
            _store_v(vcache, page, p % PAGE, g, v[i, g])


def _rotate_half_part(v, c, s):
    """Value i turns with value i + n, i < n = the tables' columns; the values from 2 n on pass."""
    n = c.shape[-1]
    a, b = v[..., :n], v[..., n:2 * n]
    return torch.cat([a * c - b * s, b * c + a * s, v[..., 2 * n:]], dim=-1)


def unrotate(rows, value_tables, positions, n_heads, scale=1.0):
    t_all = positions.numel()
    x = rows.double().view(t_all, n_heads, -1)
    if value_tables is not None:
        pos = positions.long()
        x = _rotate_pairs(x, value_tables[0][pos].double()[:, None, :], -value_tables[1][pos].double()[:, None, :])
    rows.copy_((x * scale).reshape(t_all, -1).to(rows.dtype))


# ------------------------------------------------------------------ mixture of experts
MOE_MAX_EXPERTS = 1024
MOE_SPARSE_TOKENS, MOE_SPARSE_PAIRS = 16, 128


MOE_ACTS = {"clamped_swish": 0, "silu": 1}


MOE_SCORES = {"softmax": 0, "sigmoid": 1}


def moe_route(x, router, dense, chosen, weights, n_groups, keep, bias=None, score="softmax", correction=None,
              group_top=1, weight_scale=1.0):
    logits = x.double() @ router.double().t()
    if bias is not None:
        logits = logits + bias.double()
    logits = logits.float()
    n_tok, E = logits.shape
    top = chosen.shape[1]
    per = E // n_groups
    s = torch.sigmoid(logits.float()) if score == "sigmoid" else torch.softmax(logits.float(), dim=-1)
    choice = s if correction is None else s + correction.float()
    if dense is not None:
        dense.zero_()
    for t in range(n_tok):
        gs = torch.sort(choice[t].view(n_groups, per), dim=1, descending=True).values[:, :group_top].sum(dim=1)
        kept = torch.argsort(-gs, stable=True)[:keep]
        masked = torch.full((E,), float("-inf"))
        for g in kept.tolist():
            masked[g * per:(g + 1) * per] = choice[t, g * per:(g + 1) * per]
        pick = torch.argsort(-masked, stable=True)[:top]
        w = s[t, pick] / (s[t, pick].sum() + 1e-20) * weight_scale
        chosen[t] = pick.to(torch.int32)
        weights[t] = w
        if dense is not None:
            dense[t, pick] = w


def _expert_act(g, u, limit, act=0):
    if act == 1:
        return g * torch.sigmoid(g) * u
    g = torch.clamp(g, max=limit)
    u = torch.clamp(u, -limit, limit)
    return g * torch.sigmoid(1.702 * g) * (u + 1.0)


def moe_act(gu, dense, out, limit, act=0):
    n_tok, E = dense.shape
    F = gu.shape[1] // (2 * E)
    x = gu.double().view(n_tok, E, 2, F)
    y = _expert_act(x[:, :, 0], x[:, :, 1], limit, act) * dense.double()[:, :, None]
    out.copy_(y.reshape(n_tok, E * F).to(out.dtype))


def moe_sparse(x, gate_up, down, chosen, weights, out, n_experts, limit, act=0):
    n_tok, K = x.shape
    _, N, F = down.shape
    gu = gate_up.double().view(n_experts, 2, F, K)
    dn = down.double()
    for t in range(n_tok):
        for k in range(chosen.shape[1]):
            e = int(chosen[t, k])
            y = _expert_act(gu[e, 0] @ x[t].double(), gu[e, 1] @ x[t].double(), limit, act).to(x.dtype).double()
            out[t] += (float(weights[t, k]) * (dn[e] @ y)).float()


def moe_group(chosen, n_experts, rank, counts):
    seen = [0] * n_experts
    flat, r = chosen.reshape(-1), rank.view(-1)
    for p in range(flat.numel()):
        r[p] = seen[int(flat[p])]
        seen[int(flat[p])] += 1
    counts.copy_(torch.tensor(seen, dtype=torch.int32))


def _rows_of(chosen, rank, offsets):
    return (offsets.long()[chosen.long()] + rank.long()).reshape(-1)


def moe_gather(x, chosen, rank, offsets, xs):
    top = chosen.shape[1]
    xs[_rows_of(chosen, rank, offsets)] = x.repeat_interleave(top, dim=0)


def moe_combine(rows, chosen, rank, offsets, weights, out, accumulate=True):
    n_tok, top = chosen.shape
    picked = rows[_rows_of(chosen, rank, offsets)].double().view(n_tok, top, -1)
    acc = out.double() if accumulate else torch.zeros(out.shape, dtype=torch.float64)
    for k in range(top):
        acc = acc + weights.double()[:, k, None] * picked[:, k]
    out.copy_(acc.float())


# ------------------------------------------------------------------ sampling
def argmax(logits, out):
    import plain_qwen2 as pq
    for i in range(logits.shape[0]):
        out[i] = pq.greedy(logits[i].numpy())


def stream_uniform(stream_i64: int, step: int) -> float:
    """The draw of a stream id (as an int64 tensor holds it) at a step: the device's uniform01."""
    from minfer_amd.sampling.rng import mix64
    h = mix64((stream_i64 & 0xFFFFFFFFFFFFFFFF) ^ (step & 0xFFFFFFFFFFFFFFFF))
    return (h >> 40) / 16777216.0


def sample(logits, temp, streams, steps, out, forced_r=None):
    import plain_qwen2 as pq
    for i in range(logits.shape[0]):
        if temp < 1e-6:
            out[i] = pq.greedy(logits[i].numpy())
            continue
        r = float(forced_r[i]) if forced_r is not None else stream_uniform(int(streams[i]), int(steps[i]))
        out[i] = pq.sample_from_probs(pq.temperature_probs(logits[i].numpy(), temp), r)


def penalties(logits, prev, n_prev, repeat, frequency, presence):
    import plain_qwen2 as pq
    for i in range(logits.shape[0]):
        window = prev[i, :int(n_prev[i])].tolist()
        logits[i] = torch.from_numpy(pq.apply_penalties(logits[i].numpy(), window, repeat, frequency, presence))


def top_k(logits, k):
    import plain_qwen2 as pq
    for i in range(logits.shape[0]):
        logits[i] = torch.from_numpy(pq.apply_top_k(logits[i].numpy(), k))


def top_p(logits, p):
    import plain_qwen2 as pq
    for i in range(logits.shape[0]):
        logits[i] = torch.from_numpy(pq.apply_top_p(logits[i].numpy(), p))


def sample_filtered_takes(vocab, k, temp):
    return 1 <= k <= 48 and k < vocab <= 32 * 256 * 32 and temp >= 1e-6


def sample_filtered(logits, k, p, temp, streams, steps, out, forced_r=None):
    work = logits.clone()
    top_k(work, k)
    if 0.0 < p < 1.0:
        top_p(work, p)
    sample(work, temp, streams, steps, out, forced_r)


def advance(next_ids, sampled, positions, steps, prev=None, n_prev=None, cursor=None):
    next_ids.copy_(sampled)
    positions += 1
    steps += 1
    if prev is not None:
        for i in range(next_ids.numel()):
            c = int(cursor[i])
            prev[i, c] = sampled[i]
            cursor[i] = (c + 1) % prev.shape[1]
            n_prev[i] = min(int(n_prev[i]) + 1, prev.shape[1])


NAMES = ["embed", "rmsnorm", "gather_rows", "swiglu", "convert", "fill_normal", "rope_table",
         "rope_kvwrite", "rope_inplace", "linear", "attn_tokens", "attn_prefill", "argmax", "sample", "penalties",
         "top_k", "top_p", "sample_filtered", "sample_filtered_takes", "advance", "interleave_gate_up", "linear_swiglu", "linear_normed", "linear_fused", "attn_decode_rope",
         "group_rmsnorm", "xielu", "rope_table_freqs", "rope_pairs_inplace", "mingru_scan", "latent_prep",
         "headwise_linear", "latent_attn", "headwise_mfma_takes", "headwise_linear_mfma",
         "embed_pos", "gelu_tanh", "weighted_sum", "lightning_scan", "gated_rmsnorm", "rope_half_inplace",
         "qkv_conv_prep", "capped_attn", "capped_mfma_takes", "capped_attn_prefill", "moe_route", "moe_act", "moe_sparse", "moe_group", "moe_gather", "moe_combine",
         "add_rows", "gr_chunks", "gated_scan", "head_rmsnorm", "qk_norm_prep", "unrotate", "softcap"]


def install(monkeypatch):
    """Replaces the HIP launchers by the plain versions and lets models live on the CPU."""
    from minfer_amd.engine import loading
    from minfer_amd.kernels import ops
    for name in NAMES:
        monkeypatch.setattr(ops, name, globals()[name], raising=False)
    monkeypatch.setattr(loading, "require_gpu", lambda device: torch.device("cpu"))
