"""A stand-in for ``kappai_amd.kernels.ops`` made of torch CPU operations, so that the
engine's own logic (row tables, cache manager, step function, scheduler, replay) can be
tested where there is no GPU.  It belongs to the tests; the package never imports it.
Every function has the contract of the kernel it stands for, including the dtype in which
results are stored."""
from __future__ import annotations

import numpy as np
import torch

F32, BF16 = torch.float32, torch.bfloat16
ROT_NONE, ROT_HALF, ROT_INTERLEAVED = 0, 1, 2


def embed_rows(ids, table):
    return table[ids.long()].to(F32)


def add_rmsnorm(resid, delta, weight, eps, out_dtype, rows=None, write_resid=True,
                fragment=False):
    assert not fragment, "rows in fragment order are made on the GPU only"
    x = resid
    if delta is not None:
        parts = delta if delta.dim() == 3 else delta[None]
        for p in parts:                       # partial sums are added in order
            x = x + p.to(F32)
    if delta is not None and write_resid and rows is None:
        resid.copy_(x)
    if rows is not None:
        x = x[rows.long()]
    y = x * (1.0 / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)) * weight
    return y.to(out_dtype)


def sum_partial_sums(parts):
    out = parts[0].to(F32).clone()
    for p in parts[1:]:
        out += p
    return out


def add_residual(resid, delta):
    resid.add_(delta.to(F32))


def swiglu(gate_up):
    F = gate_up.shape[1] // 2
    g, u = gate_up[:, :F].to(F32), gate_up[:, F:].to(F32)
    return (g / (1.0 + torch.exp(-g)) * u).to(gate_up.dtype)


def cast(x, dtype):
    return x.to(dtype)


def linear(x, weight, bias=None, out_dtype=None, force_kernel=0, partial_sums=False,
           split_k=None, weight_frag=None, add_into=None):
    # ``add_into`` is an offer the stand-in does not take up: the result comes back as always
    out_dtype = out_dtype or x.dtype
    y = x.to(F32) @ weight.to(F32).T
    if bias is not None:
        y = y + bias
    return y.to(out_dtype)


SWIGLU_GROUP = 16


def interleave_gate_up(gate, up):
    F, K = gate.shape
    g = gate.reshape(F // SWIGLU_GROUP, 1, SWIGLU_GROUP, K)
    u = up.reshape(F // SWIGLU_GROUP, 1, SWIGLU_GROUP, K)
    return torch.cat([g, u], dim=1).reshape(2 * F, K).contiguous()


def linear_swiglu(x, weight, force_kernel=0, weight_frag=None, out_fragment=False, activation=0):
    F = weight.shape[0] // 2
    y = (x.to(F32) @ weight.to(F32).T).reshape(x.shape[0], F // SWIGLU_GROUP, 2, SWIGLU_GROUP)
    g, u = y[:, :, 0, :].reshape(-1, F), y[:, :, 1, :].reshape(-1, F)
    if activation == 1:
        a = 0.5 * g * (1.0 + torch.tanh(0.7978845608028654 * (g + 0.044715 * g ** 3)))
    else:
        a = g / (1.0 + torch.exp(-g))
    return (a * u).to(x.dtype)


def shortconv(proj, taps, bias, state, row_seg, seg_start, seg_pos0, seg_slot):
    T = proj.shape[0]
    D, L = taps.shape
    H = L - 1
    p = proj.to(F32)
    B, C, X = p[:, :D], p[:, D:2 * D], p[:, 2 * D:]
    bx = B * X
    out = torch.empty((T, D), dtype=F32)
    for s in range(seg_pos0.shape[0]):
        t0, t1 = int(seg_start[s]), int(seg_start[s + 1])
        slot = int(seg_slot[s])
        hist = torch.zeros((H, D)) if int(seg_pos0[s]) == 0 else state[slot].T.clone()
        seq = torch.cat([hist, bx[t0:t1]], dim=0)            # [H + n, D]
        for r in range(t1 - t0):
            acc = torch.zeros(D) if bias is None else bias.clone()
            for k in range(L):
                acc = acc + taps[:, k] * seq[r + k]
            out[t0 + r] = C[t0 + r] * acc
        state[slot] = seq[-H:].T
    return out.to(proj.dtype)


def linear_shortconv_step(x, in_proj, in_bias, taps, conv_bias, state, seg_pos0, seg_slot,
                          weight_frag=None, out_fragment=False):
    M = x.shape[0]
    proj = linear(x, in_proj, in_bias)
    row_seg = torch.arange(M, dtype=torch.int32)
    seg_start = torch.arange(M + 1, dtype=torch.int32)
    return shortconv(proj, taps, conv_bias, state, row_seg, seg_start, seg_pos0, seg_slot)


def qk_norm_rope_store(qkv, n_heads, n_kv_heads, head_dim, q_norm_w, k_norm_w, eps, cos, sin,
                       rot_dim, rot_mode, k_pool, v_pool, row_pos, row_seg, block_tables,
                       page_size, store_kv=True):
    H, G, d = n_heads, n_kv_heads, head_dim
    T = qkv.shape[0]
    pos = row_pos.long()

    def norm_rot(x, w):                                      # x: [T, heads, d] float32
        if w is not None:
            x = x * (1.0 / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)) * w
        if rot_mode == ROT_NONE:
            return x
        half = rot_dim // 2
        c, s = cos[pos][:, None, :], sin[pos][:, None, :]
        y = x.clone()
        if rot_mode == ROT_HALF:
            a, b = x[..., :half], x[..., half:rot_dim]
            y[..., :half] = a * c - b * s
            y[..., half:rot_dim] = a * s + b * c
        else:
            a, b = x[..., 0:rot_dim:2], x[..., 1:rot_dim:2]
            y[..., 0:rot_dim:2] = a * c - b * s
            y[..., 1:rot_dim:2] = a * s + b * c
        return y

    q = norm_rot(qkv[:, :H * d].to(F32).reshape(T, H, d), q_norm_w)
    qkv[:, :H * d] = q.reshape(T, H * d).to(qkv.dtype)
    if not store_kv:
        return qkv
    k = norm_rot(qkv[:, H * d:(H + G) * d].to(F32).reshape(T, G, d), k_norm_w)
    v = qkv[:, (H + G) * d:(H + 2 * G) * d].reshape(T, G, d)
    for t in range(T):
        p = int(row_pos[t])
        page = int(block_tables[int(row_seg[t]), p // page_size])
        assert page >= 0, "a row is stored into a page that was given back"
        k_pool[page, :, p % page_size, :] = k[t].to(k_pool.dtype)
        v_pool[page, :, :, p % page_size] = v[t].to(v_pool.dtype)
    return qkv


def paged_attention(q, n_heads, n_kv_heads, head_dim, k_pool, v_pool, row_pos, row_seg,
                    block_tables, page_size, scale, window=0, mods=None, chunk=0, **_unused):
    H, G, d = n_heads, n_kv_heads, head_dim
    assert not (window and chunk)
    if mods is not None and not mods.active():
        mods = None
    T = q.shape[0]
    out = torch.empty((T, H * d), dtype=F32)
    for t in range(T):
        p = int(row_pos[t])
        lo = p + 1 - window if window and p + 1 > window else 0
        if chunk:
            lo = p - p % chunk
        bt = block_tables[int(row_seg[t])]
        idx = torch.arange(lo, p + 1)
        pages = bt[(idx // page_size).long()].long()
        assert bool((pages >= 0).all()), "attention reads a page that was given back"
        keys = k_pool[pages, :, (idx % page_size).long(), :].to(F32)     # [n, G, d]
        vals = v_pool[pages, :, :, (idx % page_size).long()].to(F32)             # [n, G, d]
        qt = q[t, :H * d].to(F32).reshape(H, d)
        for h in range(H):
            g = h // (H // G)
            sc = (keys[:, g, :] @ qt[h]) * scale
            if mods is not None:
                if mods.softcap > 0:
                    sc = mods.softcap * torch.tanh(sc / mods.softcap)
                if mods.distance_bias is not None:
                    col = torch.clamp(p - idx, max=mods.distance_bias.shape[1] - 1)
                    sc = sc + mods.distance_bias[h][col]
            if mods is not None and mods.sink is not None:
                a = torch.softmax(torch.cat([sc, mods.sink[h:h + 1]]), dim=0)[:-1]
            else:
                a = torch.softmax(sc, dim=0)
            out[t, h * d:(h + 1) * d] = a @ vals[:, g, :]
    return out.to(q.dtype)


def sample_rows(logits, temperature, uniform):
    out = torch.empty(logits.shape[0], dtype=torch.int32)
    for r in range(logits.shape[0]):
        lg = logits[r].double()
        t = float(temperature[r])
        if not t > 0:
            m = lg.max()
            out[r] = int(torch.nonzero(lg == m)[0])
            continue
        z = (logits[r] * (1.0 / t))
        e = torch.exp(z - z.max()).double()
        acc = torch.cumsum(e, 0)
        target = float(uniform[r]) * float(acc[-1])
        i = int(torch.searchsorted(acc, torch.tensor(target, dtype=torch.float64), right=True))
        out[r] = min(i, logits.shape[1] - 1)
    return out


FILTER_MAX_KEEP = 1024


def sample_filtered(logits, rows, keep, temperature, top_p, min_p, uniform, out):
    from plain import sampler as plain_sampler
    for i in range(rows.shape[0]):
        r = int(rows[i])
        k = int(keep[i])
        out[r] = plain_sampler.sample_filtered(
            logits[r].numpy(), float(temperature[i]), k if k < logits.shape[1] else 0,
            float(top_p[i]), float(min_p[i]), float(uniform[i]), cap=k)


def repeat_penalty(logits, row_start, tokens, penalty):
    for r in range(logits.shape[0]):
        pen = float(penalty[r])
        if pen == 1.0:
            continue
        for i in range(int(row_start[r]), int(row_start[r + 1])):
            tok = int(tokens[i])
            if 0 <= tok < logits.shape[1]:
                logits[r, tok] = logits[r, tok] / pen if logits[r, tok] > 0 else logits[r, tok] * pen


def history_set(history, seen, slots, starts, tokens):
    cap = history.shape[1]
    for i in range(slots.shape[0]):
        lo, hi = int(starts[i]), int(starts[i + 1])
        n = min(hi - lo, cap)
        history[int(slots[i]), :n] = tokens[lo:lo + n]
        seen[int(slots[i])] = n


def repeat_penalty_history(logits, rows, slots, penalty, last_n, history, seen):
    cap = history.shape[1]
    for i in range(rows.shape[0]):
        pen = float(penalty[i])
        if pen == 1.0:
            continue
        slot, total = int(slots[i]), int(seen[int(slots[i])])
        n = min(int(last_n[i]), total, cap)
        r = int(rows[i])
        for j in range(total - n, total):
            tok = int(history[slot, j % cap])
            if 0 <= tok < logits.shape[1]:
                logits[r, tok] = logits[r, tok] / pen if logits[r, tok] > 0 else logits[r, tok] * pen


def history_append(chosen, rows, slots, history, seen):
    cap = history.shape[1]
    for i in range(rows.shape[0]):
        slot = int(slots[i])
        history[slot, int(seen[slot]) % cap] = chosen[int(rows[i])]
        seen[slot] += 1



# ---- grouped norm, input convolution, positions -------------------------------------------
def add_group_rmsnorm(resid, delta, weight, eps, groups, out_dtype, rows=None, write_resid=True):
    x = resid
    if delta is not None:
        parts = delta if delta.dim() == 3 else delta[None]
        for p in parts:
            x = x + p.to(F32)
        if write_resid and rows is None:
            resid.copy_(x)
    if rows is not None:
        x = x[rows.long()]
    n, D = x.shape
    g = x.reshape(n, groups, D // groups)
    g = g * (1.0 / torch.sqrt((g * g).mean(dim=-1, keepdim=True) + eps))
    return (g.reshape(n, D) * weight).to(out_dtype)


def canon_conv(h, taps, state, row_pos, row_seg, seg_start, seg_slot, out_dtype):
    T, D = h.shape
    n = taps.shape[1]
    out = h.clone()
    for t in range(T):
        s = int(row_seg[t])
        local = t - int(seg_start[s])
        slot = int(seg_slot[s])
        for j in range(n):
            back = n - 1 - j
            if int(row_pos[t]) - back < 0:
                continue
            v = h[t - back] if local - back >= 0 else state[slot, n - 1 + local - back]
            out[t] += taps[:, j] * v
    for s in range(seg_slot.shape[0]):
        first, last = int(seg_start[s]), int(seg_start[s + 1])
        slot = int(seg_slot[s])
        hist = torch.cat([state[slot], h[first:last]], dim=0)
        state[slot] = hist[hist.shape[0] - (n - 1):]
    return out.to(out_dtype)


def add_group_rmsnorm_canon_step(resid, delta, weight, eps, groups, taps, state, row_pos, seg_slot,
                                 out_dtype):
    T = resid.shape[0]
    h = add_group_rmsnorm(resid, delta, weight, eps, groups, F32)
    ar = torch.arange(T + 1, dtype=torch.int32)
    return canon_conv(h, taps, state, row_pos, ar[:T], ar, seg_slot, out_dtype)


def scale_add_positions(x, scale, table, row_pos):
    x.mul_(scale).add_(table[row_pos.long()].to(F32))


def glu(gate_up, kind):
    F = gate_up.shape[1] // 2
    g, u = gate_up[:, :F].to(F32), gate_up[:, F:].to(F32)
    if kind == 1:
        a = 0.5 * g * (1.0 + torch.tanh(0.7978845608028654 * (g + 0.044715 * g ** 3)))
    else:
        a = g / (1.0 + torch.exp(-g))
    return (a * u).to(gate_up.dtype)


# ---- minGRU ----------------------------------------------------------------------------------
def mingru_scan(proj, state, seg_start, seg_pos0, seg_slot, out_dtype, chunks=None,
                seg_chunk0=None):
    proj = proj.to(F32)
    T, W = proj.shape[0], proj.shape[1] // 3
    out = torch.empty((T, W), dtype=F32)
    for s in range(seg_slot.shape[0]):
        slot = int(seg_slot[s])
        S = state[slot].clone() if int(seg_pos0[s]) > 0 else torch.zeros(W)
        for t in range(int(seg_start[s]), int(seg_start[s + 1])):
            z = torch.sigmoid(proj[t, :W])
            u = proj[t, W:2 * W]
            c = torch.where(u >= 0, u + 0.5, torch.sigmoid(u))
            S = (1.0 - z) * S + z * c
            g = proj[t, 2 * W:]
            out[t] = S * (g * torch.sigmoid(g))
        state[slot] = S
    return out.to(out_dtype)


# ---- differential attention -------------------------------------------------------------------
def diff_store(proj, n_heads, n_kv_heads, dim, vdim, head_size, k_pool, v_pool, row_pos, row_seg,
               block_tables, page_size, store_kv=True):
    H, G, d, dv, D = n_heads, n_kv_heads, dim, vdim, head_size
    T, R = proj.shape[0], n_heads // n_kv_heads
    q = torch.zeros((T, 2 * H, D), dtype=proj.dtype)
    qs = proj[:, :H * 2 * d].reshape(T, G, R, 2, d)
    q.view(T, G, 2, R, D)[..., :d] = qs.permute(0, 1, 3, 2, 4)
    if store_kv:
        ks = proj[:, H * 2 * d:(H + G) * 2 * d].reshape(T, 2 * G, d)
        vs = proj[:, (H + G) * 2 * d:(H + G) * 2 * d + G * dv].reshape(T, G, dv)
        for t in range(T):
            p = int(row_pos[t])
            page = int(block_tables[int(row_seg[t]), p // page_size])
            assert page >= 0, "a key is stored into a page that was given back"
            k_pool[page, :, p % page_size, :] = 0
            k_pool[page, :, p % page_size, :d] = ks[t]
            v_pool[page, :, :, p % page_size] = 0
            v_pool[page, :, :dv, p % page_size] = vs[t].repeat_interleave(2, dim=0)
    return q.reshape(T, 2 * H * D)


def diff_combine(ctx, n_heads, n_kv_heads, vdim, head_size, lam, eps, gain):
    H, G, dv, D = n_heads, n_kv_heads, vdim, head_size
    T, R = ctx.shape[0], n_heads // n_kv_heads
    a = ctx.to(F32).reshape(T, G, 2, R, D)[..., :dv]
    o = a[:, :, 0] - lam * a[:, :, 1]                      # [T, G, R, dv]
    o = o * (gain / torch.sqrt((o * o).mean(dim=-1, keepdim=True) + eps))
    return o.reshape(T, H * dv).to(ctx.dtype)


# ---- mixture of experts -----------------------------------------------------------------------
# ---------------------------------------------------------------------------------------
# the kernels of the output-norm arrangement, the scored and latent attention, the recurrences
# with a matrix of state
# ---------------------------------------------------------------------------------------
def output_norm_add(resid, a, weight, eps, rows_dtype=None, scale_a=1.0, b=None, scale_b=1.0,
                    add=True):
    y = a.to(F32)
    if y.dim() == 3:
        acc = y[0].clone()
        for part in y[1:]:
            acc = acc + part
        y = acc
    y = y * scale_a
    if b is not None:
        y = y + scale_b * b.to(F32)
    n = y * (1.0 / torch.sqrt((y * y).mean(dim=-1, keepdim=True) + eps)) * weight
    if add:
        resid.add_(n)
    else:
        resid.copy_(n)
    return None if rows_dtype is None else resid.to(rows_dtype)


def _store(k_pool, v_pool, keys, vals, row_pos, row_seg, block_tables, page_size):
    for t in range(keys.shape[0]):
        p = int(row_pos[t])
        page = int(block_tables[int(row_seg[t]), p // page_size])
        assert page >= 0, "a row is stored into a page that was given back"
        k_pool[page, :, p % page_size, :] = keys[t].to(k_pool.dtype)
        v_pool[page, :, :, p % page_size] = vals[t].to(v_pool.dtype)


def projection_norm_store(proj, n_heads, n_kv_heads, dim, vdim, head_size, q_norm_w, k_norm_w, eps,
                          temp_coef, temp_every, k_pool, v_pool, row_pos, row_seg, block_tables,
                          page_size, store_kv=True):
    H, G, d, dv, D = n_heads, n_kv_heads, dim, vdim, head_size
    T = proj.shape[0]
    p = proj.to(F32)
    q, k, v = p[:, :H * d], p[:, H * d:(H + G) * d], p[:, (H + G) * d:(H + G) * d + G * dv]
    if q_norm_w is not None:
        q = q / torch.sqrt((q * q).mean(-1, keepdim=True) + eps) * q_norm_w
    if k_norm_w is not None:
        k = k / torch.sqrt((k * k).mean(-1, keepdim=True) + eps) * k_norm_w
    if temp_coef:
        steps = torch.div(row_pos.long() + 1, temp_every, rounding_mode="floor")
        q = q * (1.0 + temp_coef * torch.log(steps.to(F32) + 1.0))[:, None]
    qo = torch.zeros((T, H, D), dtype=F32)
    qo[:, :, :d] = q.reshape(T, H, d)
    if store_kv:
        ko, vo = torch.zeros((T, G, D), dtype=F32), torch.zeros((T, G, D), dtype=F32)
        ko[:, :, :d] = k.reshape(T, G, d)
        vo[:, :, :dv] = v.reshape(T, G, dv)
        _store(k_pool, v_pool, ko, vo, row_pos, row_seg, block_tables, page_size)
    return qo.reshape(T, H * D).to(proj.dtype)


def _rotate(x, pos, cos, sin, rot_dims, rot_mode):
    if rot_mode == ROT_NONE or not rot_dims:
        return x
    half = rot_dims // 2
    shape = [x.shape[0]] + [1] * (x.dim() - 2) + [half]
    c, s = cos[pos].reshape(shape), sin[pos].reshape(shape)
    y = x.clone()
    if rot_mode == ROT_HALF:
        a, b = x[..., :half], x[..., half:rot_dims]
        y[..., :half] = a * c - b * s
        y[..., half:rot_dims] = b * c + a * s
    else:
        a, b = x[..., 0:rot_dims:2], x[..., 1:rot_dims:2]
        y[..., 0:rot_dims:2] = a * c - b * s
        y[..., 1:rot_dims:2] = b * c + a * s
    return y


def latent_store(q, kv, n_heads, dim, rot_dim, rank, head_size, c_norm_w, eps, cos, sin, rot_dims,
                 rot_mode, k_pool, v_pool, row_pos, row_seg, block_tables, page_size):
    H, d, rot, r, D = n_heads, dim, rot_dim, rank, head_size
    T = q.shape[0]
    pos = row_pos.long()
    kvf = kv.to(F32)
    c = kvf[:, :r]
    c = c / torch.sqrt((c * c).mean(-1, keepdim=True) + eps) * c_norm_w
    key = torch.zeros((T, 1, D), dtype=F32)
    key[:, 0, :r] = c
    key[:, 0, r:r + rot] = _rotate(kvf[:, r:r + rot], pos, cos, sin, rot_dims, rot_mode)
    val = torch.zeros((T, 1, D), dtype=F32)
    val[:, 0, :r] = c
    _store(k_pool, v_pool, key, val, row_pos, row_seg, block_tables, page_size)
    out = torch.zeros((T, H, D), dtype=F32)
    qr = q[:, :H * (d + rot)].to(F32).reshape(T, H, d + rot)[:, :, d:]
    out[:, :, r:r + rot] = _rotate(qr, pos, cos, sin, rot_dims, rot_mode)
    return out.reshape(T, H * D).to(q.dtype)


def headwise_linear(x, x_head_stride, weight, out=None, out_head_stride=None, out_dtype=None,
                    gate=None):
    H, n_out, n_in = weight.shape
    T = x.shape[0]
    if out is None:
        out = torch.empty((T, H * n_out), dtype=out_dtype or x.dtype)
        out_head_stride = n_out
    for h in range(H):
        xi = x[:, h * x_head_stride:h * x_head_stride + n_in].to(F32)
        y = xi @ weight[h].to(F32).T
        if gate is not None:
            y = y * torch.sigmoid(gate[:, h * n_out:(h + 1) * n_out].to(F32))
        out[:, h * out_head_stride:h * out_head_stride + n_out] = y.to(out.dtype)
    return out


CONV_SILU_MAX_TAPS = 17
GATE_SILU, GATE_SIGMOID = 0, 1


def conv_silu(x, taps, state, row_pos, row_seg, seg_start, seg_pos0, seg_slot, bias=None,
              activation=True):
    C, n = taps.shape
    xf = x[:, :C].to(F32)
    out = torch.empty((x.shape[0], C), dtype=F32)
    for s in range(seg_slot.shape[0]):
        t0, t1, slot = int(seg_start[s]), int(seg_start[s + 1]), int(seg_slot[s])
        hist = torch.zeros((n - 1, C)) if int(seg_pos0[s]) == 0 else state[slot].clone()
        seq = torch.cat([hist, xf[t0:t1]], dim=0)
        for i in range(t1 - t0):
            acc = torch.zeros(C)
            for j in range(n):
                acc = acc + taps[:, j] * seq[i + j]
            if bias is not None:
                acc = acc + bias
            out[t0 + i] = acc * torch.sigmoid(acc) if activation else acc
        if n > 1:
            state[slot] = seq[-(n - 1):]
    return out.to(x.dtype)


def matrix_state_recurrence(q, k, v, z, n_heads, n_qk_heads, dim, vdim, rate, z_bias, z_sign,
                            q_scale, state, seg_start, seg_pos0, seg_slot, beta=None,
                            unit_qk=False, unit_eps=1e-6, form="auto", decay="softplus",
                            bonus=None, silu_inputs=False, chunks=None, seg_chunk0=None,
                            chunk_rows=0):
    H, Hk, d, dv = n_heads, n_qk_heads, dim, vdim
    T = q.shape[0]

    def taken(x):
        if not silu_inputs:
            return x.to(F32)
        x = x.to(F32)
        return (x * torch.sigmoid(x)).to(q.dtype).to(F32)       # rounded as it is stored

    qf = taken(q[:, :Hk * d]).reshape(T, Hk, d)
    kf = taken(k[:, :Hk * d]).reshape(T, Hk, d)
    if unit_qk:
        qf = qf / torch.sqrt((qf * qf).sum(-1, keepdim=True) + unit_eps)
        kf = kf / torch.sqrt((kf * kf).sum(-1, keepdim=True) + unit_eps)
    qf = (qf * q_scale).repeat_interleave(H // Hk, dim=1)
    kf = kf.repeat_interleave(H // Hk, dim=1)
    vf = taken(v[:, :H * dv]).reshape(T, H, dv)
    if decay == "fixed":
        a = rate[None, :, None].expand(T, H, d)
    else:
        zz = z[:, :H * d].to(F32)
        if z_bias is not None:
            zz = zz + z_bias
        zz = zz.reshape(T, H, d)
        a = (torch.exp(-torch.exp(zz)) if decay == "double_exp" else
             torch.exp(-rate[:, None] * torch.nn.functional.softplus(z_sign * zz)))
    b = torch.sigmoid(beta[:, :H].to(F32)) if beta is not None else None
    out = torch.empty((T, H, dv), dtype=F32)
    for s in range(seg_slot.shape[0]):
        t0, t1, slot = int(seg_start[s]), int(seg_start[s + 1]), int(seg_slot[s])
        S = (torch.zeros((H, d, dv)) if int(seg_pos0[s]) == 0
             else state[slot].transpose(1, 2).clone())
        for t in range(t0, t1):
            if bonus is not None:
                kv = kf[t][:, :, None] * vf[t][:, None, :]
                out[t] = torch.einsum("hdv,hd->hv", S + bonus[:, :, None] * kv, qf[t])
                S = a[t][:, :, None] * S + kv
                continue
            S = a[t][:, :, None] * S
            if b is not None:
                u = b[t][:, None] * (vf[t] - torch.einsum("hdv,hd->hv", S, kf[t]))
            else:
                u = vf[t]
            S = S + kf[t][:, :, None] * u[:, None, :]
            out[t] = torch.einsum("hdv,hd->hv", S, qf[t])
        state[slot] = S.transpose(1, 2)
    return out.reshape(T, H * dv)


def head_norm_gate(o, weight, eps, gate, gate_kind, n_heads, vdim, out_dtype):
    H, dv = n_heads, vdim
    T = o.shape[0]
    x = o.reshape(T, H, dv)
    x = x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * weight        # [dv] or [H, dv]
    g = gate[:, :H * dv].to(F32).reshape(T, H, dv)
    g = g * torch.sigmoid(g) if gate_kind == GATE_SILU else torch.sigmoid(g)
    return (x * g).reshape(T, H * dv).to(out_dtype)



def rotate_widen_store(proj, n_heads, n_kv_heads, dim, vdim, head_size, cos, sin, rot_dims,
                       rot_mode, values_are_keys, k_pool, v_pool, row_pos, row_seg, block_tables,
                       page_size):
    H, G, d, dv, D = n_heads, n_kv_heads, dim, vdim, head_size
    T = proj.shape[0]
    p = proj.to(F32)
    pos = row_pos.long()
    q = p[:, :H * d].reshape(T, H, d)
    k = p[:, H * d:(H + G) * d].reshape(T, G, d)
    v = k if values_are_keys else p[:, (H + G) * d:(H + G) * d + G * dv].reshape(T, G, dv)
    qo, ko, vo = (torch.zeros((T, n, D), dtype=F32) for n in (H, G, G))
    qo[:, :, :d] = _rotate(q, pos, cos, sin, rot_dims, rot_mode)
    ko[:, :, :d] = _rotate(k, pos, cos, sin, rot_dims, rot_mode)
    vo[:, :, :dv] = v
    _store(k_pool, v_pool, ko, vo, row_pos, row_seg, block_tables, page_size)
    return qo.reshape(T, H * D).to(proj.dtype)


def token_shift_mix(h, mu, state, row_pos, row_seg, seg_start, seg_slot):
    T, W = h.shape
    hf = h.to(F32)
    before = torch.zeros((T, W), dtype=F32)
    for s in range(seg_slot.shape[0]):
        t0, t1, slot = int(seg_start[s]), int(seg_start[s + 1]), int(seg_slot[s])
        if t1 <= t0:
            continue
        if int(row_pos[t0]) > 0:
            before[t0] = state[slot]
        before[t0 + 1:t1] = hf[t0:t1 - 1]
        state[slot] = hf[t1 - 1]
    return (hf[None] + (before - hf)[None] * mu[:, None, :]).to(h.dtype)


def tanh(x):
    return torch.tanh(x.to(F32)).to(x.dtype)


def gated_unit_scan(gates, gate_bias, u, y, softplus_lam, rate, state, seg_start, seg_pos0,
                    seg_slot, chunks=None, seg_chunk0=None, gate_part=0):
    T, W = u.shape
    g = gates + gate_bias
    if gate_part:          # block by block (r | i) -> (r | i) of all channels
        g = g.reshape(T, W // gate_part, 2, gate_part).transpose(1, 2).reshape(T, 2 * W)
    a = torch.exp(-rate * torch.sigmoid(g[:, :W]) * softplus_lam)
    b = torch.sqrt(torch.clamp(1.0 - a * a, min=0.0)) * torch.sigmoid(g[:, W:]) * u.to(F32)
    z = y[:, :W].to(F32)
    gate = 0.5 * z * (1.0 + torch.tanh(0.7978845608028654 * (z + 0.044715 * z ** 3)))
    out = torch.empty((T, W), dtype=F32)
    for s in range(seg_slot.shape[0]):
        t0, t1, slot = int(seg_start[s]), int(seg_start[s + 1]), int(seg_slot[s])
        S = torch.zeros(W) if int(seg_pos0[s]) == 0 else state[slot].clone()
        for t in range(t0, t1):
            S = a[t] * S + b[t]
            out[t] = S * gate[t]
        state[slot] = S
    return out.to(u.dtype)


GATED_UNIT_STEP_MAX_PART = 4096


def gated_unit_step(proj, taps, conv_bias, conv_state, gate_w, gate_bias, softplus_lam, rate,
                    state, seg_pos0, seg_slot):
    T = proj.shape[0]
    W = taps.shape[0]
    part = gate_w.shape[2]
    rows = torch.arange(T, dtype=torch.int32)
    starts = torch.arange(T + 1, dtype=torch.int32)
    u = conv_silu(proj, taps, conv_state, seg_pos0, rows, starts, seg_pos0, seg_slot,
                  bias=conv_bias, activation=False)
    gates = torch.empty((T, 2 * W), dtype=F32)
    headwise_linear(u, part, gate_w, out=gates, out_head_stride=2 * part, out_dtype=F32)
    return gated_unit_scan(gates, gate_bias, u, proj[:, W:], softplus_lam, rate, state, starts,
                           seg_pos0, seg_slot, gate_part=part)


def pair_norm_sum(a, b, scale_a=1.0, scale_b=1.0, weight_a=None, weight_b=None, eps=0.0):
    def side(x, w):
        x = x.to(F32)
        if w is None:
            return x
        return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * w

    return scale_a * side(a, weight_a) + scale_b * side(b, weight_b)


def stream_enter(resid, delta, again, row):
    if delta is not None:
        resid.add_(delta.to(F32))
    if again is not None:
        resid.add_(again)
    if row is not None:
        resid.add_(row)


class _Plan:
    def __init__(self, experts):
        self.experts = experts


def moe_route(x, router, top, bias=None):
    logits = x.to(F32) @ router.T
    if bias is not None:
        logits = logits + bias
    best, chosen = torch.topk(logits, top, dim=-1)
    return chosen.to(torch.int32), torch.softmax(best, dim=-1)


def moe_plan(experts, n_experts):
    return _Plan(experts)


def moe_experts_gated(x, w_gate, w_up, plan):
    T, top = plan.experts.shape
    out = torch.empty((T, top, w_gate.shape[1]), dtype=x.dtype)
    for t in range(T):
        for k in range(top):
            e = int(plan.experts[t, k])
            g = w_gate[e].to(F32) @ x[t].to(F32)
            u = w_up[e].to(F32) @ x[t].to(F32)
            out[t, k] = (g / (1.0 + torch.exp(-g)) * u).to(x.dtype)
    return out


def moe_experts_down(act, w_down, plan):
    T, top = plan.experts.shape
    out = torch.empty((T, top, w_down.shape[1]), dtype=F32)
    for t in range(T):
        for k in range(top):
            out[t, k] = w_down[int(plan.experts[t, k])].to(F32) @ act[t, k].to(F32)
    return out


def moe_experts_activated(x, w_up, plan):
    T, top = plan.experts.shape
    out = torch.empty((T, top, w_up.shape[1]), dtype=x.dtype)
    for t in range(T):
        for k in range(top):
            u = torch.relu(w_up[int(plan.experts[t, k])].to(F32) @ x[t].to(F32))
            out[t, k] = (u * u).to(x.dtype)
    return out


def moe_combine(y, weights, plan, also=None):
    out = (y * weights[:, :, None]).sum(dim=1)
    if also is not None:
        for p in (also if also.dim() == 3 else also[None]):
            out = out + p.to(F32)
    return out


def head_norm_rotate_store(proj, n_heads, n_kv_heads, dim, vdim, head_size, q_norm_w, k_norm_w,
                           eps, cos, sin, rot_dims, rot_mode, k_pool, v_pool, row_pos, row_seg,
                           block_tables, page_size):
    H, G, d, dv, D = n_heads, n_kv_heads, dim, vdim, head_size
    T = proj.shape[0]
    p = proj.to(F32)
    pos = row_pos.long()
    q = p[:, :H * d].reshape(T, H, d)
    k = p[:, H * d:(H + G) * d].reshape(T, G, d)
    v = p[:, (H + G) * d:(H + G) * d + G * dv].reshape(T, G, dv)
    if q_norm_w is not None:
        q = q / torch.sqrt((q * q).mean(-1, keepdim=True) + eps) * q_norm_w
    if k_norm_w is not None:
        k = k / torch.sqrt((k * k).mean(-1, keepdim=True) + eps) * k_norm_w
    qo, ko, vo = (torch.zeros((T, n, D), dtype=F32) for n in (H, G, G))
    qo[:, :, :d] = _rotate(q, pos, cos, sin, rot_dims, rot_mode)
    ko[:, :, :d] = _rotate(k, pos, cos, sin, rot_dims, rot_mode)
    vo[:, :, :dv] = v
    _store(k_pool, v_pool, ko, vo, row_pos, row_seg, block_tables, page_size)
    return qo.reshape(T, H * D).to(proj.dtype)


HYPER_MAX_STREAMS = 8
ACT_RELU_SQUARED = 0


def hyper_step(streams, n_streams, width, source=None, y=None, mix=None, out_w=None, in_w=None,
               norm_w=None, eps=0.0, rows=None, rows_dtype=None, store=True):
    S = n_streams
    x = source[:, None, :].expand(-1, S, -1).to(F32) if source is not None else streams
    new = x
    if y is not None:
        upd = torch.zeros_like(x[:, 0])
        for p in (y if y.dim() == 3 else y[None]):
            upd = upd + p.to(F32)
        new = torch.einsum("st,nsw->ntw", mix, x) + out_w[None, :, None] * upd[:, None, :]
    if rows is None and store and streams is not None and (y is not None or source is not None):
        streams.copy_(new)
    if rows_dtype is None:
        return None
    u = torch.einsum("s,nsw->nw", in_w, new)
    if rows is not None:
        u = u[rows.long()]
    dev = u - u.mean(-1, keepdim=True)
    return (dev / torch.sqrt((dev * dev).mean(-1, keepdim=True) + eps) * norm_w).to(rows_dtype)


def rows_rmsnorm(x, n, weight, eps):
    v = x[:, :n].to(F32)
    return (v / torch.sqrt((v * v).mean(-1, keepdim=True) + eps) * weight).to(x.dtype)


def sigmoid_gate(x, gate, group):
    T, n = x.shape
    g = torch.sigmoid(gate[:, :n // group].to(F32)).repeat_interleave(group, dim=1)
    x.copy_((x.to(F32) * g).to(x.dtype))
    return x


def softcap_rows(x, cap):
    x.copy_(cap * torch.tanh(x / cap))
    return x


def activate(x, kind=0):
    r = torch.relu(x.to(F32))
    return (r * r).to(x.dtype)


ALL = ["moe_experts_activated", "head_norm_rotate_store", "hyper_step", "rows_rmsnorm", "sigmoid_gate",
       "softcap_rows", "activate", "add_group_rmsnorm", "add_group_rmsnorm_canon_step", "canon_conv", "scale_add_positions", "glu", "mingru_scan", "diff_store",
       "diff_combine", "moe_route", "moe_plan", "moe_experts_gated", "moe_experts_down", "moe_combine",
       "output_norm_add", "projection_norm_store", "latent_store", "headwise_linear", "conv_silu",
       "matrix_state_recurrence", "head_norm_gate", "rotate_widen_store", "token_shift_mix", "tanh",
       "gated_unit_scan", "gated_unit_step", "pair_norm_sum", "stream_enter",
       "embed_rows", "add_rmsnorm", "add_residual", "sum_partial_sums", "swiglu", "cast", "linear", "linear_swiglu",
       "interleave_gate_up", "shortconv", "linear_shortconv_step",
       "qk_norm_rope_store", "paged_attention", "sample_rows", "sample_filtered",
       "repeat_penalty", "history_set", "repeat_penalty_history", "history_append"]


def install(monkeypatch):
    """Replace the kernels' Python faces by these functions for one test."""
    import sys

    from kappai_amd.kernels import ops
    me = sys.modules[__name__]
    for name in ALL:
        monkeypatch.setattr(ops, name, getattr(me, name))


def make_cpu_runner(model, cache):
    """A StepRunner whose tables stay on the host (the emulated kernels read them there)."""
    from kappai_amd.engine.step import StepRunner

    class HostTableRunner(StepRunner):
        def __init__(self, model, cache):
            super().__init__(model, cache, device="cpu")

        def _upload(self, arrays):
            return {k: torch.from_numpy(np.ascontiguousarray(v).copy()) for k, v in arrays.items()}

    return HostTableRunner(model, cache)
