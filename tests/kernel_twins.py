"""Plain torch twins of every kernel: same arguments and cache layout, straightforward math.

Two uses: (1) each HIP kernel is compared with its twin on the GPU; (2) installed as the
ops backend (`PlainBackend`) they let the engine's bookkeeping (step function, cache manager,
scheduler, replay) be exercised on a machine without a GPU. They are test code: the engine
itself has no implementation but the HIP kernels.

All arithmetic is float32 (or float64 where a test asks), whatever the storage dtype; results
are rounded once to the output dtype.
"""
from __future__ import annotations

import torch


def gather_rows(src, idx, scale=None):
    if scale is not None:
        return src[idx.long()].float() * scale
    return src[idx.long()].clone()


def take_tokens(tokens, sampled, take):
    chosen = take.long() >= 0
    tokens[chosen] = sampled[take.long()[chosen]].to(tokens.dtype)


def rms_norm(x, weight, eps, residual, out_dtype, want_residual=True):
    r = x.float().sum(0) if x.dim() == 3 else x.float()
    if residual is not None:
        r = r + residual
    y = weight * (r * torch.rsqrt(r.pow(2).mean(-1, keepdim=True) + eps))
    return y.to(out_dtype), (r if want_residual else None)


def silu_and_mul(gu):
    inter = gu.shape[1] // 2
    g, u = gu[:, :inter].float(), gu[:, inter:].float()
    return (g * torch.sigmoid(g) * u).to(gu.dtype)


def _norm_rope(x, w, eps, table, positions):
    """x: [T, H, D] float32."""
    if w is not None:
        x = w * (x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps))
    if table is not None:
        cs = table[positions.long()]                        # [T, D/2, 2]
        c, s = cs[..., 0].unsqueeze(1), cs[..., 1].unsqueeze(1)
        half = x.shape[-1] // 2
        x1, x2 = x[..., :half], x[..., half:]
        x = torch.cat((x1 * c - x2 * s, x2 * c + x1 * s), dim=-1)
    return x


def write_pages(k, v, slots, k_cache, v_cache, page):
    """k, v: [T, Hkv, D] -> K [pages, Hkv, page, D], V [pages, Hkv, D, page]."""
    keep = slots >= 0
    s = slots[keep].long()
    pg, off = s // page, s % page
    k_cache[pg, :, off, :] = k[keep].to(k_cache.dtype)
    v_cache[pg, :, :, off] = v[keep].to(v_cache.dtype)


def qk_norm_rope_store(qkv, q_weight, k_weight, eps, table, positions, slots, k_cache, v_cache,
                       Hq, Hkv, D, page, store=True, position_bound=0):
    T = qkv.shape[0]
    if table is not None:
        # what the kernel's launcher refuses, and what it could not see: a position beyond the table
        assert position_bound <= table.shape[0], f"position bound {position_bound} beyond the table's {table.shape[0]} rows"
        assert T == 0 or int(positions[:T].max()) < table.shape[0], "a position beyond the rotation table"
    q = _norm_rope(qkv[:, :Hq * D].float().clone().view(T, Hq, D), q_weight, eps, table, positions)
    if Hkv:
        k = _norm_rope(qkv[:, Hq * D:(Hq + Hkv) * D].float().clone().view(T, Hkv, D), k_weight, eps, table, positions)
    qkv[:, :Hq * D] = q.reshape(T, Hq * D).to(qkv.dtype)
    if store:
        v = qkv[:, (Hq + Hkv) * D:].view(T, Hkv, D)
        write_pages(k.to(qkv.dtype), v, slots, k_cache, v_cache, page)
    elif Hkv:
        qkv[:, Hq * D:(Hq + Hkv) * D] = k.reshape(T, Hkv * D).to(qkv.dtype)


def store_kv(k, v, slots, k_cache, v_cache, page):
    write_pages(k, v, slots, k_cache, v_cache, page)


def paged_attention(q, k_cache, v_cache, page, block_tables, context_lens, seq_of_token, positions,
                    prefill_cu, num_decodes, max_decode_context, scale, window, Hq, Hkv, D,
                    force_simple=False, max_prefill_context=0, even_contexts=False, compute_dtype=torch.float32,
                    chunk=None, decode_as_prefill=False, keep_first=0, softcap=None, sinks=None):
    """Token by token: gather the keys this token may see through its request's block table
    and nothing else (so unowned pages are never read), softmax, weighted sum."""
    T = q.shape[0]
    out = torch.empty((T, Hq * D), dtype=q.dtype, device=q.device)
    G = Hq // Hkv
    seqs, where, lens = seq_of_token[:T].tolist(), positions[:T].tolist(), context_lens.tolist()      # one trip to the host
    for t in range(T):
        b, pos = seqs[t], where[t]
        lo = max(0, pos - window + 1) if window else 0
        if chunk:
            lo = pos - pos % chunk                         # a block mask: only the keys of the query's own block
        hi = min(pos + 1, lens[b])                         # a padding row (context 0) sees nothing
        if hi <= lo:
            out[t] = 0
            continue
        js = torch.arange(lo, hi, device=q.device)
        if keep_first and window and lo > 0:               # the first positions stay visible behind the window
            js = torch.cat((torch.arange(0, min(keep_first, lo, hi), device=q.device), js))
        pages = block_tables[b, (js // page).long()].long()
        assert (pages >= 0).all(), "attention would read a page the request does not hold"
        offs = js % page
        k = k_cache[pages, :, offs, :].to(compute_dtype)             # [n, Hkv, D]
        v = v_cache[pages, :, :, offs].to(compute_dtype)             # [n, Hkv, D]
        qt = q[t].to(compute_dtype).view(Hkv, G, D)                  # query head h belongs to key head h // G
        s = torch.einsum("nkd,kgd->kgn", k, qt) * scale
        if softcap:
            s = softcap * torch.tanh(s / softcap)
        if sinks is not None:                              # one more term in the denominator, no key, no value
            s = torch.cat((s, sinks.to(compute_dtype).view(Hkv, G, 1)), dim=-1)
            p = torch.softmax(s, dim=-1)[..., :-1]
        else:
            p = torch.softmax(s, dim=-1)
        out[t] = torch.einsum("kgn,nkd->kgd", p, v).reshape(Hq * D).to(q.dtype)
    return out


def decode_step_attention(qkv, q_weight, k_weight, eps, table, k_cache, v_cache, page, block_tables, context_lens,
                          max_context, scale, window, Hq, Hkv, D, even_contexts=False, compute_dtype=torch.float32,
                          chunk=None):
    """The two twins above, one after the other, on a copy of the rows: row r is request r's new token at
    position context_lens[r] - 1, its slot is what the block table names for that position (a row with
    context 0 is padding: nothing is written for it and it sees nothing)."""
    B = qkv.shape[0]
    assert table is None or max_context <= table.shape[0], f"a context of {max_context} beyond the table's {table.shape[0]} rows"
    ctx = context_lens[:B].long()
    positions = (ctx - 1).clamp(min=0).to(torch.int32)
    pages = block_tables[torch.arange(B, device=qkv.device), (positions // page).long()].long()
    slots = torch.where((ctx > 0) & (pages >= 0), pages * page + positions.long() % page, torch.full_like(pages, -1)).to(torch.int32)
    rows = qkv.clone()
    qk_norm_rope_store(rows, q_weight, k_weight, eps, table, positions, slots, k_cache, v_cache, Hq, Hkv, D, page, store=True)
    seq = torch.arange(B, dtype=torch.int32, device=qkv.device)
    return paged_attention(rows[:, :Hq * D], k_cache, v_cache, page, block_tables, context_lens, seq, positions, None, B,
                           max_context, scale, window, Hq, Hkv, D, compute_dtype=compute_dtype, chunk=chunk)


def linear(x, w, out_dtype=None, allow_partials=False, out=None):
    y = (x.float() @ w.float().t()).to(out_dtype or x.dtype)
    if out is not None:
        out.copy_(y)
        return out
    return y


def _gate(y):
    """silu(first half of the columns) * second half, on unrounded sums."""
    inter = y.shape[1] // 2
    return y[:, :inter] * torch.sigmoid(y[:, :inter]) * y[:, inter:]


def gated_linear(x, w, compute_dtype=torch.float32):
    return _gate(x.to(compute_dtype) @ w.to(compute_dtype).t()).to(x.dtype)


def norm_linear(x, residual, norm_weight, eps, w, out_dtype=None, want_residual=True, gated=False, compute_dtype=torch.float32):
    """The fused kernel's rounding points: gamma * r to the weight's dtype, product, then 1 / rms(r)."""
    r = x.float().sum(0) if x.dim() == 3 else x.float()
    if residual is not None:
        r = r + residual
    inv = torch.rsqrt(r.to(compute_dtype).pow(2).mean(-1, keepdim=True) + eps)
    y = ((norm_weight * r).to(w.dtype).to(compute_dtype) @ w.to(compute_dtype).t()) * inv
    if gated:
        y = _gate(y)
    return y.to(out_dtype or w.dtype), (r if want_residual else None)


def silu_mul_linear(gu, w, allow_partials=False):
    return linear(silu_and_mul(gu), w)


def add_rms_norm(y, weight, eps, stream, out_dtype):
    """stream + weight * y / rms(y) in float32 -> (rounded to out_dtype, float32)."""
    r = y.float().sum(0) if y.dim() == 3 else y.float()
    new = stream + weight * (r * torch.rsqrt(r.pow(2).mean(-1, keepdim=True) + eps))
    return (new if out_dtype == torch.float32 else new.to(out_dtype)), new


def activation(x, kind):
    v = x.float()
    if kind == "gelu_tanh":
        v = 0.5 * v * (1.0 + torch.tanh(0.7978845608028654 * (v + 0.044715 * v ** 3)))
    else:
        v = v * torch.sigmoid(v) if kind == "silu" else (torch.tanh(v) if kind == "tanh" else torch.relu(v) ** 2)
    return v.to(x.dtype)


def head_gate(o, gate, H, D):
    T = o.shape[0]
    o.copy_((o.float().view(T, H, D) * torch.sigmoid(gate.float())[:, :, None]).view(T, H * D).to(o.dtype))


def causal_conv(x, weight, bias, state, state_slots, cu_seqlens, q_lens):
    """x [T, C]; weight float32 [C, taps] (the last tap is the current token's), bias [C]; state [slots, C * (taps - 1)]
    float32: per channel the inputs before the request's next token, oldest first. silu(conv) in x's dtype; the state
    moves on."""
    T, C = x.shape
    taps = weight.shape[1]
    out = torch.empty((T, C), dtype=x.dtype, device=x.device)
    cu, slots = cu_seqlens.tolist(), state_slots.tolist()
    for b in range(len(cu) - 1):
        lo, hi = cu[b], cu[b + 1]
        if hi <= lo:
            continue
        held = state[slots[b]].view(C, taps - 1).t()                  # [taps - 1, C]
        seen = torch.cat((held, x[lo:hi].float()), 0)                  # [taps - 1 + n, C]
        acc = bias.float().expand(hi - lo, C).clone() if bias is not None else torch.zeros((hi - lo, C), device=x.device)
        for j in range(taps):
            acc += weight[:, j].float() * seen[j:j + hi - lo]
        out[lo:hi] = (acc * torch.sigmoid(acc)).to(x.dtype)
        state[slots[b]] = seen[seen.shape[0] - (taps - 1):].t().reshape(-1)
    return out


def softplus(x):
    return torch.where(x > 20, x, torch.log1p(torch.exp(torch.clamp(x, max=20))))


def linear_recurrence(q, k, v, state, state_slots, cu_seqlens, q_lens, H, G, N, P, decay=None, dt=None, dt_bias=None,
                      rate=None, skip=None, silu=False):
    """S_t = a S_(t-1) + b k_t v_t^T, y_t = S_t^T q_t (+ skip v_t), float32, token by token. q, k [T, G * N], v [T, H * P];
    state [slots, H * N * P]. a, b: decay[h], 1; or exp(-rate[h] dt), dt with dt = softplus(dt[t, h] + dt_bias[h])."""
    T = v.shape[0]
    y = torch.zeros((T, H * P), dtype=torch.float32, device=v.device)
    cu, slots = cu_seqlens.tolist(), state_slots.tolist()
    per = H // G
    for b in range(len(cu) - 1):
        S = state[slots[b]].view(H, N, P).clone()
        for t in range(cu[b], cu[b + 1]):
            kt, qt, vt = k[t].float().view(G, N), q[t].float().view(G, N), v[t].float().view(H, P)
            if silu:
                kt, qt, vt = (z * torch.sigmoid(z) for z in (kt, qt, vt))
            if decay is not None:
                a, bb = decay.float(), torch.ones(H)
            else:
                step = softplus(dt[t].float() + dt_bias)
                a, bb = torch.exp(-rate * step), step
            kh, qh = kt.repeat_interleave(per, 0), qt.repeat_interleave(per, 0)
            S = a[:, None, None] * S + (bb[:, None] * kh)[:, :, None] * vt[:, None, :]
            out = torch.einsum("hnp,hn->hp", S, qh)
            if skip is not None:
                out = out + skip[:, None] * vt
            y[t] = out.reshape(-1)
        state[slots[b]] = S.reshape(-1)
    return y


def gated_rms_norm(y, gate, weight, eps, groups, kind, out_dtype):
    """kind "silu_before": unit rms per group of (y * silu(gate)), times weight; "sigmoid_behind": unit rms of y, times
    weight, times sigmoid(gate). y float32 [T, n] or partial sums [S, T, n]."""
    r = y.float().sum(0) if y.dim() == 3 else y.float()
    g = gate.float()
    T, n = r.shape
    if kind == "silu_before":
        r = r * (g * torch.sigmoid(g))
    r = r.view(T, groups, n // groups)
    r = (r * torch.rsqrt(r.pow(2).mean(-1, keepdim=True) + eps)).view(T, n) * weight
    if kind == "sigmoid_behind":
        r = r * torch.sigmoid(g)
    if kind == "silu_behind":
        r = r * (g * torch.sigmoid(g))
    return r.to(out_dtype)


def add_bias(x, bias, out_dtype):
    r = (x.float().sum(0) if x.dim() == 3 else x.float()).clone()
    r[:, : bias.numel()] += bias
    return r.to(out_dtype)


def sigmoid_gate_(o, gate):
    o.copy_((o.float() * torch.sigmoid(gate.float())).to(o.dtype))
    return o


def glu_clamped(gu, limit, alpha):
    inter = gu.shape[1] // 2
    g = torch.clamp(gu[:, :inter].float(), max=limit)
    u = torch.clamp(gu[:, inter:].float(), -limit, limit)
    return (g * torch.sigmoid(alpha * g) * (u + 1.0)).to(gu.dtype)


def weighted_sum(terms, norm_weight=None, eps=0.0, stream=None, out_dtype=None):
    total = None
    for term in terms:
        t, sc, b = term[:3]
        v = t.float().sum(0) if t.dim() == 3 else t.float()
        if b is not None:
            v = v + b
        if len(term) > 3 and term[3] is not None:
            v = v * torch.sigmoid(term[3].float().reshape(-1, 1))
        total = sc * v if total is None else total + sc * v
    if norm_weight is None:
        return total
    new = stream + norm_weight * (total * torch.rsqrt(total.pow(2).mean(-1, keepdim=True) + eps))
    return (new if out_dtype in (None, torch.float32) else new.to(out_dtype)), new


def token_shift(x, mu, state, state_slots, cu_seqlens, seq_of_token):
    T, n = x.shape
    out = torch.empty((mu.shape[0], T, n), dtype=x.dtype, device=x.device)
    cu, slots = cu_seqlens.tolist(), state_slots.tolist()
    for b in range(len(slots)):
        lo, hi = cu[b], cu[b + 1]
        if hi <= lo:
            continue
        now = x[lo:hi].float()
        before = torch.cat((state[slots[b]][None, :].clone(), now[:-1]), 0)
        out[:, lo:hi] = (now[None] + (before - now)[None] * mu[:, None, :]).to(x.dtype)
        state[slots[b]] = now[-1]
    return out


def decay_rows_recurrence(q, k, v, raw, state, state_slots, cu_seqlens, q_lens, H, G, N, P, rule, base, rate=None, bonus=None,
                          beta=None, unit_eps=None, q_scale=1.0):
    """Token by token, float32. rule "bonus": y = (S + diag(bonus) k v^T)^T q, S <- diag(d) S + k v^T with d =
    exp(-exp(raw + base)); rule "delta": S <- diag(d) S with d = exp(-rate softplus(raw + base)), u = sigmoid(beta) (v -
    S^T k), S <- S + k u^T, y = S^T q."""
    T = v.shape[0]
    y = torch.zeros((T, H * P), dtype=torch.float32, device=v.device)
    cu, slots = cu_seqlens.tolist(), state_slots.tolist()
    per = H // G
    for b in range(len(slots)):
        S = state[slots[b]].view(H, N, P).clone()
        for t in range(cu[b], cu[b + 1]):
            qt = q[t].float().view(G, N).repeat_interleave(per, 0)
            kt = k[t].float().view(G, N).repeat_interleave(per, 0)
            vt = v[t].float().view(H, P)
            if unit_eps is not None:
                qt = qt / torch.sqrt(qt.pow(2).sum(-1, keepdim=True) + unit_eps)
                kt = kt / torch.sqrt(kt.pow(2).sum(-1, keepdim=True) + unit_eps)
            qt = qt * q_scale
            z = raw[t].float().view(H, N) + base.view(H, N)
            if rule == "bonus":
                d = torch.exp(-torch.exp(z))
                kv = kt[:, :, None] * vt[:, None, :]
                out = torch.einsum("hnp,hn->hp", S + bonus.view(H, N)[:, :, None] * kv, qt)
                S = d[:, :, None] * S + kv
            elif rule == "gated":
                d = torch.exp(-rate[:, None] * softplus(-z))          # sigmoid(z) ^ rate
                S = d[:, :, None] * S + kt[:, :, None] * vt[:, None, :]
                out = torch.einsum("hnp,hn->hp", S, qt)
            else:
                d = torch.exp(-rate[:, None] * softplus(z))
                S = d[:, :, None] * S
                u = torch.sigmoid(beta[t].float())[:, None] * (vt - torch.einsum("hnp,hn->hp", S, kt))
                S = S + kt[:, :, None] * u[:, None, :]
                out = torch.einsum("hnp,hn->hp", S, qt)
            y[t] = out.reshape(-1)
        state[slots[b]] = S.reshape(-1)
    return y


def scaled_sum_norm(stream, terms, mult, w1, w2, eps, out_dtype):
    """stream + mult * sum_i scale_i * term_i in float32, then up to two RMS norms of it."""
    new = stream.float()
    if terms:
        add = torch.zeros_like(new)
        for t, sc in terms:
            v = t.float().sum(0) if t.dim() == 3 else t.float()
            add = add + (v if sc is None else sc * v)
        new = new + mult * add
    elif stream.dtype == torch.float32:
        new = stream
    u = new * torch.rsqrt(new.pow(2).mean(-1, keepdim=True) + eps)
    return new, (None if w1 is None else (u * w1).to(out_dtype)), (None if w2 is None else (u * w2).to(out_dtype))


def softcap_(z, cap):
    z.copy_(cap * torch.tanh(z / cap))
    return z


def qkv_prepare_store(rows, bias, q_weight, k_weight, eps, nq, nk, temperature, positions, slots, k_cache, v_cache,
                      Hq, Hkv, D, page, vdim, mix=0, lam=None, v_first=None):
    T = rows.shape[0]
    wq, wk = Hq * D, Hkv * D
    r = rows[:, :wq + 2 * wk].float()
    if bias is not None:
        r = r + bias[:wq + 2 * wk]
    q, k, v = r[:, :wq], r[:, wq:wq + wk], r[:, wq + wk:].clone()
    if q_weight is not None:
        q = q * torch.rsqrt(q.pow(2).sum(-1, keepdim=True) / nq + eps) * q_weight
        k = k * torch.rsqrt(k.pow(2).sum(-1, keepdim=True) / nk + eps) * k_weight
    if temperature:
        coef, every = temperature
        steps = torch.div(positions[:T].long() + 1, every, rounding_mode="floor").float()
        q = q * (1.0 + coef * torch.log(steps + 1.0))[:, None]
    if mix:
        real = v.view(T, Hkv, D)[:, :, :vdim]
        if mix == 1:
            v_first.copy_(real.reshape(T, Hkv * vdim))
        else:
            real.copy_((1.0 - lam.float()) * real + lam.float() * v_first.view(T, Hkv, vdim))
    dt = k_cache.dtype
    write_pages(k.reshape(T, Hkv, D).to(dt), v.reshape(T, Hkv, D).to(dt), slots[:T], k_cache, v_cache, page)
    return q.to(dt).contiguous()


def moe_route(x, router, top, group_count=1, group_keep=1, rule=None):
    z = x.float() @ router.float().t()
    sigmoid = rule is not None and rule.scoring == "sigmoid"
    s = torch.sigmoid(z) if sigmoid else torch.softmax(z, dim=-1)
    T, E = s.shape
    m = s.clone() if rule is None or rule.correction is None else s + rule.correction
    if group_count > 1 and group_keep < group_count:
        per = E // group_count
        count = min(1 if rule is None else rule.group_top, per)
        gs = m.view(T, group_count, per).topk(count, -1).values.sum(-1)
        kept = torch.zeros((T, group_count), dtype=torch.bool, device=x.device)
        for _ in range(group_keep):
            best = torch.where(kept, torch.full_like(gs, -float("inf")), gs).argmax(-1)      # ties: the lower index
            kept[torch.arange(T), best] = True
        m = torch.where(kept.repeat_interleave(per, 1), m, torch.full_like(m, -float("inf")))
    ids = torch.empty((T, top), dtype=torch.int64, device=x.device)
    for j in range(top):
        best = m.argmax(-1)
        ids[:, j] = best
        m[torch.arange(T), best] = -float("inf")
    w = torch.gather(s, 1, ids)
    if rule is None or rule.normalise:
        w = w / (w.sum(-1, keepdim=True) + 1e-20)
    return ids.to(torch.int32), (w * (1.0 if rule is None else rule.scale)).float()


def route_and_run_experts(x, router, top, group_count, group_keep, gate_up, down, rule=None, gated=True):
    ids, weights = moe_route(x, router, top, group_count, group_keep, rule)
    return routed_experts(x, ids, weights, gate_up, down, gated=gated)


def routed_experts(x, ids, weights, gate_up, down, force_simple=False, tile_rows=None, choose_from=None, gated=True):
    T, K = x.shape
    top = ids.shape[1]
    F = gate_up.shape[1] // 2 if gated else gate_up.shape[1]
    out = torch.zeros((top, T, down.shape[1]), dtype=torch.float32, device=x.device)
    xf = x.float()
    for j in range(top):
        for e in ids[:, j].unique().tolist():
            rows = (ids[:, j] == e).nonzero().flatten()
            gu = xf[rows] @ gate_up[e].float().t()
            act = gu[:, :F] * torch.sigmoid(gu[:, :F]) * gu[:, F:] if gated else torch.relu(gu) ** 2
            out[j, rows] = (act.to(x.dtype).float() @ down[e].float().t()) * weights[rows, j][:, None]
    return out


def latent_prepare(rows, q_off, kv_off, H, dn, dr, R, D, norm_weight, eps, table, positions, slots, k_cache, v_cache, page):
    T = rows.shape[0]
    qa = torch.zeros((T, H, D), dtype=rows.dtype, device=rows.device)
    cs = table[positions.long()] if dr else None                      # [T, dr / 2, 2]

    def turn(x):                                                      # [..., dr] in adjacent pairs
        u, v = x[..., 0::2].float(), x[..., 1::2].float()
        c, s = cs[..., 0], cs[..., 1]
        while c.dim() < u.dim():
            c, s = c.unsqueeze(1), s.unsqueeze(1)
        out = torch.empty_like(x, dtype=torch.float32)
        out[..., 0::2], out[..., 1::2] = u * c - v * s, v * c + u * s
        return out

    q = rows[:, q_off:q_off + H * (dn + dr)].reshape(T, H, dn + dr)
    if dr:
        qa[:, :, R:R + dr] = turn(q[:, :, dn:]).to(rows.dtype)
    if kv_off is not None:
        kv = rows[:, kv_off:kv_off + R + dr].float()
        c = kv[:, :R] * torch.rsqrt(kv[:, :R].pow(2).mean(-1, keepdim=True) + eps) * norm_weight
        key = torch.zeros((T, 1, D), dtype=torch.float32, device=rows.device)
        key[:, 0, :R] = c
        if dr:
            key[:, 0, R:R + dr] = turn(kv[:, R:])
        val = torch.zeros((T, 1, D), dtype=torch.float32, device=rows.device)
        val[:, 0, :R] = c
        write_pages(key.to(rows.dtype), val.to(rows.dtype), slots, k_cache, v_cache, page)
    return qa.view(T, H * D)


def heads_linear(x, w, out):
    out.copy_(torch.einsum("thk,hnk->thn", x.float(), w.float()).to(out.dtype))
    return out


def _fmix32(h):
    m = 0xFFFFFFFF
    h = h & m
    h ^= h >> 16
    h = (h * 0x85EBCA6B) & m
    h ^= h >> 13
    h = (h * 0xC2B2AE35) & m
    h ^= h >> 16
    return h


def row_key(seed, stream, index):
    """The two 32-bit words that key the noise of output number `index` of the request with noise stream
    `stream` under `seed`: three rounds of SplitMix64's output function (add the golden-ratio constant, two
    xor-shift-multiplies, a last xor-shift), each taking the next of (seed, stream, index) xored into the state;
    (low word, high word) of the result. Written with numpy's wrapping 64-bit integers."""
    import numpy as np
    u = np.uint64

    def mix(x):
        with np.errstate(over="ignore"):
            x = x + u(0x9E3779B97F4A7C15)
            x = (x ^ (x >> u(30))) * u(0xBF58476D1CE4E5B9)
            x = (x ^ (x >> u(27))) * u(0x94D049BB133111EB)
        return x ^ (x >> u(31))

    x = mix(u(seed % (1 << 64)))
    x = mix(x ^ u(stream % (1 << 64)))
    x = mix(x ^ u(index % (1 << 64)))
    return int(x & u(0xFFFFFFFF)), int(x >> u(32))


def exp_noise(keys, V, device):
    """E ~ Exp(1), [S, V], the kernel's hash: fmix32(fmix32(v ^ k0) + k1) -> 24 bits -> -log(u)."""
    k = keys.to(torch.int64) & 0xFFFFFFFF
    v = torch.arange(V, dtype=torch.int64, device=device)[None, :]
    r = _fmix32((_fmix32(v ^ k[:, 0:1]) + k[:, 1:2]) & 0xFFFFFFFF)
    u = ((r >> 8).to(torch.float32) + 0.5) * (1.0 / 16777216.0)
    return -torch.log(u)


def sample_scores(logits, temperatures, keys):
    """The quantity whose argmax the sampler returns, [S, V] float32."""
    t = temperatures[:, None]
    noisy = logits / torch.where(t > 0, t, torch.ones_like(t)) - torch.log(exp_noise(keys, logits.shape[1], logits.device))
    return torch.where(t > 0, noisy, logits)


def sample(logits, temperatures, keys):
    return sample_scores(logits, temperatures, keys).argmax(dim=-1).to(torch.int32)


class PlainBackend:
    name = "plain"
    gather_rows = staticmethod(gather_rows)
    take_tokens = staticmethod(take_tokens)
    rms_norm = staticmethod(rms_norm)
    silu_and_mul = staticmethod(silu_and_mul)
    qk_norm_rope_store = staticmethod(qk_norm_rope_store)
    store_kv = staticmethod(store_kv)
    paged_attention = staticmethod(paged_attention)
    decode_step_attention = staticmethod(decode_step_attention)
    linear = staticmethod(linear)
    silu_mul_linear = staticmethod(silu_mul_linear)
    norm_linear = staticmethod(norm_linear)
    gated_linear = staticmethod(gated_linear)
    sample = staticmethod(sample)
    add_rms_norm = staticmethod(add_rms_norm)
    activation = staticmethod(activation)
    head_gate = staticmethod(head_gate)
    causal_conv = staticmethod(causal_conv)
    linear_recurrence = staticmethod(linear_recurrence)
    gated_rms_norm = staticmethod(gated_rms_norm)
    scaled_sum_norm = staticmethod(scaled_sum_norm)
    softcap_ = staticmethod(softcap_)
    qkv_prepare_store = staticmethod(qkv_prepare_store)
    add_bias = staticmethod(add_bias)
    sigmoid_gate_ = staticmethod(sigmoid_gate_)
    glu_clamped = staticmethod(glu_clamped)
    weighted_sum = staticmethod(weighted_sum)
    token_shift = staticmethod(token_shift)
    decay_rows_recurrence = staticmethod(decay_rows_recurrence)
    moe_route = staticmethod(moe_route)
    routed_experts = staticmethod(routed_experts)
    route_and_run_experts = staticmethod(route_and_run_experts)
    latent_prepare = staticmethod(latent_prepare)
    heads_linear = staticmethod(heads_linear)
