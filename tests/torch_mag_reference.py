"""Plain PyTorch (autograd, float64 state) restatement of one MAG layer, the yardstick for
nl_hecate_amd.mag_layer: sliding-window attention gated by the sigmoid of a sum of Titans
memories (core/src/gpu_forward.rs:864-1071).  Mirrors the GPU path's conventions: q/k/v of the
attention branch and the attention output pass through bf16 (straight-through), the gates see
k and v without gradient (the GPU chain drops that term), `chunkwise` takes a chunk's errors
against the chunk-start memory."""
import math

import torch


def _bf16_st(x):
    return x + (x.to(torch.bfloat16).to(x.dtype) - x).detach()


def swa(q, k, v, nh, window):
    bs, s, d = q.shape
    hd = d // nh
    qh, kh, vh = (t.view(bs, s, nh, hd).transpose(1, 2) for t in (q, k, v))
    sc = qh @ kh.transpose(-1, -2) / math.sqrt(hd)
    i = torch.arange(s)
    mask = (i[None, :] <= i[:, None]) & (i[None, :] > i[:, None] - window)
    sc = sc.masked_fill(~mask, float("-inf"))
    return (torch.softmax(sc, -1) @ vh).transpose(1, 2).reshape(bs, s, d)


def titans(kh, vh, qh, al, th, et, m0, s0, chunk=None):
    """kh,vh,qh [B,s,hd]; gates [B,s]; exact recurrence, or chunkwise (errors vs chunk-start M)."""
    B, s, hd = kh.shape
    M, S = m0.clone(), s0.clone()
    ys = []
    for t in range(s):
        if chunk and t % chunk == 0:
            M0 = M
        Me = M0 if chunk else M
        e = torch.einsum("bij,bj->bi", Me, kh[:, t]) - vh[:, t]
        S = et[:, t, None, None] * S - th[:, t, None, None] * torch.einsum("bi,bj->bij", e, kh[:, t])
        M = (1 - al[:, t, None, None]) * M + S
        ys.append(torch.einsum("bij,bj->bi", M, qh[:, t]))
    return torch.stack(ys, 1), M, S


def forward(P, x, nh, window, active, m_states, s_states, rule="exact", chunk=None, bf16_mem=False):
    """P: dict of leaf tensors (w_q, w_k, w_v, w_o, levels=[dict(...)]); returns out and final states."""
    bs, s, d = x.shape
    hd = d // nh
    x2 = x.reshape(bs * s, d)
    q, k, v = (_bf16_st(x2 @ P[n].t()).view(bs, s, d) for n in ("w_q", "w_k", "w_v"))
    attn = _bf16_st(swa(q, k, v, nh, window))
    ys, finals = [], []
    for lv, L in enumerate(P["levels"]):
        if not active[lv]:
            qr = (x2 @ L["w_q"].t()).view(bs, s, nh, hd)
            m = m_states[lv][:nh].view(nh, hd, hd)
            ys.append(torch.einsum("hij,bthj->bthi", m, qr).reshape(bs, s, d))
            finals.append((m_states[lv], s_states[lv]))
            continue
        nrm = lambda t: t / t.norm(dim=-1, keepdim=True).clamp_min(1e-8)
        km, vm, qm = nrm(x2 @ L["w_k"].t()), x2 @ L["w_v"].t(), nrm(x2 @ L["w_q"].t())
        kv = torch.cat([km.detach(), vm.detach()], -1)
        al = torch.sigmoid(kv @ L["w_alpha"] + L["b_alpha"])
        th = torch.nn.functional.softplus(kv @ L["w_theta"] + L["b_theta"])
        et = torch.sigmoid(kv @ L["w_eta"] + L["b_eta"])
        heads = lambda t: t.view(bs, s, nh, hd).transpose(1, 2).reshape(bs * nh, s, hd)
        bc = lambda g: g.view(bs, 1, s).expand(bs, nh, s).reshape(bs * nh, s)
        kh, vh, qh = heads(km), heads(vm), heads(qm)
        if bf16_mem:
            kh, vh, qh = _bf16_st(kh), _bf16_st(vh), _bf16_st(qh)
        yh, M, S = titans(kh, vh, qh, bc(al), bc(th), bc(et), m_states[lv].view(-1, hd, hd),
                          s_states[lv].view(-1, hd, hd), chunk if rule == "chunkwise" else None)
        ys.append(yh.view(bs, nh, s, hd).transpose(1, 2).reshape(bs, s, d))
        finals.append((M.reshape(-1, hd * hd), S.reshape(-1, hd * hd)))
    kk = len(P["levels"])
    y_comb = sum(ys) * (1 / math.sqrt(kk) if kk > 2 else 1.0)
    gated = attn * torch.sigmoid(y_comb)
    return (gated.view(bs * s, d) @ P["w_o"].t()).view(bs, s, d), finals
