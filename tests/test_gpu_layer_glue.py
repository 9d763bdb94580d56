"""The layer step's strided / packed glue entry points (layer_glue.hip) against the separate kernels
they replace (memory_inputs_fused, memory_grads_fused, gate_backward, split_pack_bf16, cms_combine_gate):
layout moves and bf16 splits bit-exact, sums to 1e-5 relative (other summation order)."""
import ctypes

import numpy as np
import pytest
import torch

from nl_hecate_amd import dispatch as D
from nl_hecate_amd.ffi import lib

pytestmark = pytest.mark.gpu


def _rn(gen, *sh):
    return torch.randn(*sh, device="cuda", generator=gen)


def _close(name, a, b, tol=1e-5):
    a, b = a.double(), b.double()
    err = float((a - b).abs().max() / max(float(b.abs().max()), 1e-30))
    assert err <= tol, f"{name}: relative error {err:.3e} > {tol}"


def _split(x):
    h = x.to(torch.bfloat16)
    return h, (x - h.float()).to(torch.bfloat16)


def test_split_pack_with_strides_and_offsets():
    g = torch.Generator(device="cuda").manual_seed(1)
    n, d, ld = 37, 24, 240
    wide = _rn(g, n, 3 * 40)                       # sources are column ranges of a wider tensor
    srcs = [wide[:, 0:d], wide[:, 40:40 + d], wide[:, 80:80 + d]]
    out = torch.full((n, ld), 7.0, device="cuda", dtype=torch.bfloat16)
    ptrs = (ctypes.c_void_p * 3)(*[t.data_ptr() for t in srcs])
    lib.split_pack_bf16_ld_rocm(ptrs, 3, 120, out.data_ptr(), n, d, ld, 4, 4 + 3 * d + 8, 160)
    torch.cuda.synchronize()
    for i, sx in enumerate(srcs):
        h, l = _split(sx.contiguous())
        assert torch.equal(out[:, 4 + i * d:4 + (i + 1) * d], h)
        assert torch.equal(out[:, 160 + i * d:160 + (i + 1) * d], h)
        o = 4 + 3 * d + 8 + i * d
        assert torch.equal(out[:, o:o + d], l)
    assert torch.all(out[:, :4] == 7.0) and torch.all(out[:, 4 + 3 * d:4 + 3 * d + 8] == 7.0)


def test_split_pack_weights_layouts_and_the_products_they_serve():
    g = torch.Generator(device="cuda").manual_seed(2)
    rows, rs, d, n = 96, 64, 32, 50
    pack, x, gr = 0.3 * _rn(g, rows, d), _rn(g, n, d), _rn(g, n, rs)
    wb = torch.zeros(rows, 3 * d, device="cuda", dtype=torch.bfloat16)
    ws = torch.zeros(3 * rs, d, device="cuda", dtype=torch.bfloat16)
    lib.split_pack_weights_rocm(pack.data_ptr(), rows, rs, d, wb.data_ptr(), ws.data_ptr())
    h, l = _split(pack)
    assert torch.equal(wb, torch.cat([h, l, h], 1))
    assert torch.equal(ws, torch.cat([h[:rs], h[:rs], l[:rs]], 0))
    # forward: (xh | xh | xl) . (Wh | Wl | Wh)^T ~ x W^T; backward: (H | L | H) . (Wh ; Wh ; Wl) ~ g W
    xh, xl = _split(x)
    y = torch.mm(torch.cat([xh, xh, xl], 1), wb.t(), out_dtype=torch.float32)
    _close("x W^T", y, x.double() @ pack.double().t(), 2e-5)
    gh, gl = _split(gr)
    dx = torch.mm(torch.cat([gh, gl, gh], 1), ws, out_dtype=torch.float32)
    _close("g W", dx, gr.double() @ pack[:rs].double(), 2e-5)


@pytest.mark.parametrize("bs,s,nh,hd,bf16", [(2, 37, 4, 16, False), (1, 100, 8, 64, True), (3, 5, 2, 24, True),
                                            (1, 9, 16, 64, True)])
def test_level_glue_on_strided_projections_matches_the_contiguous_kernels(bs, s, nh, hd, bf16):
    d, n, B = nh * hd, bs * s, bs * nh
    g = torch.Generator(device="cuda").manual_seed(5 + s)
    ld = 3 * d + 8
    proj = _rn(g, n, ld)
    proj[3 % n, :d] = 0.0                           # a zero k row takes the norm < eps branches
    k0, v0, q0 = (proj[:, i * d:(i + 1) * d].contiguous() for i in range(3))
    w = [0.1 * _rn(g, 2 * d) for _ in range(3)]
    bias = [_rn(g, 1) for _ in range(3)]
    hdt = torch.bfloat16 if bf16 else torch.float32
    z = lambda *sh, dt=torch.float32: torch.zeros(*sh, device="cuda", dtype=dt)
    # contiguous reference kernels
    kn1, qn1, gates1 = z(n), z(n), [z(n) for _ in range(3)]
    heads1, gh1 = [z(B, s, hd, dt=hdt) for _ in range(3)], [z(B, s) for _ in range(3)]
    D.call("memory_inputs_fused_rocm", k0, v0, q0, w[0], bias[0], w[1], bias[1], w[2], bias[2], kn1, qn1, *gates1,
           *heads1, *gh1, bs, s, nh, hd, 1e-8, int(bf16))
    # strided
    p2 = proj.clone()
    k2, v2, q2 = (p2[:, i * d:(i + 1) * d] for i in range(3))
    kn2, qn2, gates2 = z(n), z(n), [z(n) for _ in range(3)]
    heads2, gh2 = [z(B, s, hd, dt=hdt) for _ in range(3)], [z(B, s) for _ in range(3)]
    lib.level_inputs_fused_rocm(k2.data_ptr(), v2.data_ptr(), q2.data_ptr(), ld, w[0].data_ptr(), bias[0].data_ptr(),
                                w[1].data_ptr(), bias[1].data_ptr(), w[2].data_ptr(), bias[2].data_ptr(),
                                kn2.data_ptr(), qn2.data_ptr(), *[t.data_ptr() for t in gates2],
                                *[t.data_ptr() for t in heads2], *[t.data_ptr() for t in gh2], bs, s, nh, hd, 1e-8,
                                int(bf16), 1)
    torch.cuda.synchronize()
    assert torch.equal(p2[:, 3 * d:], proj[:, 3 * d:]) and torch.equal(v2, v0)
    _close("k", k2, k0); _close("q", q2, q0); _close("k_norms", kn2, kn1); _close("q_norms", qn2, qn1)
    for a, b in zip(gates2 + gh2, gates1 + gh1):
        _close("gate", a, b)
    for a, b in zip(heads2, heads1):
        _close("heads", a.float(), b.float(), 1e-2 if bf16 else 1e-5)   # one bf16 ulp where a sum differs
    # backward glue: reference = memory_grads_fused + gate_backward + split
    dh, dg = [_rn(g, B, s, hd) for _ in range(3)], [_rn(g, B, s) for _ in range(3)]
    dk1, dv1, dq1, dgs1 = z(n, d), z(n, d), z(n, d), [z(n) for _ in range(3)]
    D.call("memory_grads_fused_rocm", *dh, *dg, k0, q0, kn1, qn1, dk1, dv1, dq1, *dgs1, bs, s, nh, hd, 1e-8)
    gw1, gb1 = [z(2 * d) for _ in range(3)], [z(1) for _ in range(3)]
    D.call("gate_backward_cuda", dgs1[0], gates1[0], dgs1[1], gates1[1], dgs1[2], gates1[2], k0, v0, gw1[0], gb1[0],
           gw1[1], gb1[1], gw1[2], gb1[2], n, d, 1, 1)
    W = 3 * d + 12                                  # the slab sits at column 8 of each third of P
    P = torch.full((n, 3 * W), 3.0, device="cuda", dtype=torch.bfloat16)
    gw2, gb2 = [z(2 * d) for _ in range(3)], [z(1) for _ in range(3)]
    lib.level_grads_packed_rocm(*[t.data_ptr() for t in dh], *[t.data_ptr() for t in dg], k2.data_ptr(), v2.data_ptr(),
                                q2.data_ptr(), ld, kn2.data_ptr(), qn2.data_ptr(), *[t.data_ptr() for t in gates2],
                                P.data_ptr(), 3 * W, 8, W + 8, 2 * W + 8, gw2[0].data_ptr(), gb2[0].data_ptr(),
                                gw2[1].data_ptr(), gb2[1].data_ptr(), gw2[2].data_ptr(), gb2[2].data_ptr(), bs, s, nh,
                                hd, 1e-8, 0)
    # the same from the projections as they came (not normalised in place) and the stored norms
    p3 = proj.clone()
    k3, v3, q3 = (p3[:, i * d:(i + 1) * d] for i in range(3))
    heads3 = [z(B, s, hd, dt=hdt) for _ in range(3)]
    lib.level_inputs_fused_rocm(k3.data_ptr(), v3.data_ptr(), q3.data_ptr(), ld, w[0].data_ptr(), bias[0].data_ptr(),
                                w[1].data_ptr(), bias[1].data_ptr(), w[2].data_ptr(), bias[2].data_ptr(),
                                kn2.data_ptr(), qn2.data_ptr(), *[t.data_ptr() for t in gates2],
                                *[t.data_ptr() for t in heads3], *[t.data_ptr() for t in gh2], bs, s, nh, hd, 1e-8,
                                int(bf16), 0)
    P3 = torch.full((n, 3 * W), 3.0, device="cuda", dtype=torch.bfloat16)
    gw3, gb3 = [z(2 * d) for _ in range(3)], [z(1) for _ in range(3)]
    lib.level_grads_packed_rocm(*[t.data_ptr() for t in dh], *[t.data_ptr() for t in dg], k3.data_ptr(), v3.data_ptr(),
                                q3.data_ptr(), ld, kn2.data_ptr(), qn2.data_ptr(), *[t.data_ptr() for t in gates2],
                                P3.data_ptr(), 3 * W, 8, W + 8, 2 * W + 8, gw3[0].data_ptr(), gb3[0].data_ptr(),
                                gw3[1].data_ptr(), gb3[1].data_ptr(), gw3[2].data_ptr(), gb3[2].data_ptr(), bs, s, nh,
                                hd, 1e-8, 1)
    torch.cuda.synchronize()
    assert torch.equal(p3, proj), "the projections stay as they came"
    assert all(torch.equal(a, b) for a, b in zip(heads3, heads2)) and torch.equal(P3, P)
    assert all(torch.equal(a, b) for a, b in zip(gw3 + gb3, gw2 + gb2))
    for i, ref in enumerate((dk1, dv1, dq1)):
        c = 8 + i * d
        H, L, H2 = P[:, c:c + d], P[:, W + c:W + c + d], P[:, 2 * W + c:2 * W + c + d]
        assert torch.equal(H, H2)
        _close(f"packed gradient {i}", H.float() + L.float(), ref, 2e-5)
    assert torch.all(P[:, :8] == 3.0) and torch.all(P[:, 8 + 3 * d:W] == 3.0)
    for a, b in zip(gw2 + gb2, gw1 + gb1):
        _close("gate weight / bias gradient", a, b, 1e-4)


def test_combine_gate_with_bf16_attention_matches_the_fp32_kernels():
    g = torch.Generator(device="cuda").manual_seed(9)
    n, k = 4128, 4
    ys = [_rn(g, n) for _ in range(k)]
    attn = _rn(g, n).to(torch.bfloat16)
    af = attn.float()
    z = lambda: torch.zeros(n, device="cuda")
    yc, gate1, gated1, gate2, gated2 = z(), z(), z(), z(), z()
    ptrs = (ctypes.c_void_p * k)(*[y.data_ptr() for y in ys])
    lib.cms_combine_gate_rocm(ptrs, k, af.data_ptr(), yc.data_ptr(), gate1.data_ptr(), gated1.data_ptr(), n)
    d = 48
    pk = torch.zeros(n // d, 3 * d, device="cuda", dtype=torch.bfloat16)
    lib.cms_combine_gate_bf16_rocm(ptrs, k, attn.data_ptr(), gate2.data_ptr(), gated2.data_ptr(), pk.data_ptr(), d, n)
    _close("gate", gate2, gate1, 1e-6); _close("gated", gated2, gated1, 1e-6)
    h, l = _split(gated2.view(n // d, d))
    assert torch.equal(pk, torch.cat([h, h, l], 1))
    lib.cms_combine_gate_bf16_rocm(ptrs, k, attn.data_ptr(), gate2.data_ptr(), None, None, 0, n)
    dgt = _rn(g, n)
    da1, dy1, da2, dy2 = z(), z(), z(), z()
    D.call("cms_gate_backward_rocm", dgt, af, gate1, k, da1, dy1, n)
    lib.cms_gate_backward_bf16_rocm(dgt.data_ptr(), attn.data_ptr(), gate1.data_ptr(), k, da2.data_ptr(),
                                    dy2.data_ptr(), n)
    torch.cuda.synchronize()
    assert torch.equal(da1, da2)
    _close("d_y", dy2, dy1, 1e-6)


@pytest.mark.parametrize("levels,bs,nh,s,C,per_level", [(3, 2, 4, 150, 64, False), (2, 1, 8, 70, 16, True)])
def test_chunkwise_rule_on_token_major_rows_equals_the_head_major_entry_points(levels, bs, nh, s, C, per_level):
    """titans_chunkwise_{forward,backward}_bf16_tokens_rocm write y / read d_y in [levels, bs, s, nh*64] (d_y
    optionally shared by the levels); same kernels, other addresses: bit-equal to the head-major pair."""
    hd, B = 64, bs * nh
    nb, nc = levels * B, (s + C - 1) // C
    g = torch.Generator(device="cuda").manual_seed(77 + s)
    k, v, q = (_rn(g, nb, s, hd).to(torch.bfloat16) for _ in range(3))
    al, th, et = (torch.rand(nb, s, device="cuda", generator=g) * sc for sc in (0.1, 0.05, 0.9))
    m0, s0 = 0.1 * _rn(g, nb, hd * hd), 0.1 * _rn(g, nb, hd * hd)
    z = lambda *sh: torch.zeros(*sh, device="cuda")
    mc1, sc1, y1 = z(nb, nc + 1, hd * hd), z(nb, nc + 1, hd * hd), z(nb, s, hd)
    D.call("titans_chunkwise_forward_bf16_rocm", k, v, q, al, th, et, m0, s0, mc1, sc1, y1, s, hd, nb, C)
    mc2, sc2, y2 = z(nb, nc + 1, hd * hd), z(nb, nc + 1, hd * hd), z(levels, bs, s, nh * hd)
    D.call("titans_chunkwise_forward_bf16_tokens_rocm", k, v, q, al, th, et, m0, s0, mc2, sc2, y2, s, hd, nb, C, nh,
           levels)
    torch.cuda.synchronize()
    assert torch.equal(mc1, mc2) and torch.equal(sc1, sc2)
    assert torch.equal(y1.view(levels, bs, nh, s, hd).permute(0, 1, 3, 2, 4).reshape(levels, bs, s, nh * hd), y2)
    # backward
    dy_tok = _rn(g, levels if per_level else 1, bs, s, nh * hd)
    dy_heads = dy_tok.expand(levels, bs, s, nh * hd).reshape(levels, bs, s, nh, hd).permute(0, 1, 3, 2, 4)
    dy_heads = dy_heads.reshape(nb, s, hd).contiguous()
    outs = []
    for tokens in (False, True):
        gr = [z(nb, s, hd) for _ in range(3)] + [z(nb, s) for _ in range(3)] + [z(hd, hd), z(hd, hd)]
        if tokens:
            D.call("titans_chunkwise_backward_bf16_tokens_rocm", k, v, q, al, th, et, mc1, sc1, dy_tok, *gr, s, hd, nb,
                   C, nh, levels, int(per_level))
        else:
            D.call("titans_chunkwise_backward_bf16_rocm", k, v, q, al, th, et, mc1, sc1, dy_heads, *gr, s, hd, nb, C)
        outs.append(gr)
    torch.cuda.synchronize()
    for a, b in zip(*outs):
        assert torch.equal(a, b)
