"""GPU parity of the glue kernels and the AdamW / clipping pipeline through the
C ABI.  Elementwise fp32: relative 1e-5 (transcendentals 1e-5 abs); reductions
1e-4; bf16 conversion and layout moves are bit-exact."""
import ctypes

import numpy as np
import pytest
import torch

from nl_hecate_amd import dispatch as D
from nl_hecate_amd.ffi import lib
from oracle import pyoracle as orc
from tests.gpu_util import assert_close, dev, host, zeros

pytestmark = pytest.mark.gpu
R = np.random.default_rng(11)


def rnd(*shape):
    return R.standard_normal(shape).astype(np.float32)


@pytest.mark.parametrize("n", [1, 5, 256, 1000, 4099])
def test_elementwise_maps(n):
    a, b, c = rnd(n), rnd(n), rnd(n)
    out = zeros(n)
    D.call("sigmoid_cuda", dev(a), out, n)
    assert np.abs(host(out) - 1 / (1 + np.exp(-a.astype(np.float64)))).max() < 1e-6
    D.call("softplus_cuda", dev(a * 15), out, n)
    x = (a * 15).astype(np.float64)
    assert np.abs(host(out) - np.where(x > 20, x, np.log1p(np.exp(x)))).max() < 1e-5
    D.call("elemwise_mul_cuda", dev(a), dev(b), out, n)
    assert np.array_equal(host(out), a * b)
    da, db = zeros(n), zeros(n)
    D.call("gating_backward_cuda", dev(c), dev(a), dev(b), da, db, n)
    assert np.array_equal(host(da), c * b) and np.array_equal(host(db), c * a)
    g = (1 / (1 + np.exp(-a))).astype(np.float32)
    D.call("sigmoid_backward_cuda", dev(c), dev(g), out, n)
    assert_close("sigmoid_backward", host(out), c * g * (1 - g), 1e-6)
    y = dev(b)
    D.call("saxpy_cuda", 0.37, dev(a), y, n)
    assert_close("saxpy", host(y), b + np.float32(0.37) * a, 1e-6)
    z = dev(a)
    D.call("clamp_f32_cuda", z, n, -0.5, 0.25)
    assert np.array_equal(host(z), np.clip(a, -0.5, 0.25))
    dth = dev(c)
    D.call("theta_clamp_mask_cuda", z, dth, n, -0.5, 0.25)
    want = np.where((host(z) <= -0.5) | (host(z) >= 0.25), 0, c)
    assert np.array_equal(host(dth), want)
    # unaligned views take the scalar path
    if n > 8:
        big = dev(np.concatenate([[0.0], a]).astype(np.float32))
        o2 = zeros(n + 1)
        D.call("sigmoid_cuda", big[1:], o2[1:], n)
        assert np.abs(host(o2)[1:] - 1 / (1 + np.exp(-a.astype(np.float64)))).max() < 1e-6


def test_bf16_conversion_is_bit_exact():
    x = np.concatenate([rnd(5003) * 10 ** R.uniform(-5, 5, 5003).astype(np.float32),
                        [0.0, -0.0, 1.00390625, np.inf, -np.inf]]).astype(np.float32)
    n = x.size
    h = torch.zeros(n, dtype=torch.uint16, device="cuda")
    D.call("f32_to_bf16_cuda", dev(x), h, n)
    want = orc.f32_to_bf16(x)
    assert np.array_equal(h.cpu().numpy(), want)
    back = zeros(n)
    D.call("bf16_to_f32_cuda", h, back, n)
    assert np.array_equal(host(back), orc.bf16_to_f32(want))


@pytest.mark.parametrize("T,d", [(7, 8), (300, 64), (65, 512)])
def test_gate_compute_and_backward(T, d):
    k, v = rnd(T, d), rnd(T, d)
    w = (rnd(2 * d) / np.sqrt(2 * d)).astype(np.float32)
    bias = np.array([0.3], np.float32)
    for act in (0, 1):
        out = zeros(T)
        D.call("gate_compute_cuda", dev(k), dev(v), dev(w), dev(bias), out, T, d, act)
        assert_close(f"gate act={act}", host(out), orc.gate_compute(k, v, w, 0.3, act), 1e-5)
    alpha, theta, eta = (orc.gate_compute(k, v, w, 0.3, a) for a in (0, 1, 0))
    c = rnd(3, T)
    for has_theta, has_eta in ((1, 1), (1, 0), (0, 0)):
        o = {n: torch.full((2 * d,), 7.0, device="cuda") for n in ("wa", "wt", "we")}
        o.update({n: torch.full((1,), 7.0, device="cuda") for n in ("ba", "bt", "be")})
        D.call("gate_backward_cuda", dev(c[0]), dev(alpha), dev(c[1]), dev(theta), dev(c[2]), dev(eta),
               dev(k), dev(v), o["wa"], o["ba"], o["wt"], o["bt"], o["we"], o["be"], T, d, has_theta, has_eta)
        want = orc.gate_backward(c[0], alpha, c[1], theta, c[2], eta, k, v, has_theta, has_eta)
        assert_close("d_w_alpha", host(o["wa"]), want["d_w_alpha"])
        assert_close("d_b_alpha", host(o["ba"]), want["d_b_alpha"])
        if has_theta:
            assert_close("d_w_theta", host(o["wt"]), want["d_w_theta"])
            assert_close("d_b_theta", host(o["bt"]), want["d_b_theta"])
        else:
            assert np.all(host(o["wt"]) == 7.0), "ignored outputs stay untouched"
        if has_eta:
            assert_close("d_w_eta", host(o["we"]), want["d_w_eta"])


@pytest.mark.parametrize("n,d", [(5, 8), (100, 64), (33, 512), (3, 100)])
def test_l2_normalize_rows_and_backward(n, d):
    x = rnd(n, d)
    x[0] = 0  # zero row: the eps branch
    xd, norms = dev(x), zeros(n)
    D.call("l2_normalize_rows_f32_cuda", xd, norms, n, d, 1e-8)
    xn, no = orc.l2_normalize_rows(x)
    assert_close("x_norm", host(xd), xn, 1e-6)
    assert_close("norms", host(norms), no, 1e-6)
    g, din = rnd(n, d), zeros(n, d)
    D.call("l2_normalize_backward_f32_cuda", dev(g), dev(xn), dev(no), din, n, d, 1e-8)
    assert_close("d_in", host(din), orc.l2_normalize_backward(g, xn, no), 1e-5)


def test_head_layout_moves():
    bs, s, nh, hd = 3, 17, 4, 16
    x = rnd(bs, s, nh, hd)
    out = zeros(bs, nh, s, hd)
    D.call("transpose_heads_f32_cuda", dev(x), out, bs, s, nh, hd, 1)
    assert np.array_equal(host(out), x.transpose(0, 2, 1, 3))
    back = zeros(bs, s, nh, hd)
    D.call("transpose_heads_f32_cuda", out, back, bs, s, nh, hd, 0)
    assert np.array_equal(host(back), x)
    x3 = rnd(2, 5, 3, 3)  # hd not a multiple of 4: scalar path
    o3 = zeros(2, 3, 5, 3)
    D.call("transpose_heads_f32_cuda", dev(x3), o3, 2, 5, 3, 3, 1)
    assert np.array_equal(host(o3), x3.transpose(0, 2, 1, 3))
    gt = rnd(bs, s)
    bo = zeros(bs, nh, s)
    D.call("broadcast_heads_f32_cuda", dev(gt), bo, bs, s, nh)
    assert np.array_equal(host(bo), np.repeat(gt[:, None, :], nh, 1))
    y = rnd(bs, nh, s)
    so = zeros(bs, s)
    D.call("sum_heads_f32_cuda", dev(y), so, bs, s, nh)
    assert_close("sum_heads", host(so), y.sum(1), 1e-6)
    src = rnd(bs, 64)
    dst = zeros(bs, 5, 64)
    assert D.call("broadcast_fill_f32_cuda", dst, dev(src), 64, 5, bs) == 0
    assert np.array_equal(host(dst), np.repeat(src[:, None, :], 5, 1))


def test_m_norm_clamp_and_delta_norm():
    """core/tests/test_cuda_m_norm_clamp.rs:19: batched clamp == per-matrix loop."""
    B, d = 5, 32
    m = rnd(B, d, d) * np.linspace(0.01, 0.5, B, dtype=np.float32)[:, None, None]
    mx = 3.0
    md = dev(m)
    D.call("m_norm_clamp_batch_f32_cuda", md, d, B, mx)
    fn = np.sqrt((m.astype(np.float64) ** 2).sum((1, 2)))
    want = m * np.where(fn > mx, mx / fn, 1.0)[:, None, None].astype(np.float32)
    assert (fn > mx).any() and (fn < mx).any()
    assert_close("clamp", host(md), want, 1e-6)
    one = dev(m[-1])
    D.call("m_norm_clamp_f32_cuda", one, d, mx)
    assert np.array_equal(host(one), host(md)[-1])
    untouched = dev(m)
    D.call("m_norm_clamp_batch_f32_cuda", untouched, d, B, 0.0)
    D.call("m_norm_clamp_batch_f32_cuda", untouched, d, B, 1e30)
    assert np.array_equal(host(untouched), m)
    k, v, o = rnd(d), rnd(d), zeros(1)
    D.call("dgd_delta_norm_cuda", dev(m[2]), dev(k), dev(v), o, d)
    assert_close("delta_norm", host(o)[0], np.linalg.norm(m[2] @ k - v), 1e-5)


@pytest.mark.parametrize("n", [1, 255, 256, 1027, 262144])
def test_adamw_update_matches_oracle_and_torch(n):
    w, g = rnd(n), rnd(n)
    m, v = np.abs(rnd(n)) * 0.1, np.abs(rnd(n)) * 0.01
    lr, b1, b2, eps, wd, step = 3e-4, 0.9, 0.95, 1e-8, 0.1, 3
    bc1, bc2 = 1 / (1 - b1 ** step), 1 / (1 - b2 ** step)
    wd_, md_, vd_ = dev(w), dev(m), dev(v)
    rc = D.call("adamw_update_cuda", wd_, dev(g), md_, vd_, n, lr, b1, b2, eps, bc1, bc2, wd)
    assert rc == 0
    wo, mo, vo = w.copy(), m.copy(), v.copy()
    orc.adamw_step(wo, g, mo, vo, lr, b1, b2, eps, bc1, bc2, wd)
    assert_close("w", host(wd_), wo, 1e-6)
    assert_close("m", host(md_), mo, 1e-6)
    assert_close("v", host(vd_), vo, 1e-6)


def test_clip_pipeline_reference_symbols():
    n, mx = 10007, 1.0
    g = rnd(n)
    gd = dev(g)
    nblk = ctypes.c_int(0)
    part = zeros((n + 255) // 256)
    assert D.call("grad_norm_sq_cuda", gd, part, n, ctypes.byref(nblk)) == 0
    assert nblk.value == (n + 255) // 256
    pads = np.concatenate([g, np.zeros(nblk.value * 256 - n, np.float32)]).reshape(-1, 256)
    assert_close("partials", host(part), (pads.astype(np.float64) ** 2).sum(1), 1e-5)
    b = rnd(n)
    assert D.call("dot_product_partial_f32_cuda", gd, dev(b), part, n, ctypes.byref(nblk)) == 0
    padb = np.concatenate([b, np.zeros(nblk.value * 256 - n, np.float32)]).reshape(-1, 256)
    assert abs(host(part).sum() - (pads.astype(np.float64) * padb).sum()) < 1e-2
    D.call("grad_norm_sq_cuda", gd, part, n, ctypes.byref(nblk))
    norm, scale = zeros(1), zeros(1)
    assert D.call("reduce_partials_clip_cuda", part, nblk.value, mx, norm, scale) == 0
    on, os_ = orc.grad_norm_clip([g], mx)
    assert_close("norm", host(norm)[0], on, 1e-5)
    assert_close("scale", host(scale)[0], os_, 1e-5)
    assert D.call("grad_scale_conditional_cuda", gd, scale, n) == 0
    assert_close("clipped", host(gd), g * np.float32(os_), 1e-5)
    one = dev(np.array([1.0], np.float32))
    before = host(gd).copy()
    D.call("grad_scale_conditional_cuda", gd, one, n)
    assert np.array_equal(host(gd), before), "scale >= 1 leaves the gradient untouched"
    D.call("grad_scale_cuda", gd, 2.0, n)
    assert_close("scaled", host(gd), before * 2, 1e-6)


def test_multi_tensor_adamw_and_clip():
    # > 40 tensors: two launches; the empty tensor in the first batch of 40 must not shift the batch
    # boundary (the tensors after slot 40 would be updated twice)
    sizes = [262144, 1025, 1, 512, 262144, 77] + [300] * 10 + [0] + [300] * 34
    ws, gs, ms, vs = ([rnd(max(n, 1))[:n] for n in sizes] for _ in range(4))
    ms = [np.abs(m) * 0.1 for m in ms]
    vs = [np.abs(v) * 0.01 for v in vs]
    dws, dgs, dms, dvs = ([dev(a) for a in L] for L in (ws, gs, ms, vs))
    cnt = len(sizes)
    arr = lambda L: (ctypes.c_void_p * cnt)(*[t.data_ptr() for t in L])
    n_arr = (ctypes.c_int * cnt)(*sizes)
    # clip
    norm, scale = zeros(1), zeros(1)
    assert D.call("grad_norm_clip_multi_rocm", arr(dgs), n_arr, cnt, 1.0, norm, scale) == 0
    on, os_ = orc.grad_norm_clip(gs, 1.0)
    assert_close("norm", host(norm)[0], on, 1e-5)
    gs = [g * np.float32(os_) for g in gs]
    for a, b in zip(dgs, gs):
        if b.size:
            assert_close("clipped", host(a), b, 1e-5)
    # per-tensor bias corrections (levels with their own step counters)
    lr, b1, b2, eps, wd = 3e-4, 0.9, 0.95, 1e-8, 0.1
    steps = [1 + (i % 4) for i in range(cnt)]
    bc1 = (ctypes.c_float * cnt)(*[1 / (1 - b1 ** t) for t in steps])
    bc2 = (ctypes.c_float * cnt)(*[1 / (1 - b2 ** t) for t in steps])
    assert D.call("adamw_update_multi_rocm", arr(dws), arr(dgs), arr(dms), arr(dvs), n_arr, bc1, bc2, cnt,
                  lr, b1, b2, eps, wd) == 0
    for i in range(cnt):
        if sizes[i] == 0:
            continue
        gi = host(dgs[i])
        orc.adamw_step(ws[i], gi, ms[i], vs[i], lr, b1, b2, eps, bc1[i], bc2[i], wd)
        assert_close(f"w[{i}]", host(dws[i]), ws[i], 1e-6)
        assert_close(f"v[{i}]", host(dvs[i]), vs[i], 1e-6)


@pytest.mark.parametrize("bs,s,nh,hd,bf16", [(2, 37, 4, 16, False), (1, 100, 8, 64, True), (3, 5, 2, 24, True)])
def test_fused_level_glue_equals_the_separate_kernels(bs, s, nh, hd, bf16):
    """memory_inputs_fused_rocm / memory_grads_fused_rocm against the launches they replace
    (l2_normalize_rows, gate_compute, transpose_heads, broadcast_heads, sum_heads, l2_normalize_backward):
    same lane pattern in every sum, so equal to the last bit."""
    d, n, B = nh * hd, bs * s, bs * nh
    g = torch.Generator(device="cuda").manual_seed(5 + s)
    rn = lambda *sh: torch.randn(*sh, device="cuda", generator=g)
    k0, v, q0 = rn(n, d), rn(n, d), rn(n, d)
    k0[3 % n] = 0.0   # a zero row takes the norm < eps branch of the backward
    w = [0.1 * rn(2 * d) for _ in range(3)]
    bias = [rn(1) for _ in range(3)]
    # separate kernels
    k1, q1 = k0.clone(), q0.clone()
    kn1, qn1 = torch.zeros(n, device="cuda"), torch.zeros(n, device="cuda")
    D.call("l2_normalize_rows_f32_cuda", k1, kn1, n, d, 1e-8)
    D.call("l2_normalize_rows_f32_cuda", q1, qn1, n, d, 1e-8)
    gates1 = [torch.zeros(n, device="cuda") for _ in range(3)]
    for gt, ww, bb, act in zip(gates1, w, bias, (0, 1, 0)):
        D.call("gate_compute_cuda", k1, v, ww, bb, gt, n, d, act)
    heads1 = [torch.zeros(B, s, hd, device="cuda") for _ in range(3)]
    for src, dst in zip((k1, v, q1), heads1):
        D.call("transpose_heads_f32_cuda", src, dst, bs, s, nh, hd, 1)
    gh1 = [torch.zeros(B, s, device="cuda") for _ in range(3)]
    for src, dst in zip(gates1, gh1):
        D.call("broadcast_heads_f32_cuda", src, dst, bs, s, nh)
    # fused
    k2, q2 = k0.clone(), q0.clone()
    kn2, qn2 = torch.zeros(n, device="cuda"), torch.zeros(n, device="cuda")
    gates2 = [torch.zeros(n, device="cuda") for _ in range(3)]
    hdt = torch.bfloat16 if bf16 else torch.float32
    heads2 = [torch.zeros(B, s, hd, device="cuda", dtype=hdt) for _ in range(3)]
    gh2 = [torch.zeros(B, s, device="cuda") for _ in range(3)]
    D.call("memory_inputs_fused_rocm", k2, v, q2, w[0], bias[0], w[1], bias[1], w[2], bias[2], kn2, qn2, *gates2,
           *heads2, *gh2, bs, s, nh, hd, 1e-8, int(bf16))
    torch.cuda.synchronize()
    assert torch.equal(k1, k2) and torch.equal(q1, q2) and torch.equal(kn1, kn2) and torch.equal(qn1, qn2)
    for a, b in zip(gates1 + gh1, gates2 + gh2):
        assert torch.equal(a, b)
    for a, b in zip(heads1, heads2):
        assert torch.equal(a.to(hdt), b)
    # backward glue
    dh = [rn(B, s, hd) for _ in range(3)]
    dg = [rn(B, s) for _ in range(3)]
    tok1 = [torch.zeros(n, d, device="cuda") for _ in range(3)]
    for src, dst in zip(dh, tok1):
        D.call("transpose_heads_f32_cuda", src, dst, bs, s, nh, hd, 0)
    dgs1 = [torch.zeros(n, device="cuda") for _ in range(3)]
    for src, dst in zip(dg, dgs1):
        D.call("sum_heads_f32_cuda", src, dst, bs, s, nh)
    dk1, dq1 = torch.zeros(n, d, device="cuda"), torch.zeros(n, d, device="cuda")
    D.call("l2_normalize_backward_f32_cuda", tok1[0], k1, kn1, dk1, n, d, 1e-8)
    D.call("l2_normalize_backward_f32_cuda", tok1[2], q1, qn1, dq1, n, d, 1e-8)
    dk2, dv2, dq2 = (torch.zeros(n, d, device="cuda") for _ in range(3))
    dgs2 = [torch.zeros(n, device="cuda") for _ in range(3)]
    D.call("memory_grads_fused_rocm", *dh, *dg, k1, q1, kn1, qn1, dk2, dv2, dq2, *dgs2, bs, s, nh, hd, 1e-8)
    torch.cuda.synchronize()
    assert torch.equal(dk1, dk2) and torch.equal(tok1[1], dv2) and torch.equal(dq1, dq2)
    for a, b in zip(dgs1, dgs2):
        assert torch.equal(a, b)


def test_a_recorded_error_does_not_stop_later_valid_calls():
    """Record mode keeps the message of a failed call until nlh_clear_error; a valid call made in
    between must still do its work (entry points look only at errors of their own call)."""
    from nl_hecate_amd.ffi import lib
    n, d = 64, 32
    x = rnd(n, d)
    lib.nlh_set_error_mode(1)
    try:
        lib.nlh_clear_error()
        big = 4096   # layer_norm_backward_cuda refuses d > 2048
        D.call("layer_norm_backward_cuda", zeros(1, big), zeros(1, big), zeros(big), zeros(1), zeros(1),
               zeros(1, big), zeros(big), zeros(big), 1, big)
        assert b"layer_norm_backward_cuda" in lib.nlh_last_error()
        # uses the scratch arena and an error check of its own
        g, mean, rstd = np.ones(d, np.float32), zeros(n), zeros(n)
        out = zeros(n, d)
        D.call("layer_norm_forward_cuda", dev(x), dev(g), dev(np.zeros(d, np.float32)), out, mean, rstd, n, d, 1e-5)
        dx, dg, db = zeros(n, d), zeros(d), zeros(d)
        D.call("layer_norm_backward_cuda", dev(np.ones((n, d), np.float32)), dev(x), dev(g), mean, rstd, dx, dg, db, n, d)
        torch.cuda.synchronize()
        assert b"layer_norm_backward_cuda" in lib.nlh_last_error(), "message kept until cleared"
        assert_close("d_beta", host(db), np.full(d, n, np.float32), 1e-6)
        assert np.abs(host(dg)).max() > 0
    finally:
        lib.nlh_clear_error()
        lib.nlh_set_error_mode(0)
