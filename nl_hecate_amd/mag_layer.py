"""Host orchestration of one MAG layer (sliding-window attention gated by a CMS of
Titans memories) on the GPU library: the recipe of
core/src/gpu_forward.rs:864-1071 (forward), core/src/gpu_backward.rs:212-435
(backward) and, per level, gpu_memory_forward (gpu_forward.rs:1197-1540) /
gpu_memory_backward (gpu_backward.rs:459-640, 2047-2115).

Everything heavy is a call into the C ABI; the dense projections are plain
GEMMs (torch.matmul, i.e. rocBLAS/hipBLASLt: the reference's cublasSgemm call
sites).  Tensors are float32 CUDA tensors unless noted.  The gate -> k/v
gradient term is not propagated, as on the reference's GPU path.
"""
import ctypes
import math
from dataclasses import dataclass, field
from typing import List, Optional

import torch

from . import dispatch as D
from .cms import Conductor, ContextState, ErrorBuffer, FrequencyAwareAdamW, Pulse
from .ffi import lib

F32_MAX = 3.4028234663852886e38


@dataclass
class MemoryLevelParams:
    """Outer-loop parameters of one CMS level (core/src/model.rs MemoryLevelParams)."""
    w_k: torch.Tensor          # [d, d]
    w_v: torch.Tensor
    w_q: torch.Tensor
    w_alpha: torch.Tensor      # [2d]
    b_alpha: torch.Tensor      # [1]
    w_theta: torch.Tensor
    b_theta: torch.Tensor
    w_eta: torch.Tensor
    b_eta: torch.Tensor

    def tensors(self):
        return [self.w_k, self.w_v, self.w_q, self.w_alpha, self.b_alpha, self.w_theta, self.b_theta,
                self.w_eta, self.b_eta]


@dataclass
class MagParams:
    w_q: torch.Tensor          # attention branch, [d, d] each
    w_k: torch.Tensor
    w_v: torch.Tensor
    w_o: torch.Tensor
    levels: List[MemoryLevelParams] = field(default_factory=list)
    flat: Optional[torch.Tensor] = None    # gradients only: the one buffer all tensors are views of
    pack: Optional[torch.Tensor] = None    # gradients only: the projection matrices' rows, [3(1+k)d, d]

    def tensors(self):
        return [self.w_q, self.w_k, self.w_v, self.w_o] + [t for l in self.levels for t in l.tensors()]


def init_params(d, k, seed=0, device="cuda"):
    """Xavier-uniform matrices, small gate vectors, biases that start alpha low, theta small, eta high."""
    g = torch.Generator(device="cpu").manual_seed(seed)
    lim = math.sqrt(6.0 / (2 * d))
    mat = lambda: ((torch.rand(d, d, generator=g) * 2 - 1) * lim).to(device)
    vec = lambda: ((torch.rand(2 * d, generator=g) * 2 - 1) * 0.05).to(device)
    one = lambda x: torch.full((1,), x, dtype=torch.float32, device=device)
    p = MagParams(mat(), mat(), mat(), mat())
    for _ in range(k):
        p.levels.append(MemoryLevelParams(mat(), mat(), mat(), vec(), one(-2.0), vec(), one(-3.0), vec(), one(2.0)))
    return p


def _new(*shape, dtype=torch.float32):
    return torch.empty(*shape, dtype=dtype, device="cuda")


def _zeros(*shape, dtype=torch.float32):
    return torch.zeros(*shape, dtype=dtype, device="cuda")


def _wgrad(dy, x):
    """dy^T x for [n, d_out], [n, d_in] with n >> d: the contraction is cut into 16 slabs that run as one
    batched GEMM (16x the workgroups of the plain product, which leaves most of the chip idle) and are summed."""
    n = dy.shape[0]
    parts = 16
    if n % parts or n < 64 * parts:
        return dy.t() @ x
    return torch.bmm(dy.view(parts, n // parts, -1).transpose(1, 2), x.view(parts, n // parts, -1)).sum(0)


class MagLayer:
    """k Titans levels + SWA, MAG sigmoid gating.  `rule`: "exact" (checkpointed exact recurrence,
    fp32) or "chunkwise" (frozen-M0 chunkwise rule in matrix form, bf16 k/v/q)."""

    def __init__(self, d, heads, k, window, periods, rule="exact", chunk=64, params=None, seed=0,
                 precision="bf16x3"):
        """precision: how the dense projections run.  "bf16x3": operands split into hi + lo bf16 pairs, three
        products per GEMM (agrees with an fp32 GEMM to 5e-6).  "bf16": operands rounded once to bf16, fp32
        accumulation, and the level step (projections, normalisation, gates, head split, rule, and the whole
        backward down to d_x and the weight gradients) is ONE call into the library per direction
        (titans_levels_{forward,backward}_bf16_rocm): no GEMM is issued from this module.  Needs the chunkwise
        rule at head size 64, d in {256, 512}, chunk <= 64, window <= 512; other layers keep "bf16x3"."""
        assert d % heads == 0
        assert precision in ("bf16x3", "bf16")
        self.precision = precision
        self.d, self.nh, self.hd, self.k, self.window = d, heads, d // heads, k, window
        self.rule, self.chunk = rule, chunk
        self.p = params if params is not None else init_params(d, k, seed)
        self.conductor = Conductor(k, list(periods))
        # The 3 + 3k projections of x and the output projection share one packed weight tensor (the parameters become views of
        # it), so that one pass per step produces their bf16 operand copies (see _split_operands).
        tens = ([self.p.w_q, self.p.w_k, self.p.w_v] + [w for l in self.p.levels for w in (l.w_k, l.w_v, l.w_q)]
                + [self.p.w_o])
        self._pack = torch.cat([w.reshape(d, d) for w in tens], 0).contiguous()
        views = [self._pack[i * d:(i + 1) * d] for i in range(len(tens))]
        self.p.w_q, self.p.w_k, self.p.w_v, self.p.w_o = views[0], views[1], views[2], views[-1]
        for lv, l in enumerate(self.p.levels):
            l.w_k, l.w_v, l.w_q = views[3 + 3 * lv], views[4 + 3 * lv], views[5 + 3 * lv]
        self.split_gemm = True
        self.split_wgrad = True    # weight gradients of a projection group from the same packed operand
        self.stack_levels = True   # chunkwise rule: active levels run as one batch of chains
        self.fused_glue = True     # one pass per level for the glue either side of the rule
        # per-level context memory, one matrix per (batch element, head); created on first use
        self.m_state: List[Optional[torch.Tensor]] = [None] * k
        self.s_state: List[Optional[torch.Tensor]] = [None] * k

    # Projections of x as "3 x bf16" products: x = xh + xl, W = Wh + Wl (bf16 pairs, 16 mantissa bits),
    # x W^T ~ xh Wh^T + xh Wl^T + xl Wh^T as ONE bf16 GEMM with fp32 accumulation over the tripled
    # contraction [xh | xh | xl] . [Wh | Wl | Wh]^T.  Agrees with the fp32 GEMM to 5e-6 and runs about
    # three times faster on the bf16 matrix cores; the operand copies are made once per step.
    # The backward's d_x = sum_j g_j W_j over a set of projections j is the same construction with the
    # upstream gradients side by side: P = [H | L | H] (H, L the hi / lo parts of [g_0 | g_1 | ...])
    # against the rows [Wh ; Wh ; Wl] of those projections; and the weight gradients g_j^T x come from
    # the same P as H^T xh + L^T xh + H^T xl.
    @staticmethod
    def _pack_split(srcs):
        """[n, d] float tensors -> [n, 3*len*d] bf16: [hi(all) | lo(all) | hi(all)] (one pass)."""
        n, d = srcs[0].shape
        out = _new(n, 3 * len(srcs) * d, dtype=torch.bfloat16)
        ptrs = (ctypes.c_void_p * len(srcs))(*[t.data_ptr() for t in srcs])
        lib.split_pack_bf16_rocm(ptrs, len(srcs), out.data_ptr(), n, d)
        return out

    def _split_operands(self, x2, rows_stack=0):
        """The step's packed operands: xa [n, 3d] = (xh | xh | xl); wb [15d.., 3d] = (Wh | Wl | Wh) per
        weight row; wstack [3 * rows_stack, d] = (Wh ; Wh ; Wl) of the first rows_stack weight rows."""
        d, n, rows = self.d, x2.shape[0], self._pack.shape[0]
        xa = _new(n, 3 * d, dtype=torch.bfloat16)
        ptrs = (ctypes.c_void_p * 1)(x2.data_ptr())
        lib.split_pack_bf16_ld_rocm(ptrs, 1, d, xa.data_ptr(), n, d, 3 * d, 0, 2 * d, d)
        wb = _new(rows, 3 * d, dtype=torch.bfloat16)
        wstack = _new(max(3 * rows_stack, 1), d, dtype=torch.bfloat16)
        lib.split_pack_weights_rocm(self._pack.data_ptr(), rows, rows_stack, d, wb.data_ptr(), wstack.data_ptr())
        return dict(xa=xa, wb=wb, wstack=wstack, rows_stack=rows_stack)

    def _group_grads(self, ops, group, x2, grads3, weights3, wgrads3):
        """Projection group `group` (0: attention q, k, v; 1 + lv: level k, v, q): adds the three weight gradients
        grads3[s]^T x2 to wgrads3 and returns the input gradient sum_s grads3[s] @ weights3[s].
        With split operands both come from ONE packing of the three upstream gradients, P = [H | L | H] (9d wide):
        the input gradient as P . [Wh ; Wh ; Wl], and the weight gradients, the contraction now over tokens, by
        reading P as 3n rows (H_t, L_t, H_t) against the rows (xh_t, xh_t, xl_t) of the packed x:
        G^T x ~ H^T xh + L^T xh + H^T xl in one bf16 GEMM with fp32 accumulation, cut into up to 16 slabs along the
        contraction like _wgrad."""
        d = self.d
        n = x2.shape[0]
        if ops is None:
            for g, w in zip(grads3, wgrads3):
                w += _wgrad(g, x2)
            return grads3[0] @ weights3[0] + grads3[1] @ weights3[1] + grads3[2] @ weights3[2]
        P = self._pack_split(list(grads3))
        wg = ops["wb"][group * 3 * d:(group + 1) * 3 * d]
        stack = torch.cat([wg[:, :d], wg[:, :d], wg[:, d:2 * d]], 0)              # [9d, d]: Wh ; Wh ; Wl
        if not self.split_wgrad:
            for g, w in zip(grads3, wgrads3):
                w += _wgrad(g, x2)
            return torch.mm(P, stack, out_dtype=torch.float32)
        parts = next(p for p in (16, 8, 4, 2, 1) if (3 * n) % p == 0)
        rows = 3 * n // parts
        dw = torch.bmm(P.view(parts, rows, 3 * d).transpose(1, 2), ops["xa"].view(parts, rows, d),
                       out_dtype=torch.float32).sum(0)                            # [3 d_out, d_in]
        for i, w in enumerate(wgrads3):
            w += dw[i * d:(i + 1) * d]
        return torch.mm(P, stack, out_dtype=torch.float32)

    def _project(self, ops, x2, w, index, bf16_out=False):
        """x2 @ w^T for the packed projection number `index` (w is its fp32 view); bf16_out: rounded once, at
        the GEMM's store (what the attention kernels take)."""
        if ops is None:
            y = x2 @ w.t()
            return y.to(torch.bfloat16) if bf16_out else y
        d = self.d
        wt = ops["wb"][index * d:(index + 1) * d].t()
        return torch.mm(ops["xa"], wt) if bf16_out else torch.mm(ops["xa"], wt, out_dtype=torch.float32)

    def new_grads(self):
        """A MagParams of zeroed gradients whose tensors are views of ONE buffer (`flat`): the 3 + 3k projection
        matrices and w_o first, in the order of the packed weights, then the gate vectors."""
        d, k = self.d, self.k
        rows = self._pack.shape[0]
        sizes = [rows * d] + [2 * d, 4, 2 * d, 4, 2 * d, 4] * k
        flat = _zeros(sum(sizes))
        offs = [0]
        for z in sizes:
            offs.append(offs[-1] + z)
        gp = flat[:rows * d].view(rows, d)
        mats = [gp[i * d:(i + 1) * d] for i in range(rows // d)]
        levels = []
        for lv in range(k):
            o = offs[1 + 6 * lv:1 + 6 * lv + 6]
            gate = [flat[o[0]:o[0] + 2 * d], flat[o[1]:o[1] + 1], flat[o[2]:o[2] + 2 * d], flat[o[3]:o[3] + 1],
                    flat[o[4]:o[4] + 2 * d], flat[o[5]:o[5] + 1]]
            levels.append(MemoryLevelParams(mats[3 + 3 * lv], mats[4 + 3 * lv], mats[5 + 3 * lv], *gate))
        g = MagParams(mats[0], mats[1], mats[2], mats[-1], levels=levels)
        g.flat, g.pack = flat, gp
        return g

    def ensure_state(self, bs):
        """Creates the (zero) context memories of every level for batch size bs if they do not exist.
        The levels' memories are slices of one tensor, so that a prefix of levels is one batch of chains."""
        if self.m_state[0] is None:
            self._m_all = _zeros(self.k, bs * self.nh, self.hd * self.hd)
            self._s_all = _zeros(self.k, bs * self.nh, self.hd * self.hd)
            for lv in range(self.k):
                self.m_state[lv], self.s_state[lv] = self._m_all[lv], self._s_all[lv]

    def context_state(self, bs):
        """The layer's persistent memories as a ContextState (conductor.rs:156-221): reset() at a document
        boundary zeroes every level's M and S in place (addresses stay fixed for captured graphs)."""
        self.ensure_state(bs)
        return ContextState(self.m_state, self.s_state)

    # ── one level ────────────────────────────────────────────────────────────
    def _level_forward(self, lv, x2, bs, s, active, ops=None):
        """gpu_memory_forward: projections, L2 norm, gates, head split, recurrence."""
        d, nh, hd = self.d, self.nh, self.hd
        lp = self.p.levels[lv]
        B = bs * nh
        n = bs * s
        self.ensure_state(bs)
        y = _new(bs, s, d)
        if not active:
            # frozen level (gpu_memory_read_only, gpu_forward.rs:2906-2950): y = M_h q with the raw
            # projection q and the context memory of the first batch slot, shared by the batch
            q_raw = self._project(ops, x2, lp.w_q, 5 + 3 * lv)
            m_shared = self.m_state[lv][:nh].contiguous()
            D.call("memory_read_only_f32_rocm", q_raw, m_shared, y, n, nh, hd)
            return y, dict(active=False, m_shared=m_shared)
        kh, vh, qh = _new(B, s, hd), _new(B, s, hd), _new(B, s, hd)
        ah, th, eh = _new(B, s), _new(B, s), _new(B, s)
        c = self._level_inputs(lv, x2, bs, s, ops, (kh, vh, qh, ah, th, eh))
        yh = _new(B, s, hd)
        C = self.chunk
        if self.rule == "exact":
            n_ck = 1 + sum(1 for t in range(s) if (t + 1) % C == 0 or t + 1 == s)
            mc, sc = _new(B, n_ck, hd * hd), _new(B, n_ck, hd * hd)
            D.call("titans_forward_ckpt_batched_f32_rocm", kh, vh, qh, ah, th, eh, self.m_state[lv],
                   self.s_state[lv], mc, sc, yh, s, hd, B, C, 0.0, F32_MAX)
        else:
            nc = (s + C - 1) // C
            mc, sc = _new(B, nc + 1, hd * hd), _new(B, nc + 1, hd * hd)
            kh, vh, qh = kh.to(torch.bfloat16), vh.to(torch.bfloat16), qh.to(torch.bfloat16)
            D.call("titans_chunkwise_forward_bf16_rocm", kh, vh, qh, ah, th, eh, self.m_state[lv],
                   self.s_state[lv], mc, sc, yh, s, hd, B, C)
        # context memory carries over to the next step (copy_final_m_batch, gpu_forward.rs:2824)
        # (in place: the buffers keep their addresses, so a captured step can be replayed)
        self.m_state[lv].copy_(mc[:, -1])
        self.s_state[lv].copy_(sc[:, -1])
        D.call("transpose_heads_f32_cuda", yh, y, bs, s, nh, hd, 0)
        c.update(kh=kh, vh=vh, qh=qh, ah=ah, th=th, eh=eh, mc=mc, sc=sc)
        return y, c

    def _level_inputs(self, lv, x2, bs, s, ops, dst):
        """Projections, L2 norm, gates and head split of level lv; the head-major k, v, q [B, s, hd] and
        gates [B, s] go to the six tensors of dst.  Returns the level's cache of token-major tensors."""
        d, nh, hd = self.d, self.nh, self.hd
        lp = self.p.levels[lv]
        n = bs * s
        k_mem = self._project(ops, x2, lp.w_k, 3 + 3 * lv)
        v_mem = self._project(ops, x2, lp.w_v, 4 + 3 * lv)
        q_mem = self._project(ops, x2, lp.w_q, 5 + 3 * lv)
        k_norms, q_norms = _new(n), _new(n)
        alpha, theta, eta = _new(n), _new(n), _new(n)
        if self.fused_glue:   # the eleven launches below as one pass over the tokens
            D.call("memory_inputs_fused_rocm", k_mem, v_mem, q_mem, lp.w_alpha, lp.b_alpha, lp.w_theta, lp.b_theta,
                   lp.w_eta, lp.b_eta, k_norms, q_norms, alpha, theta, eta, *dst, bs, s, nh, hd, 1e-8,
                   int(dst[0].dtype == torch.bfloat16))
        else:
            D.call("l2_normalize_rows_f32_cuda", k_mem, k_norms, n, d, 1e-8)
            D.call("l2_normalize_rows_f32_cuda", q_mem, q_norms, n, d, 1e-8)
            D.call("gate_compute_cuda", k_mem, v_mem, lp.w_alpha, lp.b_alpha, alpha, n, d, 0)
            D.call("gate_compute_cuda", k_mem, v_mem, lp.w_theta, lp.b_theta, theta, n, d, 1)
            D.call("gate_compute_cuda", k_mem, v_mem, lp.w_eta, lp.b_eta, eta, n, d, 0)
            for src, dst_t in zip((k_mem, v_mem, q_mem), dst[:3]):
                D.call("transpose_heads_f32_cuda", src, dst_t, bs, s, nh, hd, 1)
            for src, dst_t in zip((alpha, theta, eta), dst[3:]):
                D.call("broadcast_heads_f32_cuda", src, dst_t, bs, s, nh)
        return dict(k_mem=k_mem, v_mem=v_mem, q_mem=q_mem, k_norms=k_norms, q_norms=q_norms, active=True, ops=ops,
                    alpha=alpha, theta=theta, eta=eta)

    # The active levels of the chunkwise rule as ONE batch of chains.  The levels are independent
    # memories over the same tokens, and the chain kernels want at least 128 chains to fill the chip, so
    # the head-major tensors of the active levels (always a prefix: the periods are nested) are stacked
    # along the chain dimension and the rule runs once, forward and backward.
    def _levels_forward_stacked(self, na, x2, bs, s, ops):
        d, nh, hd, C = self.d, self.nh, self.hd, self.chunk
        B, n = bs * nh, bs * s
        self.ensure_state(bs)
        # k, v, q of every active level from one GEMM: [n, 3 na d], level lv at columns 3 lv d ..
        ld = 3 * na * d
        proj = torch.mm(ops["xa"], ops["wb"][3 * d:3 * d + ld].t(), out_dtype=torch.float32)
        kh, vh, qh = (_new(na * B, s, hd, dtype=torch.bfloat16) for _ in range(3))
        ah, th, eh = _new(na * B, s), _new(na * B, s), _new(na * B, s)
        caches = []
        for lv in range(na):
            lp = self.p.levels[lv]
            sl = slice(lv * B, (lv + 1) * B)
            k_mem, v_mem, q_mem = (proj[:, (3 * lv + i) * d:(3 * lv + i + 1) * d] for i in range(3))
            k_norms, q_norms, alpha, theta, eta = (_new(n) for _ in range(5))
            lib.level_inputs_fused_rocm(
                k_mem.data_ptr(), v_mem.data_ptr(), q_mem.data_ptr(), ld, lp.w_alpha.data_ptr(), lp.b_alpha.data_ptr(),
                lp.w_theta.data_ptr(), lp.b_theta.data_ptr(), lp.w_eta.data_ptr(), lp.b_eta.data_ptr(),
                k_norms.data_ptr(), q_norms.data_ptr(), alpha.data_ptr(), theta.data_ptr(), eta.data_ptr(),
                kh[sl].data_ptr(), vh[sl].data_ptr(), qh[sl].data_ptr(), ah[sl].data_ptr(), th[sl].data_ptr(),
                eh[sl].data_ptr(), bs, s, nh, hd, 1e-8, 1, 0)
            caches.append(dict(k_mem=k_mem, v_mem=v_mem, q_mem=q_mem, ld=ld, k_norms=k_norms, q_norms=q_norms,
                               active=True, ops=ops, alpha=alpha, theta=theta, eta=eta))
        nc = (s + C - 1) // C
        mc, sc = _new(na * B, nc + 1, hd * hd), _new(na * B, nc + 1, hd * hd)
        m0, s0 = self._m_all[:na].view(na * B, hd * hd), self._s_all[:na].view(na * B, hd * hd)
        y_all = _new(na, bs, s, d)   # the rule writes every level's output token-major: no head transposes
        D.call("titans_chunkwise_forward_bf16_tokens_rocm", kh, vh, qh, ah, th, eh, m0, s0, mc, sc, y_all, s, hd,
               na * B, C, nh, na)
        m0.copy_(mc[:, -1])
        s0.copy_(sc[:, -1])
        ys = [y_all[lv] for lv in range(na)]
        return ys, caches, dict(na=na, kh=kh, vh=vh, qh=qh, ah=ah, th=th, eh=eh, mc=mc, sc=sc, proj=proj)

    def _levels_backward_stacked(self, st, caches, d_y, bs, s, grads, P, rows_stack):
        """Rule backward of the stacked levels; every level's projection-input gradients go straight into its
        column slab of the packed operand P [n, 2 rows_stack] (see backward), its gate gradients into grads."""
        d, nh, hd, C, na = self.d, self.nh, self.hd, self.chunk, st["na"]
        B = bs * nh
        dkh, dvh, dqh = _new(na * B, s, hd), _new(na * B, s, hd), _new(na * B, s, hd)
        dah, dth, deh = _new(na * B, s), _new(na * B, s), _new(na * B, s)
        dm, ds = _zeros(hd, hd), _zeros(hd, hd)
        # every level reads the one token-major upstream gradient in place
        D.call("titans_chunkwise_backward_bf16_tokens_rocm", st["kh"], st["vh"], st["qh"], st["ah"], st["th"],
               st["eh"], st["mc"], st["sc"], d_y, dkh, dvh, dqh, dah, dth, deh, dm, ds, s, hd, na * B, C, nh, na, 0)
        for lv in range(na):
            c, g = caches[lv], grads.levels[lv]
            sl = slice(lv * B, (lv + 1) * B)
            col = (3 + 3 * lv) * d
            lib.level_grads_packed_rocm(
                dkh[sl].data_ptr(), dvh[sl].data_ptr(), dqh[sl].data_ptr(), dah[sl].data_ptr(), dth[sl].data_ptr(),
                deh[sl].data_ptr(), c["k_mem"].data_ptr(), c["v_mem"].data_ptr(), c["q_mem"].data_ptr(), c["ld"],
                c["k_norms"].data_ptr(), c["q_norms"].data_ptr(), c["alpha"].data_ptr(), c["theta"].data_ptr(),
                c["eta"].data_ptr(), P.data_ptr(), 2 * rows_stack, col, rows_stack + col, -1,
                g.w_alpha.data_ptr(), g.b_alpha.data_ptr(), g.w_theta.data_ptr(), g.b_theta.data_ptr(),
                g.w_eta.data_ptr(), g.b_eta.data_ptr(), bs, s, nh, hd, 1e-8, 1)

    def _level_backward(self, lv, c, x2, d_y, bs, s, grads):
        """gpu_memory_backward + accumulate_projection_grads; returns the level's d_x [bs*s, d]."""
        d, nh, hd = self.d, self.nh, self.hd
        lp, g = self.p.levels[lv], grads.levels[lv]
        B, n = bs * nh, bs * s
        if not c["active"]:
            # read-only level: y = M_h q, only the q path carries gradient
            dq = _new(n, d)
            D.call("memory_read_only_backward_f32_rocm", d_y, c["m_shared"], dq, n, nh, hd)
            g.w_q += _wgrad(dq, x2)
            return dq @ lp.w_q
        dyh = _new(B, s, hd)
        D.call("transpose_heads_f32_cuda", d_y, dyh, bs, s, nh, hd, 1)
        dkh, dvh, dqh = _new(B, s, hd), _new(B, s, hd), _new(B, s, hd)
        dah, dth, deh = _new(B, s), _new(B, s), _new(B, s)
        dm, ds = _zeros(hd, hd), _zeros(hd, hd)
        C = self.chunk
        if self.rule == "exact":
            D.call("titans_backward_ckpt_f32_rocm", c["kh"], c["vh"], c["qh"], c["ah"], c["th"], c["eh"], c["mc"],
                   c["sc"], dyh, dkh, dvh, dqh, dah, dth, deh, dm, ds, s, hd, B, C, 0.0, F32_MAX)
        else:
            D.call("titans_chunkwise_backward_bf16_rocm", c["kh"], c["vh"], c["qh"], c["ah"], c["th"], c["eh"],
                   c["mc"], c["sc"], dyh, dkh, dvh, dqh, dah, dth, deh, dm, ds, s, hd, B, C)
        return self._level_param_grads(lv, c, x2, (dkh, dvh, dqh, dah, dth, deh), bs, s, grads)

    def _level_param_grads(self, lv, c, x2, head_grads, bs, s, grads):
        """From the rule's head-major gradients (d_k, d_v, d_q [B, s, hd], d_alpha, d_theta, d_eta [B, s]) of
        level lv: gate and projection weight gradients (accumulated into grads) and the level's d_x."""
        d, nh, hd = self.d, self.nh, self.hd
        lp, g = self.p.levels[lv], grads.levels[lv]
        n = bs * s
        dkh, dvh, dqh, dah, dth, deh = head_grads
        d_alpha, d_theta, d_eta = _new(n), _new(n), _new(n)
        dk_in, dv, dq_in = _new(n, d), _new(n, d), _new(n, d)
        if self.fused_glue:   # head sums, head merge and both normalisation backwards in one pass
            D.call("memory_grads_fused_rocm", dkh, dvh, dqh, dah, dth, deh, c["k_mem"], c["q_mem"], c["k_norms"],
                   c["q_norms"], dk_in, dv, dq_in, d_alpha, d_theta, d_eta, bs, s, nh, hd, 1e-8)
        else:
            for src, dst in ((dah, d_alpha), (dth, d_theta), (deh, d_eta)):
                D.call("sum_heads_f32_cuda", src, dst, bs, s, nh)
            dk, dq = _new(n, d), _new(n, d)
            for src, dst in ((dkh, dk), (dvh, dv), (dqh, dq)):
                D.call("transpose_heads_f32_cuda", src, dst, bs, s, nh, hd, 0)
            D.call("l2_normalize_backward_f32_cuda", dk, c["k_mem"], c["k_norms"], dk_in, n, d, 1e-8)
            D.call("l2_normalize_backward_f32_cuda", dq, c["q_mem"], c["q_norms"], dq_in, n, d, 1e-8)
        # gate projections (d_w, d_b) from the cached gate outputs
        D.call("gate_backward_cuda", d_alpha, c["alpha"], d_theta, c["theta"], d_eta, c["eta"], c["k_mem"],
               c["v_mem"], g.w_alpha, g.b_alpha, g.w_theta, g.b_theta, g.w_eta, g.b_eta, n, d, 1, 1)
        return self._group_grads(c.get("ops"), 1 + lv, x2, (dk_in, dv, dq_in), (lp.w_k, lp.w_v, lp.w_q),
                                 (g.w_k, g.w_v, g.w_q))

    # ── the layer ────────────────────────────────────────────────────────────
    def forward(self, x):
        """x [bs, s, d] -> (out [bs, s, d], cache).  Does not advance the Conductor."""
        bs, s, d = x.shape
        p, nh, hd = self.p, self.nh, self.hd
        x2 = x.reshape(bs * s, d)
        self.conductor.set_seq_len(s)
        pulse = self.conductor.pulse()
        active = [bool(a) for a in pulse.active_levels]
        na = active.index(False) if False in active else self.k
        if self._single_bf16_ok(active, na):
            return self._forward_bf16(x, pulse, active, na)
        stacked = (self.rule == "chunkwise" and self.stack_levels and self.split_gemm and self.fused_glue
                   and na >= 2 and not any(active[na:]) and hd == 64 and self.chunk <= 64 and d <= 1024)
        ops = self._split_operands(x2, 3 * d * (1 + na) if stacked else 0) if self.split_gemm else None
        q = self._project(ops, x2, p.w_q, 0, bf16_out=True).view(bs, s, d)
        k = self._project(ops, x2, p.w_k, 1, bf16_out=True).view(bs, s, d)
        v = self._project(ops, x2, p.w_v, 2, bf16_out=True).view(bs, s, d)
        attn = _new(bs, s, d, dtype=torch.bfloat16)
        if hd == 64 and self.window <= 512:
            # per-query softmax statistics instead of the [bs, nh, s, window] weight tensor
            aw = _new(bs, nh, s, 2)
            D.call("swa_forward_lse_bf16_rocm", q, k, v, attn, aw, s, nh, hd, self.window, bs)
        else:
            aw = _new(bs, nh, s, self.window, dtype=torch.bfloat16)
            D.call("swa_forward_f32_cuda", q, k, v, attn, aw, s, nh, hd, self.window, bs, 0)
        ys, caches, stack = [], [], None
        if stacked:
            ys, caches, stack = self._levels_forward_stacked(na, x2, bs, s, ops)
        for lv in range(len(ys), self.k):
            y, c = self._level_forward(lv, x2, bs, s, active[lv], ops)
            ys.append(y)
            caches.append(c)
        gate = _new(bs, s, d)
        ptrs = (ctypes.c_void_p * self.k)(*[y.data_ptr() for y in ys])
        if d % 4 == 0 and ops is not None:
            # the attention output is consumed as bf16; gated leaves as the packed operand of the output
            # projection (hi | hi | lo), which is the last d rows of the packed weights
            gated = _new(bs * s, 3 * d, dtype=torch.bfloat16)
            lib.cms_combine_gate_bf16_rocm(ptrs, self.k, attn.data_ptr(), gate.data_ptr(), None, gated.data_ptr(), d,
                                           bs * s * d)
            out = torch.mm(gated, ops["wb"][-d:].t(), out_dtype=torch.float32).view(bs, s, d)
        else:
            gated = _new(bs, s, d)
            lib.cms_combine_gate_rocm(ptrs, self.k, attn.to(torch.float32).data_ptr(), None, gate.data_ptr(),
                                      gated.data_ptr(), bs * s * d)
            out = (gated.view(bs * s, d) @ p.w_o.t()).view(bs, s, d)
        cache = dict(x=x, q=q, k=k, v=v, aw=aw, attn=attn, gate=gate, gated=gated, levels=caches, pulse=pulse,
                     ys=ys, ops=ops, stack=stack)
        return out, cache

    # ── the layer with single-bf16 projections: every heavy step is one call into the library ─────────────
    def _single_bf16_ok(self, active, na):
        return (self.precision == "bf16" and self.rule == "chunkwise" and self.hd == 64 and self.d in (256, 512)
                and self.chunk <= 64 and self.window <= 512 and not any(active[na:]))

    def _gate_ptrs(self, levels):
        return (ctypes.c_void_p * (6 * len(levels)))(*[t.data_ptr() for l in levels for t in
                                                       (l.w_alpha, l.b_alpha, l.w_theta, l.b_theta, l.w_eta, l.b_eta)])

    def _forward_bf16(self, x, pulse, active, na):
        bs, s, d = x.shape
        nh, hd, C, k = self.nh, self.hd, self.chunk, self.k
        B, n = bs * nh, bs * s
        self.ensure_state(bs)
        bf = torch.bfloat16
        q, kk, v = (_new(bs, s, d, dtype=bf) for _ in range(3))
        xb = _new(n, d, dtype=bf)
        kh, vh, qh = (_new(max(na, 1) * B, s, hd, dtype=bf) for _ in range(3))
        ah, th, eh = (_new(max(na, 1) * B, s) for _ in range(3))
        k_norms, q_norms, alpha, theta, eta = (_new(max(na, 1), n) for _ in range(5))
        nc = (s + C - 1) // C
        mc, sc = _new(max(na, 1) * B, nc + 1, hd * hd), _new(max(na, 1) * B, nc + 1, hd * hd)
        y_all = _new(max(na, 1), bs, s, d)
        extra = (ctypes.c_void_p * 3)(q.data_ptr(), kk.data_ptr(), v.data_ptr())
        lib.titans_levels_forward_bf16_rocm(
            x.data_ptr(), self._pack.data_ptr(), 3, extra, self._pack[3 * d:].data_ptr(), self._gate_ptrs(self.p.levels[:na]),
            self._m_all.data_ptr(), self._s_all.data_ptr(), xb.data_ptr(), kh.data_ptr(), vh.data_ptr(), qh.data_ptr(),
            ah.data_ptr(), th.data_ptr(), eh.data_ptr(), k_norms.data_ptr(), q_norms.data_ptr(), alpha.data_ptr(),
            theta.data_ptr(), eta.data_ptr(), mc.data_ptr(), sc.data_ptr(), y_all.data_ptr(), bs, s, nh, hd, na, C, 1e-8)
        attn = _new(bs, s, d, dtype=bf)
        aw = _new(bs, nh, s, 2)
        D.call("swa_forward_lse_bf16_rocm", q, kk, v, attn, aw, s, nh, hd, self.window, bs)
        ys, frozen = [y_all[lv] for lv in range(na)], []
        for lv in range(na, k):
            # frozen level (gpu_memory_read_only, gpu_forward.rs:2906-2950): y = M_h q with the raw projection q
            q_raw, y = _new(n, d), _new(bs, s, d)
            lib.linear_forward_bf16_rocm(xb.data_ptr(), self.p.levels[lv].w_q.data_ptr(), q_raw.data_ptr(), n, d, d)
            m_shared = self.m_state[lv][:nh].contiguous()
            D.call("memory_read_only_f32_rocm", q_raw, m_shared, y, n, nh, hd)
            ys.append(y)
            frozen.append(m_shared)
        gate, gated = _new(bs, s, d), _new(n, d, dtype=bf)
        ptrs = (ctypes.c_void_p * k)(*[y.data_ptr() for y in ys])
        lib.cms_combine_gate_bf16x1_rocm(ptrs, k, attn.data_ptr(), gate.data_ptr(), gated.data_ptr(), n * d)
        out = _new(bs, s, d)
        lib.linear_forward_bf16_rocm(gated.data_ptr(), self.p.w_o.data_ptr(), out.data_ptr(), n, d, d)
        cache = dict(bf16=True, x=x, xb=xb, q=q, k=kk, v=v, aw=aw, attn=attn, gate=gate, gated=gated, pulse=pulse, ys=ys, na=na,
                     kh=kh, vh=vh, qh=qh, ah=ah, th=th, eh=eh, k_norms=k_norms, q_norms=q_norms, alpha=alpha, theta=theta,
                     eta=eta, mc=mc, sc=sc, frozen=frozen)
        return out, cache

    def _backward_bf16(self, c, d_out, grads):
        x = c["x"]
        bs, s, d = x.shape
        nh, hd, k, na = self.nh, self.hd, self.k, c["na"]
        n = bs * s
        d_gated = _new(n, d)
        lib.linear_backward_bf16_rocm(d_out.data_ptr(), c["gated"].data_ptr(), self.p.w_o.data_ptr(), d_gated.data_ptr(),
                                      grads.w_o.data_ptr(), n, d, d)
        d_attn, d_ycomb = _new(bs, s, d), _new(bs, s, d)
        lib.cms_gate_backward_bf16_rocm(d_gated.data_ptr(), c["attn"].data_ptr(), c["gate"].data_ptr(), k,
                                        d_attn.data_ptr(), d_ycomb.data_ptr(), n * d)
        # the attention gradients go straight into their columns of the level step's bf16 GEMM operand
        ld = ctypes.c_longlong(0)
        g_op = lib.level_grad_operand_rocm(bs, s, nh, hd, na, 3, ctypes.byref(ld))
        if not g_op:
            raise RuntimeError("level_grad_operand_rocm failed")
        lib.swa_backward_lse_bf16_cols_rocm(c["q"].data_ptr(), c["k"].data_ptr(), c["v"].data_ptr(), c["aw"].data_ptr(),
                                            d_attn.data_ptr(), g_op, g_op + 2 * d, g_op + 4 * d, ld.value, s, nh, hd,
                                            self.window, bs)
        d_x = _new(bs, s, d)
        seeds = _zeros(2, hd, hd)
        d_extra = (ctypes.c_void_p * 3)(None, None, None)
        gl = grads.levels[:na]
        gate_out = (ctypes.c_void_p * (6 * na))(*[t.data_ptr() for g in gl for t in
                                                  (g.w_alpha, g.b_alpha, g.w_theta, g.b_theta, g.w_eta, g.b_eta)])
        lib.titans_levels_backward_bf16_rocm(
            c["xb"].data_ptr(), self._pack.data_ptr(), 3, d_extra, self._pack[3 * d:].data_ptr(), c["kh"].data_ptr(),
            c["vh"].data_ptr(), c["qh"].data_ptr(), c["ah"].data_ptr(), c["th"].data_ptr(), c["eh"].data_ptr(),
            c["k_norms"].data_ptr(), c["q_norms"].data_ptr(), c["alpha"].data_ptr(), c["theta"].data_ptr(),
            c["eta"].data_ptr(), c["mc"].data_ptr(), c["sc"].data_ptr(), d_ycomb.data_ptr(), d_x.data_ptr(),
            grads.pack.data_ptr(), grads.pack[3 * d:].data_ptr(), gate_out, seeds[0].data_ptr(), seeds[1].data_ptr(),
            bs, s, nh, hd, na, self.chunk, 1e-8)
        for i, lv in enumerate(range(na, k)):
            # read-only level: only the q path carries gradient
            dq_l, dx_l = _new(n, d), _new(n, d)
            D.call("memory_read_only_backward_f32_rocm", d_ycomb, c["frozen"][i], dq_l, n, nh, hd)
            lib.linear_backward_bf16_rocm(dq_l.data_ptr(), c["xb"].data_ptr(), self.p.levels[lv].w_q.data_ptr(),
                                          dx_l.data_ptr(), grads.levels[lv].w_q.data_ptr(), n, d, d)
            d_x.view(n, d).add_(dx_l)
        return d_x

    # ── decode: one token with a KV cache ────────────────────────────────────
    def decode_reset(self, max_len):
        """A new, empty bf16 KV cache of the attention branch (room for max_len tokens)."""
        from .serving import GpuKVCache   # serving imports this module
        self._kv = GpuKVCache(max_len, self.d, 1)

    def decode_step(self, x_t, pulse=None):
        """One token of one sequence, x_t [d] -> out [d]: the layer part of gpu_single_token_forward
        (core/src/gpu_forward.rs:3377-3500): q/k/v projections, K and V appended to the bf16 cache, attention of
        the newest token over the cache (swa_single_token_cuda), every level with seq_len = 1 (active: the full
        rule on the carried context memory, frozen: read-only), combine, sigmoid gate, W_o.  The caller advances
        the Conductor; `pulse` defaults to its current one."""
        d, nh, hd, p = self.d, self.nh, self.hd, self.p
        kv = self._kv
        assert kv.len < kv.max_len, "KV cache full"
        if pulse is None:
            self.conductor.set_seq_len(1)
            pulse = self.conductor.pulse()
        x2 = x_t.reshape(1, d)
        q = (x2 @ p.w_q.t()).to(torch.bfloat16)
        kv.append_f32(x2 @ p.w_k.t(), x2 @ p.w_v.t(), 1)
        attn_bf = _new(1, d, dtype=torch.bfloat16)
        D.call("swa_single_token_cuda", q, kv.k_cache_bf16, kv.v_cache_bf16, attn_bf, kv.len, nh, hd, self.window, 0)
        ys = [self._level_forward(lv, x2, 1, 1, bool(pulse.active_levels[lv]))[0] for lv in range(self.k)]
        y_comb, gate, gated = _new(1, 1, d), _new(1, 1, d), _new(1, 1, d)
        ptrs = (ctypes.c_void_p * self.k)(*[y.data_ptr() for y in ys])
        attn = attn_bf.to(torch.float32)
        lib.cms_combine_gate_rocm(ptrs, self.k, attn.data_ptr(), y_comb.data_ptr(), gate.data_ptr(),
                                  gated.data_ptr(), d)
        return (gated.view(1, d) @ p.w_o.t()).view(d)

    def backward(self, cache, d_out, grads=None):
        """-> (d_x [bs, s, d], grads: MagParams of gradients).  `grads`: a MagParams from new_grads() to write
        into (zeroed here first); a new one is made otherwise."""
        x = cache["x"]
        bs, s, d = x.shape
        p, nh, hd = self.p, self.nh, self.hd
        n = bs * s
        x2 = x.reshape(n, d)
        do2 = d_out.reshape(n, d)
        if grads is None:
            grads = self.new_grads()
        else:
            grads.flat.zero_()
        if cache.get("bf16"):
            return self._backward_bf16(cache, d_out, grads), grads
        ops, stack = cache["ops"], cache["stack"]
        if cache["gated"].dtype == torch.bfloat16:
            # d_gated = d_out W_o and d_W_o = d_out^T gated from one packing (H | L | H) of d_out
            Pd, wo = self._pack_split([do2]), ops["wb"][-d:]
            d_gated = torch.mm(Pd, torch.cat([wo[:, :d], wo[:, :d], wo[:, d:2 * d]], 0), out_dtype=torch.float32)
            parts = next(q_ for q_ in (16, 8, 4, 2, 1) if (3 * n) % q_ == 0)
            rows = 3 * n // parts
            torch.sum(torch.bmm(Pd.view(parts, rows, d).transpose(1, 2), cache["gated"].view(parts, rows, d),
                                out_dtype=torch.float32), 0, out=grads.w_o)
        else:
            d_gated = do2 @ p.w_o
            grads.w_o += _wgrad(do2, cache["gated"].view(n, d))
        d_attn, d_ycomb = _new(bs, s, d), _new(bs, s, d)
        if d % 4 == 0:
            lib.cms_gate_backward_bf16_rocm(d_gated.data_ptr(), cache["attn"].data_ptr(), cache["gate"].data_ptr(),
                                            self.k, d_attn.data_ptr(), d_ycomb.data_ptr(), n * d)
        else:
            D.call("cms_gate_backward_rocm", d_gated, cache["attn"].to(torch.float32), cache["gate"], self.k, d_attn,
                   d_ycomb, n * d)
        first, P, rows_stack, d_x = 0, None, 0, None
        if stack is not None:
            # ONE packed operand for the attention group and every stacked level: P = (H | L), each half
            # rows_stack wide with the projections in the order of the packed weights
            first, rows_stack = stack["na"], ops["rows_stack"]
            P = _new(n, 2 * rows_stack, dtype=torch.bfloat16)
            self._levels_backward_stacked(stack, cache["levels"], d_ycomb, bs, s, grads, P, rows_stack)
        for lv in range(first, self.k):
            dx = self._level_backward(lv, cache["levels"][lv], x2, d_ycomb, bs, s, grads)
            d_x = dx if d_x is None else d_x.add_(dx)
        dq, dk, dv = _new(bs, s, d), _zeros(bs, s, d), _zeros(bs, s, d)
        if cache["aw"].dtype == torch.float32:
            D.call("swa_backward_lse_bf16_rocm", cache["q"], cache["k"], cache["v"], cache["aw"], d_attn, dq, dk, dv,
                   s, nh, hd, self.window, bs)
        else:
            D.call("swa_backward_f32_cuda", cache["q"], cache["k"], cache["v"], cache["aw"], d_attn, dq, dk, dv, s,
                   nh, hd, self.window, bs, 0)
        dq2, dk2, dv2 = dq.view(n, d), dk.view(n, d), dv.view(n, d)
        if P is None:
            dx = self._group_grads(ops, 0, x2, (dq2, dk2, dv2), (p.w_q, p.w_k, p.w_v),
                                   (grads.w_q, grads.w_k, grads.w_v))
            d_x = dx if d_x is None else d_x.add_(dx)
            return d_x.view(bs, s, d), grads
        ptrs = (ctypes.c_void_p * 3)(dq2.data_ptr(), dk2.data_ptr(), dv2.data_ptr())
        lib.split_pack_bf16_ld_rocm(ptrs, 3, d, P.data_ptr(), n, d, 2 * rows_stack, 0, rows_stack, -1)
        # d_x = H Wh + L Wh + H Wl: (H | L) . (Wh ; Wh), then H . Wl added by a second GEMM on the H columns
        ws = ops["wstack"]
        dx = torch.mm(P, ws[:2 * rows_stack], out_dtype=torch.float32)
        dx = torch.addmm(dx, P[:, :rows_stack], ws[2 * rows_stack:], out_dtype=torch.float32)
        d_x = dx if d_x is None else d_x.add_(dx)
        # weight gradients of all these projections: (H^T xh ; L^T xh) and H^T xl, the contraction over the
        # tokens cut into slabs that run as one batched GEMM and are summed
        parts = next(q_ for q_ in (4, 2, 1) if n % q_ == 0)
        Pv, xv = P.view(parts, n // parts, 2 * rows_stack), ops["xa"].view(parts, n // parts, 3 * d)
        dw_hl = torch.bmm(Pv.transpose(1, 2), xv[:, :, :d], out_dtype=torch.float32).sum(0)
        dw_h = torch.bmm(Pv[:, :, :rows_stack].transpose(1, 2), xv[:, :, 2 * d:], out_dtype=torch.float32).sum(0)
        gp = grads.pack[:rows_stack]
        torch.add(dw_hl[:rows_stack], dw_hl[rows_stack:], out=gp)
        gp += dw_h
        return d_x.view(bs, s, d), grads


class GraphCache:
    """Captured graphs keyed by (pulse pattern, shape), valid for one generation of the library's
    scratch arena: a graph holds the scratch addresses of the calls it recorded, and when a slot has
    been reallocated since (a larger shape, nlh_release_workspace) those addresses are dead, so every
    cached graph is dropped and captured again rather than replayed."""

    def __init__(self, generation_fn):
        self._gen_fn, self._gen, self._graphs = generation_fn, None, {}

    def get(self, key):
        if self._gen != self._gen_fn():
            self._graphs.clear()
        return self._graphs.get(key)

    def put(self, key, value):
        """Call after the capture: the generation that the captured addresses belong to is read here."""
        gen = self._gen_fn()
        if self._gen != gen:
            self._graphs.clear()
            self._gen = gen
        self._graphs[key] = value

    def __len__(self):
        return len(self._graphs)


class MagTrainer:
    """forward + backward + frequency-aware AdamW step (core/src/gpu_optimizer.rs:403-515)."""

    def __init__(self, layer: MagLayer, lr=3e-4, beta1=0.9, beta2=0.95, eps=1e-8, weight_decay=0.1,
                 max_grad_norm=1.0):
        self.layer, self.lr, self.max_grad_norm = layer, lr, max_grad_norm
        p = layer.p
        self.grads = layer.new_grads()
        self.opt = FrequencyAwareAdamW(layer.k, beta1, beta2, eps, weight_decay)
        self.state = []
        groups = [-1] * 4 + [lv for lv in range(layer.k) for _ in range(9)]
        for grp, w, g in zip(groups, p.tensors(), self.grads.tensors()):
            m, v = torch.zeros_like(w), torch.zeros_like(w)
            self.state.append((m, v))
            tid = self.opt.add_tensor(grp, w, g, m, v)
            # b_theta is held in [-10, 2] after every level update (gpu_optimizer.rs:491-493)
            if grp >= 0 and any(w is lp.b_theta for lp in p.levels):
                self.opt.set_clamp(tid, -10.0, 2.0)
        self.scale = torch.zeros(2, dtype=torch.float32, device="cuda")
        # gradients that reach a level while it is frozen wait here until it fires (conductor.rs:224-261)
        self.error_buffers = [ErrorBuffer(l.tensors()) for l in p.levels]

    def _optimizer_and_error_buffers(self, pulse):
        """The step's parameter updates in the reference's order (core/tests/test_cms.rs:66-84): the
        optimizer for everything that fired, then, for a level that fired with gradients waiting from its
        frozen steps, their plain gradient step; a frozen level's gradients of this step join its buffer."""
        layer = self.layer
        for lv in range(layer.k):
            if not pulse.active_levels[lv]:
                self.error_buffers[lv].accumulate(self.grads.levels[lv].tensors())
        self.opt.step(pulse, self.lr, self.max_grad_norm, self.scale)
        for lv in range(layer.k):
            eb = self.error_buffers[lv]
            if pulse.active_levels[lv] and eb.steps_accumulated > 0:
                eb.apply_and_reset(layer.p.levels[lv].tensors(), self.lr)

    def _forward_backward(self, x, d_out):
        out, cache = self.layer.forward(x)
        self.layer.backward(cache, d_out, self.grads)
        return out

    def step_graphed(self, x, d_out):
        """One training step with a given upstream gradient.  Forward + backward (some 330 launches,
        launch-bound on the host) are replayed from a HIP graph captured once per pulse pattern and
        input shape; the optimizer runs eagerly, its bias corrections change every step.  Returns the
        layer output (a buffer the next replay overwrites)."""
        layer = self.layer
        layer.conductor.set_seq_len(x.shape[1])
        pulse = layer.conductor.pulse()
        key = (tuple(bool(a) for a in pulse.active_levels), tuple(x.shape))
        graphs = self.__dict__.setdefault("_graphs", GraphCache(lib.nlh_workspace_generation))
        entry = graphs.get(key)
        if entry is None:
            entry = self._capture(x, d_out)
            graphs.put(key, entry)
        graph, xs, ds, out = entry
        # the graph reads its inputs at fixed addresses; a caller that already writes its batch there
        # (graph_inputs) spares the two copies
        if x.data_ptr() != xs.data_ptr():
            xs.copy_(x)
        if d_out.data_ptr() != ds.data_ptr():
            ds.copy_(d_out)
        graph.replay()
        self._optimizer_and_error_buffers(pulse)
        layer.conductor.advance()
        return out

    def graph_inputs(self, shape):
        """The input and upstream-gradient buffers that the captured step for the current pulse pattern and this
        input shape reads (None before its first step_graphed): a producer that fills them in place and passes
        them to step_graphed avoids a copy of each per step."""
        pulse = self.layer.conductor.pulse()
        graphs = self.__dict__.get("_graphs")
        entry = None if graphs is None else graphs.get((tuple(bool(a) for a in pulse.active_levels), tuple(shape)))
        return None if entry is None else (entry[1], entry[2])

    def _capture(self, x, d_out):
        """Warm-up on a side stream, then the capture.  Whatever happens in between (a recorded scratch error, an
        allocation failure), the library's launch stream goes back to the null stream and the context memories that
        the warm-up advanced are put back: a failed capture must not leave every later call of the process launching
        on a dead or capturing stream."""
        layer = self.layer
        xs, ds = x.clone(), d_out.clone()
        layer.ensure_state(x.shape[0])
        saved = [(m.clone(), z.clone()) for m, z in zip(layer.m_state, layer.s_state)]
        restored = False
        try:
            # the warm-up sizes every scratch buffer (nothing may allocate while a graph is captured)
            side = torch.cuda.Stream()
            side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(side):
                lib.nlh_set_stream(ctypes.c_void_p(side.cuda_stream))
                self._forward_backward(xs, ds)
                for (m, z), m0, z0 in zip(saved, layer.m_state, layer.s_state):
                    m0.copy_(m); z0.copy_(z)
                restored = True
            torch.cuda.current_stream().wait_stream(side)
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                lib.nlh_set_stream(ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
                out = self._forward_backward(xs, ds)
            return (graph, xs, ds, out)
        finally:
            lib.nlh_set_stream(None)
            if not restored:
                for (m, z), m0, z0 in zip(saved, layer.m_state, layer.s_state):
                    m0.copy_(m); z0.copy_(z)

    def step(self, x, d_out_fn):
        """One training step; d_out_fn(out) gives the upstream gradient.  Returns out."""
        out, cache = self.layer.forward(x)
        self.layer.backward(cache, d_out_fn(out), self.grads)
        self._optimizer_and_error_buffers(cache["pulse"])
        self.layer.conductor.advance()
        return out
