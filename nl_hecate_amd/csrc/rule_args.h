// Argument blocks of the exact / frozen-M0 memory-rule kernels, shared by the tiled kernels
// (memory_rules.hip: head sizes 8, 16, 32, 64, 128 in registers) and the general ones
// (memory_rules_generic.hip: any head size, state in memory).
#pragma once

namespace nlh {

struct FwdArgs {
    const float *k, *v, *q, *alpha, *theta, *eta, *m_initial, *s_initial;
    float *m_out, *s_out, *y;
    int seq_len, input_stride, ckpt_interval, parts;
    long long m_stride;      // elements between chains in m_initial / s_initial
    long long state_stride;  // elements between chains in m_out / s_out
    float error_clip, m_norm_max;
    // uncoupled kernels only, may be null: [batch * parts] upper bounds of max_t sum(M_t^2) over the workgroup's rows
    // (every lane keeps the largest sum of squares its own elements reached; the lanes' maxima are added up)
    float *msq_part;
};

enum { STORE_NONE = 0, STORE_TRAJ = 1, STORE_CKPT = 2 };

// Reverse sweep over [t_start, t_end) of every chain, reading the trajectory
// M_{t_start..t_end}, S_{t_start..t_end-1} from memory (the reference's
// *_backward and *_backward_segment contract).
struct BwdArgs {
    const float *k, *v, *q, *alpha, *theta, *eta, *m_states, *s_states, *d_y;
    const float *d_m_seed, *d_s_seed;      // [B, dd] or null (zero)
    float *d_k, *d_v, *d_q, *d_alpha, *d_theta, *d_eta;
    float *ws_dq, *ws_dk, *ws_gate;        // partial sums when parts > 1
    float *d_m_out, *d_s_out;              // [B, dd]
    int seq_len, t_start, t_end, parts, batch;
    long long traj_stride;                 // elements between chains in m_states
    float error_clip;
};


// Any head size d >= 1, clip and projection included: one workgroup per chain, the state in memory.
void launch_fwd_generic(const FwdArgs &a, int d, int batch, bool has_s, int store, bool frozen);
void launch_bwd_generic(const BwdArgs &a, int d, bool has_s, bool frozen);

}  // namespace nlh
