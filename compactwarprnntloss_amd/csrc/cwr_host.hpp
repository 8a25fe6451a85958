// Host-side declarations shared by the translation units of libcwarp_rnnt_hip.so.
#pragma once

#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

#include "../../include/cwarp_rnnt_hip.h"
#include "cwr_device.hpp"

namespace cwr {

typedef long long i64;

// One batch as the kernels see it.
struct Batch {
    const void* x;
    int dtype;
    i64 R;
    int V;
    const int* lx;
    const int* ly;
    const int* y;
    i64 y_stride;
    i64 y_len;
    int N;
    int blank;
    int mode;
    i64 max_u;
    const i64* row_off;
    const i64* lab_off;
    int* status;
    hipStream_t stream;
};

// Scratch carved out of the caller's workspace.  lp / alpha / beta use the strip layout of
// lattice_slot(); all values are base-2 logarithms.
struct Workspace {
    i64* pad_off;   // N+1  first lattice slot of each sequence (-1: sequence skipped)
    i64* fill_off;  // N+1  first chunk of each sequence in k_fill's work list (a running sum: searchable)
    i64* bnd_off;   // N+1  first boundary-stream entry of each sequence
    int* seqmode;   // N+1  per sequence: 0 = walked in the scaled linear domain; bit 0 = in the log domain
                    //      (set by the gather pass), bits 1 / 2 = alpha / beta repeated in the log domain
    LpStore lp;     // 2 x slot_cap  gathered (blank, label) probabilities and log-probabilities
    double* alpha;  // slot_cap  log2(alpha), or alpha * 2^scale_a[block][column] (see seqmode)
    double* beta;   // slot_cap
    int* scale_a;   // slot_cap/16+1  per strip: exponent of each (16-step block, column) of the alpha walk
    int* scale_b;   // same for beta
    double* bnd_a;  // bnd_cap   alpha values handed from one 64-label strip to the next
    double* bnd_b;  // bnd_cap   same for beta
    char* aux;      // 12 R bytes  per-row outputs of the gather pass when the caller keeps none
    i64 slot_cap;
    i64 bnd_cap;
};

size_t workspace_bytes(i64 N, i64 R, i64 max_u);
bool carve_workspace(void* base, size_t bytes, i64 N, i64 R, i64 max_u, Workspace* ws);
int workspace_section(i64 N, i64 R, i64 max_u, int which, size_t* offset, size_t* bytes);

int launch_offsets(const int* lx, const int* ly, i64 N, i64 R, i64 max_u, i64 slot_cap, i64 bnd_cap,
                   i64* row_off, i64* lab_off, i64* pad_off, i64* fill_off, i64* bnd_off, int* seqmode, int* status,
                   float* costs_or_null, float* reduced_or_null, hipStream_t stream);
// grads (may be null): rows of skipped sequences get a zero record there
int launch_gather(const Batch& b, const Workspace& ws, float* lse, int* rowinfo, float* grads);
int launch_rowinfo(const Batch& b, int* rowinfo);
// The fused output layer: logits = h (R,H) x W^T (V,H) + bias, never stored.  b.dtype is the type of
// h and W (CWR_F16 or CWR_BF16), b.V the vocabulary, b.x unused.
struct JointOperands {
    const void* h;
    const void* w;
    const float* bias;  // may be null
    i64 H;
    // h == null: the joint rows are formed in the kernel, row(n,t,u) = act(f[n,t,:] + g[n,u,:]), from
    // f (N,T_pad,H) and g (N,Up_pad,H); h_out (may be null) receives them
    const void* f;
    const void* g;
    void* h_out;
    int act;
    i64 T_pad, Up_pad;
};
int launch_joint_gather(const Batch& b, const Workspace& ws, const JointOperands& j, float* lse, int* rowinfo,
                        float* grads);
int launch_lattice(const Batch& b, const Workspace& ws, bool beta_only);
// reduced (may be null): 2 floats, sum and mean of the N costs
int launch_fill(const Batch& b, const Workspace& ws, const int* rowinfo, float* grads, float* costs,
                float* reduced);
int launch_cost_from_beta(const Batch& b, const Workspace& ws, float* costs, float* reduced);
// d(total) / d(cost of sequence n) = p[n * stride] * scale; stride 0 broadcasts one value
struct GradOut {
    const float* p;
    i64 stride;
    float scale;
};
int launch_grad(const Batch& b, const int* rowinfo, const float* grads, const float* lse,
                const GradOut grad_costs, void* grad_x);

// d loss / d logits of the rows [0, R) of a block, from logits formed again on the matrix cores
int launch_joint_dlogits(int dtype, const JointOperands& j, i64 R, i64 V, i64 N, int blank, const int* rowinfo,
                         const float* grads, const float* lse, const GradOut go, void* dlogits, hipStream_t stream);

int launch_export(const int* lx, const int* ly, int N, i64 T_pad, i64 Up_pad, const Workspace& ws,
                  double* alphas_out, double* betas_out, hipStream_t stream);
int launch_repack(const void* src, void* dst, size_t esize, const int* lx, const int* ly, const i64* row_off, i64 N,
                  i64 T_pad, i64 Up_pad, i64 V, i64 R, bool unpack, int* status, hipStream_t stream);

// forward (backward = false): a = f, b = g, o1 = out; backward: a = dh, b = h (unused without an
// activation), o1 = df, o2 = dg
int launch_join(int dtype, int act, bool backward, const void* a, const void* b, void* o1, void* o2, const int* lx,
                const int* ly, const i64* row_off, i64 N, i64 T_pad, i64 Up_pad, i64 H, i64 R, int* status,
                hipStream_t stream);

// Launches go through CWR_LAUNCH, which first drops whatever error an earlier HIP call of this thread
// (the caller's, or another library's) left pending, so that check_launch() reports this launch and
// nothing else.  The runtime's own code is kept for cwr_strerror.
#define CWR_LAUNCH(...)                      \
    do {                                     \
        (void)hipGetLastError();             \
        hipLaunchKernelGGL(__VA_ARGS__);     \
    } while (0)

extern thread_local int g_last_hip_error;  // hipError_t of the last refused launch or failed call

inline int check_launch() {
    const hipError_t e = hipGetLastError();
    if (e == hipSuccess) return CWR_OK;
    g_last_hip_error = (int)e;
    return CWR_ERR_LAUNCH;
}

void set_wait_limit(int polls);  // lattice.hip: polls a wait inside k_lattice may spend (<= 0: default)

}  // namespace cwr
