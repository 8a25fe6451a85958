// extern "C" entry points of libcwarp_rnnt_hip.so: argument validation (host only, before any HIP
// call), workspace carving and kernel sequencing.  Mirrors the orchestration of
// cwarp_cuda.cpp:58-136 without its host synchronisations and allocations.
#include <cstdio>
#include <mutex>

#include "../../include/cwarp_rnnt_hip_testing.h"
#include "cwr_device.hpp"
#include "cwr_host.hpp"

// Scratch of cwr_forward_noalloc: one copy per GPU, held from the moment the library's code is
// loaded on that GPU until the process ends.  Host code never uses this name as an address (it is
// a host-side stand-in); it asks the runtime for the device address once per GPU, below.
static __device__ __align__(256) unsigned char scratch[CWR_NOALLOC_SCRATCH_BYTES];

namespace cwr {

thread_local int g_last_hip_error = 0;

constexpr int kMaxDevices = 64;
static std::mutex g_scratch_mu;
static void* g_scratch_ptr[kMaxDevices];  // device address of `scratch` on each GPU, once known

// Address of the current GPU's copy of `scratch`.  The first call on a GPU asks the runtime; later
// calls are a table look-up.
static int scratch_of_current_device(void** out) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) { g_last_hip_error = (int)e; return CWR_ERR_RUNTIME; }
    if (dev < 0 || dev >= kMaxDevices) return CWR_ERR_TOO_LARGE;
    std::lock_guard<std::mutex> lock(g_scratch_mu);
    if (!g_scratch_ptr[dev]) {
        void* p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !p) { g_last_hip_error = (int)e; return CWR_ERR_RUNTIME; }
        g_scratch_ptr[dev] = p;
    }
    *out = g_scratch_ptr[dev];
    return CWR_OK;
}

static size_t align_up(size_t v) { return (v + 255) & ~(size_t)255; }

struct Layout {
    size_t pad_off, fill_off, bnd_off, seqmode, lp, lpl, alpha, beta, scale_a, scale_b, bnd_a, bnd_b, aux, total;
    i64 slot_cap, bnd_cap;
};

// Upper bounds, from what the host knows (N, R, max_u), of the lattice slots and boundary-stream
// entries a batch can need: every strip adds at most (63 + 2*kRowShift) * 128 padding slots to the
// R real cells (one padding row per lane but the first, and the rows in front and behind), a
// sequence's last strip one column of padding when its width is odd (one slot per frame: R of them
// for a batch without labels, none when every width is even), and a sequence has at most
// ceil((max_u+1)/128) strips.
static Layout layout_for(i64 N, i64 R, i64 max_u) {
    Layout l;
    const i64 n = N > 0 ? N : 0, r = R > 0 ? R : 0, mu = max_u > 0 ? max_u : 0;
    const i64 strips = strip_count(mu + 1);
    i64 by_strips = 2 * r + n * strips * (63 + 2 * kRowShift) * kStripCols;
    // a strip holds at most 2 * (1 + 2*kRowShift) slots per cell (one frame, one column)
    i64 by_rows = r * (2 + 4 * kRowShift);
    l.slot_cap = by_strips < by_rows ? by_strips : by_rows;
    if (l.slot_cap < 0) l.slot_cap = 0;
    // boundary streams: (S-1)*(T+kBndPad) per sequence, with (S-1)*128 <= U < rows of the sequence
    const i64 bnd_by_strips = n * (strips - 1) * kBndPad, bnd_by_rows = r * (kBndPad / 64);
    l.bnd_cap = r / kStripCols + (bnd_by_strips < bnd_by_rows ? bnd_by_strips : bnd_by_rows) + 1;
    size_t at = 0;
    l.pad_off = at; at = align_up(at + (size_t)(n + 1) * sizeof(i64));
    l.fill_off = at; at = align_up(at + (size_t)(n + 1) * sizeof(i64));
    l.bnd_off = at; at = align_up(at + (size_t)(n + 1) * sizeof(i64));
    l.seqmode = at; at = align_up(at + (size_t)(n + 1) * sizeof(int));
    l.lp = at; at = align_up(at + (size_t)l.slot_cap * sizeof(float2));
    l.lpl = at; at = align_up(at + (size_t)l.slot_cap * sizeof(float2));
    l.alpha = at; at = align_up(at + (size_t)l.slot_cap * sizeof(double));
    l.beta = at; at = align_up(at + (size_t)l.slot_cap * sizeof(double));
    l.scale_a = at; at = align_up(at + ((size_t)l.slot_cap / 16 + 1) * sizeof(int));
    l.scale_b = at; at = align_up(at + ((size_t)l.slot_cap / 16 + 1) * sizeof(int));
    l.bnd_a = at; at = align_up(at + (size_t)l.bnd_cap * sizeof(double));
    l.bnd_b = at; at = align_up(at + (size_t)l.bnd_cap * sizeof(double));
    l.aux = at; at = align_up(at + (size_t)r * 12);  // cwr_loss: row records (8 B) + lse (4 B) per row
    l.total = at;
    return l;
}

size_t workspace_bytes(i64 N, i64 R, i64 max_u) { return layout_for(N, R, max_u).total; }

bool carve_workspace(void* base, size_t bytes, i64 N, i64 R, i64 max_u, Workspace* ws) {
    Layout l = layout_for(N, R, max_u);
    if (bytes < l.total) return false;
    char* p = static_cast<char*>(base);
    ws->pad_off = reinterpret_cast<i64*>(p + l.pad_off);
    ws->fill_off = reinterpret_cast<i64*>(p + l.fill_off);
    ws->bnd_off = reinterpret_cast<i64*>(p + l.bnd_off);
    ws->seqmode = reinterpret_cast<int*>(p + l.seqmode);
    ws->lp.p = reinterpret_cast<float2*>(p + l.lp);
    ws->lp.l = reinterpret_cast<float2*>(p + l.lpl);
    ws->scale_a = reinterpret_cast<int*>(p + l.scale_a);
    ws->scale_b = reinterpret_cast<int*>(p + l.scale_b);
    ws->alpha = reinterpret_cast<double*>(p + l.alpha);
    ws->beta = reinterpret_cast<double*>(p + l.beta);
    ws->bnd_a = reinterpret_cast<double*>(p + l.bnd_a);
    ws->bnd_b = reinterpret_cast<double*>(p + l.bnd_b);
    ws->aux = p + l.aux;
    ws->slot_cap = l.slot_cap;
    ws->bnd_cap = l.bnd_cap;
    return true;
}

int workspace_section(i64 N, i64 R, i64 max_u, int which, size_t* offset, size_t* bytes) {
    if (!offset || !bytes) return CWR_ERR_NULL;
    if (N < 0 || R < 0 || max_u < 0) return CWR_ERR_SHAPE;
    Layout l = layout_for(N, R, max_u);
    switch (which) {
        case 0: *offset = l.lp; *bytes = (size_t)l.slot_cap * sizeof(float2); return CWR_OK;
        case 1: *offset = l.alpha; *bytes = (size_t)l.slot_cap * sizeof(double); return CWR_OK;
        case 2: *offset = l.beta; *bytes = (size_t)l.slot_cap * sizeof(double); return CWR_OK;
        case 3: *offset = l.pad_off; *bytes = (size_t)(N + 1) * sizeof(i64); return CWR_OK;
        case 4: *offset = l.seqmode; *bytes = (size_t)(N + 1) * sizeof(int); return CWR_OK;
        case 5: *offset = l.scale_a; *bytes = ((size_t)l.slot_cap / 16 + 1) * sizeof(int); return CWR_OK;
        case 6: *offset = l.scale_b; *bytes = ((size_t)l.slot_cap / 16 + 1) * sizeof(int); return CWR_OK;
        case 7: *offset = l.lpl; *bytes = (size_t)l.slot_cap * sizeof(float2); return CWR_OK;
    }
    return CWR_ERR_SHAPE;
}

static size_t elem_size(int dtype) {
    switch (dtype) {
        case CWR_F32: return 4;
        case CWR_F16: return 2;
        case CWR_BF16: return 2;
        case CWR_F64: return 8;
    }
    return 0;
}

static bool misaligned(const void* p, size_t a) { return (reinterpret_cast<uintptr_t>(p) & (a - 1)) != 0; }

// Checks shared by the three compute entry points.
static int check_common(const void* x, bool need_x, int dtype, int64_t R, int64_t V, const int32_t* lx,
                        const int32_t* ly, const int32_t* y, int64_t y_len, int64_t N, int32_t blank,
                        int mode, bool need_lengths = true) {
    if (dtype < CWR_F32 || dtype > CWR_F64) return CWR_ERR_DTYPE;
    if (mode != CWR_MODE_LOGPROB && mode != CWR_MODE_FUSED) return CWR_ERR_MODE;
    if (N < 0 || R < 0 || V < 1 || y_len < 0) return CWR_ERR_SHAPE;
    if (N > 0x3fffffff || V > 0x3fffffff) return CWR_ERR_TOO_LARGE;
    if (R > 0 && N == 0) return CWR_ERR_SHAPE;
    if (blank < 0 || blank >= V) return CWR_ERR_BLANK;
    if (need_lengths && N > 0 && (!lx || !ly)) return CWR_ERR_NULL;
    if (need_lengths && y_len > 0 && !y) return CWR_ERR_NULL;
    if (need_x && R > 0 && !x) return CWR_ERR_NULL;
    if (x && misaligned(x, elem_size(dtype))) return CWR_ERR_ALIGN;
    if (misaligned(lx, 4) || misaligned(ly, 4) || misaligned(y, 4)) return CWR_ERR_ALIGN;
    return CWR_OK;
}

static Batch make_batch(const void* x, int dtype, int64_t R, int64_t V, const int32_t* lx, const int32_t* ly,
                        const int32_t* y, int64_t y_stride, int64_t y_len, int64_t N, int32_t blank, int mode,
                        int64_t max_u, const int64_t* row_off, const int64_t* lab_off, int32_t* status,
                        void* stream) {
    Batch b;
    b.x = x; b.dtype = dtype; b.R = R; b.V = (int)V; b.lx = lx; b.ly = ly; b.y = y;
    b.y_stride = y_stride; b.y_len = y_len; b.N = (int)N; b.blank = blank; b.mode = mode; b.max_u = max_u;
    b.row_off = reinterpret_cast<const i64*>(row_off);
    b.lab_off = reinterpret_cast<const i64*>(lab_off);
    b.status = status;
    b.stream = static_cast<hipStream_t>(stream);
    return b;
}

}  // namespace cwr

using namespace cwr;

extern "C" {

int cwr_version(void) { return 130; }

const char* cwr_strerror(int status) {
    switch (status) {
        case CWR_OK: return "success";
        case CWR_ERR_NULL: return "a required pointer is NULL";
        case CWR_ERR_DTYPE: return "unsupported dtype (expected CWR_F32, CWR_F16, CWR_BF16 or CWR_F64)";
        case CWR_ERR_MODE: return "unsupported mode (expected CWR_MODE_LOGPROB or CWR_MODE_FUSED)";
        case CWR_ERR_SHAPE: return "negative or inconsistent sizes";
        case CWR_ERR_BLANK: return "blank index outside [0, V)";
        case CWR_ERR_ALIGN: return "a buffer is not aligned to its element size";
        case CWR_ERR_LAUNCH:
        case CWR_ERR_RUNTIME: {
            // with the runtime's own words for the last failure seen by this thread
            static thread_local char buf[192];
            snprintf(buf, sizeof buf, "%s: %s", status == CWR_ERR_LAUNCH ? "the HIP runtime refused a kernel launch"
                                                                         : "a HIP runtime call failed",
                     hipGetErrorString((hipError_t)g_last_hip_error));
            return buf;
        }
        case CWR_ERR_TOO_LARGE: return "a size exceeds what the kernels can index (or the built-in scratch can hold)";
    }
    return "unknown status";
}

size_t cwr_workspace_bytes(int64_t N, int64_t R, int64_t max_u) {
    if (N < 0 || R < 0 || max_u < 0) return 0;
    return workspace_bytes(N, R, max_u);
}

int cwr_workspace_section(int64_t N, int64_t R, int64_t max_u, int which, size_t* offset, size_t* bytes) {
    return workspace_section(N, R, max_u, which, offset, bytes);
}

int cwr_cost_rule(double fwd_log2, double bwd_log2, float* cost) {
    if (!cost) return -1;
    return cost_rule(fwd_log2, bwd_log2, cost) ? 1 : 0;
}

void cwr_debug_wait_limit(int polls) { set_wait_limit(polls); }

int64_t cwr_lattice_slot(int64_t t, int64_t u, int64_t T, int64_t U) {
    if (t < 0 || u < 0 || t >= T || u > U) return -1;
    return lattice_slot(t, u, T, U + 1);
}

int cwr_offsets(const int32_t* lx, const int32_t* ly, int64_t N, int64_t R, int64_t* row_off,
                int64_t* lab_off, int32_t* status, void* stream) {
    if (N < 0) return CWR_ERR_SHAPE;
    if (N > 0x3fffffff) return CWR_ERR_TOO_LARGE;
    if (!row_off || !lab_off || !status || (N > 0 && (!lx || !ly))) return CWR_ERR_NULL;
    if (misaligned(lx, 4) || misaligned(ly, 4) || misaligned(row_off, 8) || misaligned(lab_off, 8) ||
        misaligned(status, 4))
        return CWR_ERR_ALIGN;
    return launch_offsets(lx, ly, N, R, 0, 0, 0, reinterpret_cast<i64*>(row_off),
                          reinterpret_cast<i64*>(lab_off), nullptr, nullptr, nullptr, nullptr, status, nullptr, nullptr,
                          static_cast<hipStream_t>(stream));
}

// Everything the host can judge about a forward call's arguments, before any HIP call.
static int check_forward(const void* x, int dtype, int64_t R, int64_t V, const int32_t* lx, const int32_t* ly,
                         const int32_t* y, int64_t y_len, int64_t N, int32_t blank, int mode, int64_t max_u,
                         const int64_t* row_off, const int64_t* lab_off, const int32_t* status,
                         const int32_t* rowinfo, const float* lse, const float* grads, const float* costs,
                         const float* reduced, bool with_grad, bool joint) {
    int rc = check_common(x, !joint, dtype, R, V, lx, ly, y, y_len, N, blank, mode);
    if (rc != CWR_OK) return rc;
    if (max_u < 0) return CWR_ERR_SHAPE;
    if (!row_off || !lab_off || !status) return CWR_ERR_NULL;
    if (N > 0 && !costs) return CWR_ERR_NULL;
    if (R > 0 && mode == CWR_MODE_FUSED && !lse) return CWR_ERR_NULL;
    if (R > 0 && (!rowinfo || (with_grad && !grads))) return CWR_ERR_NULL;
    if (misaligned(row_off, 8) || misaligned(lab_off, 8) || misaligned(status, 4) || misaligned(lse, 4) ||
        misaligned(rowinfo, 8) || misaligned(grads, 8) || misaligned(costs, 4) || misaligned(reduced, 4))
        return CWR_ERR_ALIGN;
    return CWR_OK;
}

static int forward_impl(const void* x, int dtype, int64_t R, int64_t V, const int32_t* lx, const int32_t* ly,
                        const int32_t* y, int64_t y_stride, int64_t y_len, int64_t N, int32_t blank, int mode,
                        int64_t max_u, void* workspace, size_t workspace_bytes_, int64_t* row_off,
                        int64_t* lab_off, int32_t* status, int32_t* rowinfo, float* lse, float* grads,
                        float* costs, float* reduced, void* stream, bool with_grad,
                        const JointOperands* joint = nullptr, hipEvent_t* marks = nullptr) {
    int rc = check_forward(x, dtype, R, V, lx, ly, y, y_len, N, blank, mode, max_u, row_off, lab_off, status,
                           rowinfo, lse, grads, costs, reduced, with_grad, joint != nullptr);
    if (rc != CWR_OK) return rc;
    if (!workspace) return CWR_ERR_NULL;
    if (misaligned(workspace, 256)) return CWR_ERR_ALIGN;
    Workspace ws;
    if (!carve_workspace(workspace, workspace_bytes_, N, R, max_u, &ws)) return CWR_ERR_SHAPE;

    hipStream_t s = static_cast<hipStream_t>(stream);
    // marks (measurement hook only): five events, recorded in front of and behind the four stages
    auto mark = [&](int i) { if (marks) (void)hipEventRecord(marks[i], s); };
    mark(0);
    rc = launch_offsets(lx, ly, N, R, max_u, ws.slot_cap, ws.bnd_cap, reinterpret_cast<i64*>(row_off),
                        reinterpret_cast<i64*>(lab_off), ws.pad_off, ws.fill_off, ws.bnd_off, ws.seqmode, status, costs,
                        reduced, s);
    if (rc != CWR_OK) return rc;
    mark(1);
    Batch b = make_batch(x, dtype, R, V, lx, ly, y, y_stride, y_len, N, blank, mode, max_u, row_off, lab_off,
                         status, stream);
    rc = joint ? launch_joint_gather(b, ws, *joint, lse, rowinfo, with_grad ? grads : nullptr)
               : launch_gather(b, ws, lse, rowinfo, with_grad ? grads : nullptr);
    if (rc != CWR_OK) return rc;
    mark(2);
    rc = launch_lattice(b, ws, !with_grad);
    if (rc != CWR_OK) return rc;
    mark(3);
    rc = with_grad ? launch_fill(b, ws, rowinfo, grads, costs, reduced) : launch_cost_from_beta(b, ws, costs, reduced);
    mark(4);
    return rc;
}

int cwr_forward(const void* x, int dtype, int64_t R, int64_t V, const int32_t* lx, const int32_t* ly,
                const int32_t* y, int64_t y_stride, int64_t y_len, int64_t N, int32_t blank, int mode,
                int64_t max_u, void* workspace, size_t workspace_bytes_, int64_t* row_off, int64_t* lab_off,
                int32_t* status, int32_t* rowinfo, float* lse, float* grads, float* costs, void* stream) {
    return forward_impl(x, dtype, R, V, lx, ly, y, y_stride, y_len, N, blank, mode, max_u, workspace,
                        workspace_bytes_, row_off, lab_off, status, rowinfo, lse, grads, costs, nullptr, stream,
                        true);
}

int cwr_debug_forward_stage_times(const void* x, int dtype, int64_t R, int64_t V, const int32_t* lx,
                                  const int32_t* ly, const int32_t* y, int64_t y_stride, int64_t y_len, int64_t N,
                                  int32_t blank, int mode, int64_t max_u, void* workspace, size_t workspace_bytes_,
                                  int64_t* row_off, int64_t* lab_off, int32_t* status, int32_t* rowinfo, float* lse,
                                  float* grads, float* costs, void* stream, float* stage_us) {
    if (!stage_us) return CWR_ERR_NULL;
    hipEvent_t ev[5];
    int made = 0;
    int rc = CWR_OK;
    for (; made < 5; ++made) {
        const hipError_t e = hipEventCreate(&ev[made]);
        if (e != hipSuccess) { g_last_hip_error = (int)e; rc = CWR_ERR_RUNTIME; break; }
    }
    if (rc == CWR_OK)
        rc = forward_impl(x, dtype, R, V, lx, ly, y, y_stride, y_len, N, blank, mode, max_u, workspace,
                          workspace_bytes_, row_off, lab_off, status, rowinfo, lse, grads, costs, nullptr, stream,
                          true, nullptr, ev);
    if (rc == CWR_OK) {
        const hipError_t e = hipEventSynchronize(ev[4]);
        if (e != hipSuccess) { g_last_hip_error = (int)e; rc = CWR_ERR_RUNTIME; }
    }
    for (int i = 0; rc == CWR_OK && i < 4; ++i) {
        float ms = 0.f;
        const hipError_t e = hipEventElapsedTime(&ms, ev[i], ev[i + 1]);
        if (e != hipSuccess) { g_last_hip_error = (int)e; rc = CWR_ERR_RUNTIME; }
        stage_us[i] = ms * 1000.f;
    }
    for (int i = 0; i < made; ++i) (void)hipEventDestroy(ev[i]);
    return rc;
}

int cwr_forward_noalloc(const void* x, int dtype, int64_t R, int64_t V, const int32_t* lx, const int32_t* ly,
                        const int32_t* y, int64_t y_stride, int64_t y_len, int64_t N, int32_t blank, int mode,
                        int64_t max_u, int64_t* row_off, int64_t* lab_off, int32_t* status, int32_t* rowinfo,
                        float* lse, float* grads, float* costs, void* stream) {
    // everything the host can judge first, so that a call that cannot run touches no GPU
    int rc = check_forward(x, dtype, R, V, lx, ly, y, y_len, N, blank, mode, max_u, row_off, lab_off, status,
                           rowinfo, lse, grads, costs, nullptr, true, false);
    if (rc != CWR_OK) return rc;
    const size_t need = workspace_bytes(N, R, max_u);
    if (need > (size_t)CWR_NOALLOC_SCRATCH_BYTES) return CWR_ERR_TOO_LARGE;
    void* ws = nullptr;
    rc = scratch_of_current_device(&ws);
    if (rc != CWR_OK) return rc;
    return forward_impl(x, dtype, R, V, lx, ly, y, y_stride, y_len, N, blank, mode, max_u, ws, need, row_off,
                        lab_off, status, rowinfo, lse, grads, costs, nullptr, stream, true);
}

int cwr_joint_forward(const void* h, const void* w, const float* bias, int dtype, int64_t R, int64_t H, int64_t V,
                      const int32_t* lx, const int32_t* ly, const int32_t* y, int64_t y_stride, int64_t y_len,
                      int64_t N, int32_t blank, int64_t max_u, void* workspace, size_t workspace_bytes_,
                      int64_t* row_off, int64_t* lab_off, int32_t* status, int32_t* rowinfo, float* lse,
                      float* grads, float* costs, void* stream) {
    if (dtype != CWR_F16 && dtype != CWR_BF16) return CWR_ERR_DTYPE;
    if (H < 32 || H % 32 != 0) return CWR_ERR_SHAPE;  // K-slices of 32
    if (H > 0x3fffffff) return CWR_ERR_TOO_LARGE;
    if (R > 0 && (!h || !w)) return CWR_ERR_NULL;
    if (misaligned(h, 16) || misaligned(w, 16) || misaligned(bias, 4)) return CWR_ERR_ALIGN;
    JointOperands j;
    j.h = h; j.w = w; j.bias = bias; j.H = H;
    j.f = nullptr; j.g = nullptr; j.h_out = nullptr; j.act = 0; j.T_pad = 0; j.Up_pad = 0;
    return forward_impl(nullptr, dtype, R, V, lx, ly, y, y_stride, y_len, N, blank, CWR_MODE_FUSED, max_u, workspace,
                        workspace_bytes_, row_off, lab_off, status, rowinfo, lse, grads, costs, nullptr, stream, true,
                        &j);
}

int cwr_joint_forward_fg(const void* f, const void* g, int act, int64_t T_pad, int64_t Up_pad, void* h_out,
                         const void* w, const float* bias, int dtype, int64_t R, int64_t H, int64_t V,
                         const int32_t* lx, const int32_t* ly, const int32_t* y, int64_t y_stride, int64_t y_len,
                         int64_t N, int32_t blank, int64_t max_u, void* workspace, size_t workspace_bytes_,
                         int64_t* row_off, int64_t* lab_off, int32_t* status, int32_t* rowinfo, float* lse,
                         float* grads, float* costs, void* stream) {
    if (dtype != CWR_F16 && dtype != CWR_BF16) return CWR_ERR_DTYPE;
    if (act < CWR_ACT_NONE || act > CWR_ACT_RELU) return CWR_ERR_MODE;
    // the joint sizes whose rows a wave keeps in registers
    // the joint sizes whose rows a wave keeps in registers
    if (H % 64 != 0 || H < 128 || H > 1024) return CWR_ERR_SHAPE;
    if (T_pad < 0 || Up_pad < 0) return CWR_ERR_SHAPE;
    if (T_pad > 0x3fffffff || Up_pad > 0x3fffffff) return CWR_ERR_TOO_LARGE;
    if (R > 0 && (!f || !g || !w)) return CWR_ERR_NULL;
    if (R > 0 && (T_pad == 0 || Up_pad == 0)) return CWR_ERR_SHAPE;
    if (misaligned(f, 16) || misaligned(g, 16) || misaligned(h_out, 16) || misaligned(w, 16) || misaligned(bias, 4))
        return CWR_ERR_ALIGN;
    JointOperands j;
    j.h = nullptr; j.w = w; j.bias = bias; j.H = H;
    j.f = f; j.g = g; j.h_out = h_out; j.act = act; j.T_pad = T_pad; j.Up_pad = Up_pad;
    return forward_impl(nullptr, dtype, R, V, lx, ly, y, y_stride, y_len, N, blank, CWR_MODE_FUSED, max_u, workspace,
                        workspace_bytes_, row_off, lab_off, status, rowinfo, lse, grads, costs, nullptr, stream, true,
                        &j);
}

int cwr_joint_backward(const void* h, const void* w, const float* bias, int dtype, int64_t R, int64_t H, int64_t V,
                       int64_t N, int32_t blank, const int32_t* rowinfo, const float* grads, const float* lse,
                       const float* grad_costs, int64_t grad_stride, float grad_scale, void* dlogits, void* stream) {
    if (dtype != CWR_F16 && dtype != CWR_BF16) return CWR_ERR_DTYPE;
    if (R < 0 || N < 0 || V < 1) return CWR_ERR_SHAPE;
    if (H < 32 || H % 32 != 0) return CWR_ERR_SHAPE;  // K-slices of 32
    if (H > 0x3fffffff || V > 0x3fffffff || N > 0x3fffffff) return CWR_ERR_TOO_LARGE;
    if (blank < 0 || blank >= V) return CWR_ERR_BLANK;
    if (grad_stride != 0 && grad_stride != 1) return CWR_ERR_SHAPE;
    if (R == 0) return CWR_OK;
    if (!h || !w || !rowinfo || !grads || !lse || !grad_costs || !dlogits) return CWR_ERR_NULL;
    if (misaligned(h, 16) || misaligned(w, 16) || misaligned(bias, 4) || misaligned(rowinfo, 8) ||
        misaligned(grads, 8) || misaligned(lse, 4) || misaligned(grad_costs, 4) ||
        misaligned(dlogits, (V & 7) == 0 ? 16 : ((V & 3) == 0 ? 8 : 2)))  // rows leave as 16- / 8-byte stores
        return CWR_ERR_ALIGN;
    JointOperands j;
    j.h = h; j.w = w; j.bias = bias; j.H = H;
    const GradOut go = {grad_costs, grad_stride, grad_scale};
    return launch_joint_dlogits(dtype, j, R, V, N, blank, rowinfo, grads, lse, go, dlogits,
                                static_cast<hipStream_t>(stream));
}

int cwr_forward_reduced(const void* x, int dtype, int64_t R, int64_t V, const int32_t* lx, const int32_t* ly,
                        const int32_t* y, int64_t y_stride, int64_t y_len, int64_t N, int32_t blank, int mode,
                        int64_t max_u, void* workspace, size_t workspace_bytes_, int64_t* row_off,
                        int64_t* lab_off, int32_t* status, int32_t* rowinfo, float* lse, float* grads,
                        float* costs, float* reduced, void* stream) {
    if (!reduced) return CWR_ERR_NULL;
    return forward_impl(x, dtype, R, V, lx, ly, y, y_stride, y_len, N, blank, mode, max_u, workspace,
                        workspace_bytes_, row_off, lab_off, status, rowinfo, lse, grads, costs, reduced, stream,
                        true);
}

static int loss_impl(const void* x, int dtype, int64_t R, int64_t V, const int32_t* lx, const int32_t* ly,
                     const int32_t* y, int64_t y_stride, int64_t y_len, int64_t N, int32_t blank, int mode,
                     int64_t max_u, void* workspace, size_t workspace_bytes_, int64_t* row_off, int64_t* lab_off,
                     int32_t* status, float* costs, float* reduced, void* stream) {
    // the gather still needs somewhere to put lse and the row records: the workspace's aux section
    Workspace ws;
    float* lse = nullptr;
    int32_t* rowinfo = nullptr;
    if (workspace && N >= 0 && R >= 0 && max_u >= 0 &&
        carve_workspace(workspace, workspace_bytes_, N, R, max_u, &ws)) {
        rowinfo = reinterpret_cast<int32_t*>(ws.aux);
        lse = reinterpret_cast<float*>(ws.aux + (size_t)R * 8);
    }
    return forward_impl(x, dtype, R, V, lx, ly, y, y_stride, y_len, N, blank, mode, max_u, workspace,
                        workspace_bytes_, row_off, lab_off, status, rowinfo, lse, nullptr, costs, reduced, stream,
                        false);
}

int cwr_loss(const void* x, int dtype, int64_t R, int64_t V, const int32_t* lx, const int32_t* ly,
             const int32_t* y, int64_t y_stride, int64_t y_len, int64_t N, int32_t blank, int mode,
             int64_t max_u, void* workspace, size_t workspace_bytes_, int64_t* row_off, int64_t* lab_off,
             int32_t* status, float* costs, void* stream) {
    return loss_impl(x, dtype, R, V, lx, ly, y, y_stride, y_len, N, blank, mode, max_u, workspace,
                     workspace_bytes_, row_off, lab_off, status, costs, nullptr, stream);
}

int cwr_loss_reduced(const void* x, int dtype, int64_t R, int64_t V, const int32_t* lx, const int32_t* ly,
                     const int32_t* y, int64_t y_stride, int64_t y_len, int64_t N, int32_t blank, int mode,
                     int64_t max_u, void* workspace, size_t workspace_bytes_, int64_t* row_off, int64_t* lab_off,
                     int32_t* status, float* costs, float* reduced, void* stream) {
    if (!reduced) return CWR_ERR_NULL;
    return loss_impl(x, dtype, R, V, lx, ly, y, y_stride, y_len, N, blank, mode, max_u, workspace,
                     workspace_bytes_, row_off, lab_off, status, costs, reduced, stream);
}

int cwr_backward(const void* x, int dtype, int64_t R, int64_t V, const int32_t* lx, const int32_t* ly,
                 const int32_t* y, int64_t y_stride, int64_t y_len, int64_t N, int32_t blank, int mode,
                 const int64_t* row_off, const int64_t* lab_off, const int32_t* rowinfo,
                 const float* grads, const float* lse, const float* grad_costs, int64_t grad_stride,
                 float grad_scale, void* grad_x, void* stream) {
    int rc = check_common(x, mode == CWR_MODE_FUSED, dtype, R, V, lx, ly, y, y_len, N, blank, mode, false);
    if (rc != CWR_OK) return rc;
    (void)row_off;
    (void)lab_off;
    if (R > 0 && (!rowinfo || !grads || !grad_x || !grad_costs)) return CWR_ERR_NULL;
    if (grad_stride != 0 && grad_stride != 1) return CWR_ERR_SHAPE;
    if (R > 0 && mode == CWR_MODE_FUSED && !lse) return CWR_ERR_NULL;
    if (misaligned(rowinfo, 8) || misaligned(grads, 8) || misaligned(lse, 4) || misaligned(grad_costs, 4) ||
        misaligned(grad_x, elem_size(dtype)))
        return CWR_ERR_ALIGN;
    // no status word here: the forward pass has already flagged bad labels
    Batch b = make_batch(x, dtype, R, V, lx, ly, y, y_stride, y_len, N, blank, mode, 0, row_off, lab_off,
                         nullptr, stream);
    GradOut go;
    go.p = grad_costs; go.stride = grad_stride; go.scale = grad_scale;
    return launch_grad(b, rowinfo, grads, lse, go, grad_x);
}

int cwr_rowinfo(const int32_t* lx, const int32_t* ly, const int32_t* y, int64_t y_stride, int64_t y_len,
                int64_t N, int64_t R, int64_t V, const int64_t* row_off, const int64_t* lab_off,
                int32_t* rowinfo, void* stream) {
    if (N < 0 || R < 0 || V < 1 || y_len < 0) return CWR_ERR_SHAPE;
    if (N > 0x3fffffff || V > 0x3fffffff) return CWR_ERR_TOO_LARGE;
    if (R > 0 && N == 0) return CWR_ERR_SHAPE;
    if ((N > 0 && (!lx || !ly)) || (y_len > 0 && !y) || !row_off || !lab_off || (R > 0 && !rowinfo))
        return CWR_ERR_NULL;
    if (misaligned(lx, 4) || misaligned(ly, 4) || misaligned(y, 4) || misaligned(row_off, 8) ||
        misaligned(lab_off, 8) || misaligned(rowinfo, 8))
        return CWR_ERR_ALIGN;
    Batch b = make_batch(nullptr, CWR_F32, R, V, lx, ly, y, y_stride, y_len, N, 0, CWR_MODE_LOGPROB, 0,
                         row_off, lab_off, nullptr, stream);
    return launch_rowinfo(b, rowinfo);
}

int cwr_export_lattice(const int32_t* lx, const int32_t* ly, int64_t N, int64_t R, int64_t max_u,
                       const void* workspace, size_t workspace_bytes_, int64_t T_pad, int64_t Up_pad,
                       double* alphas, double* betas, void* stream) {
    if (N < 0 || R < 0 || max_u < 0 || T_pad < 0 || Up_pad < 0) return CWR_ERR_SHAPE;
    if (N > 0x3fffffff || T_pad > 0x3fffffff || Up_pad > 0x3fffffff) return CWR_ERR_TOO_LARGE;
    if (!workspace || (N > 0 && (!lx || !ly))) return CWR_ERR_NULL;
    if (!alphas && !betas) return CWR_ERR_NULL;
    if (misaligned(lx, 4) || misaligned(ly, 4) || misaligned(alphas, 8) || misaligned(betas, 8) ||
        misaligned(workspace, 256))
        return CWR_ERR_ALIGN;
    Workspace ws;
    if (!carve_workspace(const_cast<void*>(workspace), workspace_bytes_, N, R, max_u, &ws)) return CWR_ERR_SHAPE;
    return launch_export(lx, ly, (int)N, T_pad, Up_pad, ws, alphas, betas, static_cast<hipStream_t>(stream));
}

static int repack_impl(const void* src, void* dst, int dtype, int64_t N, int64_t T_pad, int64_t Up_pad, int64_t V,
                       const int32_t* lx, const int32_t* ly, const int64_t* row_off, int64_t R, int32_t* status,
                       void* stream, bool unpack) {
    if (dtype < CWR_F32 || dtype > CWR_F64) return CWR_ERR_DTYPE;
    if (N < 0 || T_pad < 0 || Up_pad < 0 || V < 1 || R < 0) return CWR_ERR_SHAPE;
    if (N > 0x3fffffff || V > 0x3fffffff || T_pad > 0x3fffffff || Up_pad > 0x3fffffff) return CWR_ERR_TOO_LARGE;
    const bool any_padded = N > 0 && T_pad > 0 && Up_pad > 0;
    if (N > 0 && (!lx || !ly || !row_off)) return CWR_ERR_NULL;
    if (any_padded && (unpack ? !dst : !src)) return CWR_ERR_NULL;
    if (R > 0 && (unpack ? !src : !dst)) return CWR_ERR_NULL;
    if (misaligned(src, elem_size(dtype)) || misaligned(dst, elem_size(dtype)) || misaligned(lx, 4) ||
        misaligned(ly, 4) || misaligned(row_off, 8) || misaligned(status, 4))
        return CWR_ERR_ALIGN;
    return launch_repack(src, dst, elem_size(dtype), lx, ly, reinterpret_cast<const i64*>(row_off), N, T_pad, Up_pad,
                         V, R, unpack, status, static_cast<hipStream_t>(stream));
}

int cwr_pack(const void* x_padded, int dtype, int64_t N, int64_t T_pad, int64_t Up_pad, int64_t V,
             const int32_t* lx, const int32_t* ly, const int64_t* row_off, int64_t R, void* x_compact,
             int32_t* status, void* stream) {
    return repack_impl(x_padded, x_compact, dtype, N, T_pad, Up_pad, V, lx, ly, row_off, R, status, stream, false);
}

int cwr_unpack(const void* g_compact, int dtype, int64_t N, int64_t T_pad, int64_t Up_pad, int64_t V,
               const int32_t* lx, const int32_t* ly, const int64_t* row_off, int64_t R, void* g_padded,
               void* stream) {
    return repack_impl(g_compact, g_padded, dtype, N, T_pad, Up_pad, V, lx, ly, row_off, R, nullptr, stream, true);
}

static int join_check(int dtype, int act, int64_t N, int64_t T_pad, int64_t Up_pad, int64_t H, int64_t R,
                      const int32_t* lx, const int32_t* ly, const int64_t* row_off) {
    if (dtype < CWR_F32 || dtype > CWR_F64) return CWR_ERR_DTYPE;
    if (act < CWR_ACT_NONE || act > CWR_ACT_RELU) return CWR_ERR_MODE;
    if (N < 0 || T_pad < 0 || Up_pad < 0 || H < 1 || R < 0) return CWR_ERR_SHAPE;
    if (N > 0x3fffffff || H > 0x3fffffff || T_pad > 0x3fffffff || Up_pad > 0x3fffffff) return CWR_ERR_TOO_LARGE;
    if (N > 0 && (!lx || !ly || !row_off)) return CWR_ERR_NULL;
    if (misaligned(lx, 4) || misaligned(ly, 4) || misaligned(row_off, 8)) return CWR_ERR_ALIGN;
    return CWR_OK;
}

int cwr_join(const void* f, const void* g, int dtype, int act, int64_t N, int64_t T_pad, int64_t Up_pad, int64_t H,
             const int32_t* lx, const int32_t* ly, const int64_t* row_off, int64_t R, void* h, int32_t* status,
             void* stream) {
    int rc = join_check(dtype, act, N, T_pad, Up_pad, H, R, lx, ly, row_off);
    if (rc != CWR_OK) return rc;
    if (N > 0 && T_pad > 0 && Up_pad > 0 && (!f || !g)) return CWR_ERR_NULL;
    if (R > 0 && !h) return CWR_ERR_NULL;
    const size_t es = elem_size(dtype);
    if (misaligned(f, es) || misaligned(g, es) || misaligned(h, es) || misaligned(status, 4)) return CWR_ERR_ALIGN;
    return launch_join(dtype, act, false, f, g, h, nullptr, lx, ly, reinterpret_cast<const i64*>(row_off), N, T_pad,
                       Up_pad, H, R, status, static_cast<hipStream_t>(stream));
}

int cwr_join_backward(const void* dh, const void* h, int dtype, int act, int64_t N, int64_t T_pad, int64_t Up_pad,
                      int64_t H, const int32_t* lx, const int32_t* ly, const int64_t* row_off, int64_t R, void* df,
                      void* dg, void* stream) {
    int rc = join_check(dtype, act, N, T_pad, Up_pad, H, R, lx, ly, row_off);
    if (rc != CWR_OK) return rc;
    if (R > 0 && (!dh || (act != CWR_ACT_NONE && !h))) return CWR_ERR_NULL;
    if (N > 0 && ((T_pad > 0 && !df) || (Up_pad > 0 && !dg))) return CWR_ERR_NULL;
    const size_t es = elem_size(dtype);
    if (misaligned(dh, es) || misaligned(h, es) || misaligned(df, es) || misaligned(dg, es)) return CWR_ERR_ALIGN;
    return launch_join(dtype, act, true, dh, h, df, dg, lx, ly, reinterpret_cast<const i64*>(row_off), N, T_pad,
                       Up_pad, H, R, nullptr, static_cast<hipStream_t>(stream));
}

}  // extern "C"
