// C ABI of the gfx950 GPT-OSS attention library (declared in include/gptoss_attn.h):
// host-side argument validation, launch geometry, and the kernel launches.
// No torch headers, no allocation; the only process-wide state is three per-device caches that are
// written once (compute-unit count, the window kernel's LDS attribute, the address of the built-in scratch).
#include <hip/hip_runtime.h>

#include <atomic>

#include "../../include/gptoss_attn.h"
#include "attn_bwd.h"
#include "attn_bwd_dkdv64.h"
#include "attn_bwd_window.h"
#include "attn_common.h"
#include "attn_f32.h"
#include "attn_fwd.h"
#include "attn_fwd_pipe.h"
#include "attn_fwd_window.h"
#include "mfma_rate.h"

using namespace gptoss;

namespace {

bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// A tensor's rows must start on 16-byte boundaries for the 128-bit accesses.
int check_tensor(const void *p, const gptoss_attn_strides &s, int elem_bytes, int D) {
    if (!p) return GPTOSS_ATTN_ERR_NULL_TENSOR;
    if (!aligned16(p)) return GPTOSS_ATTN_ERR_ALIGNMENT;
    const int64_t per16 = 16 / elem_bytes;
    if (s.b % per16 || s.h % per16 || s.s % per16) return GPTOSS_ATTN_ERR_ALIGNMENT;
    if (s.s < D || s.s > (1 << 24)) return GPTOSS_ATTN_ERR_STRIDE;   // 64 rows x stride is kept in 32 bits by the tile copies
    return GPTOSS_ATTN_OK;
}

Strides cvt(const gptoss_attn_strides &s) { return Strides{s.b, s.h, s.s}; }

// A window that reaches back past the first key from every query position is no window: such a
// call is the full-causal layer and takes exactly its kernels (same bits).
// (Not decidable on the host when the query offset lives in device memory.)
int effective_window(const gptoss_attn_params *p) {
    if (p->q_offset_dev) return p->window;
    return (p->window > 0 && (int64_t)p->window >= (int64_t)p->Sq + p->q_offset) ? 0 : p->window;
}

// Scratch layout: the fp32 row statistics (-delta, then lse * log2 e: 8 bytes per row, rounded up to 16
// bytes), the same statistics in split form (16 bytes per row), then the dK/dV partial sums.
size_t fp32_stats_bytes(const gptoss_attn_params *p) {
    const size_t n = (size_t)2 * sizeof(float) * (size_t)p->B * (size_t)p->H * (size_t)p->Sq;
    return (n + 15) & ~(size_t)15;
}

KArgs make_args(const gptoss_attn_params *p) {
    KArgs a{};
    a.q = static_cast<const bf16 *>(p->q);
    a.k = static_cast<const bf16 *>(p->k);
    a.v = static_cast<const bf16 *>(p->v);
    a.sinks = p->sinks;
    a.seqlens = p->seqlens;
    a.doc_start = p->doc_start;
    a.o = static_cast<bf16 *>(p->o);
    a.lse = p->lse;
    a.d_o = static_cast<const bf16 *>(p->d_o);
    a.dq = static_cast<bf16 *>(p->dq);
    a.dk = static_cast<bf16 *>(p->dk);
    a.dv = static_cast<bf16 *>(p->dv);
    a.dsinks = p->dsinks;
    a.delta = p->delta;
    a.split = reinterpret_cast<u32x4 *>(reinterpret_cast<char *>(p->delta) + fp32_stats_bytes(p));
    a.qs = cvt(p->q_stride); a.ks = cvt(p->k_stride); a.vs = cvt(p->v_stride); a.os = cvt(p->o_stride);
    a.dos = cvt(p->do_stride); a.dqs = cvt(p->dq_stride); a.dks = cvt(p->dk_stride); a.dvs = cvt(p->dv_stride);
    a.B = p->B; a.H = p->H; a.G = p->G; a.Sq = p->Sq; a.Skv = p->Skv;
    a.r = p->H / p->G;
    a.window = effective_window(p);
    a.q_offset = p->q_offset_dev ? 0 : p->q_offset;
    a.q_offset_dev = p->q_offset_dev;
    a.scale = p->scale;
    a.scale_log2 = p->scale * kLog2e;
    a.dkdv_parts = 1;
    a.chunk_tiles = 0;
    a.dsink_partial = nullptr;
    a.boundary_partial = nullptr;
    return a;
}

int hpb_for(int r) { return r >= 4 ? 4 : (r >= 2 ? 2 : 1); }

// 32-row query blocks per wavefront in the forward and dQ kernels.  Two blocks (64 rows)
// halve the LDS fragment traffic per MFMA and win on long key loops (full-causal layers);
// one block (32 rows, three wavefronts per SIMD) wastes less of the narrow band of a
// sliding-window layer and hides its short loops' latency better.
int query_blocks_for(int window) { return (window > 0 && window <= 1024) ? 1 : 2; }

// 32-key blocks per wavefront in the dK/dV kernel
constexpr int kDkdvNB = 1;
constexpr int kDkdvWaves = 4;                        // wavefronts per dK/dV workgroup
constexpr int kDkdvKeys = 32 * kDkdvNB * kDkdvWaves; // keys per dK/dV workgroup

// Workgroups per key block in the dK/dV kernel.  One workgroup per (batch, KV head, 128 keys) fills
// the 256 CUs (two workgroups each) only from S = 16384 on, and the causal triangle makes the first
// key blocks many times longer than the last; shorter problems cut each key block's query tiles into
// slices so that there are about a thousand workgroups, and sum the slices' fp32 partials afterwards.
// A slice keeps at least four query tiles (sliding-window layers are never cut).
int dkdv_parts_for(const gptoss_attn_params *p) {
    if (p->dtype != GPTOSS_ATTN_BF16) return 1;
    const int64_t blocks = (int64_t)p->G * p->B * ((p->Skv + kDkdvKeys - 1) / kDkdvKeys);
    int parts = (int)(1024 / (blocks > 0 ? blocks : 1));
    const int window = effective_window(p);
    const int64_t rows_seen = window > 0 ? (int64_t)kDkdvKeys + window - 1 : (int64_t)p->Sq;
    const int tiles = (int)((rows_seen < p->Sq ? rows_seen : p->Sq) + 63) / 64;
    if (parts > tiles / 4) parts = tiles / 4;
    if (parts > 8) parts = 8;
    return parts < 1 ? 1 : parts;
}

// Full-causal self-attention goes to attn_bwd_dkdv64_kernel (64 keys per wavefront, one wavefront per SIMD)
// when the shape is the one it is written for (bf16, no window, no packed rows, no offset, Sq == Skv a
// multiple of 64; right-padded batch rows are fine) and there is enough of it: more than 512 key blocks of 128 (then key blocks are
// whole: at least 257 workgroups of 256 keys, and the same bits as the 32-key kernel), or rows of 2048 keys
// or more that the host cuts into `parts` slices anyway (the same number of slices as the 32-key kernel
// would get, so the scratch is the same; -15 % at S = 2048 ... 8192).
// (The kernel walks Q, dO and the row statistics of one KV head's group of query heads with 32-bit byte
// offsets from the group's first row: head strides must not be negative and the group's span must stay
// below 2^31 bytes; anything else takes the 32-key kernel.)
bool walk_fits_32_bits(const gptoss_attn_strides &s, int64_t heads, int64_t rows) {
    return s.h >= 0 && ((heads - 1) * s.h + rows * s.s) * 2 < ((int64_t)1 << 31);
}
bool dkdv64_route(const gptoss_attn_params *p, int parts) {
    const int64_t blocks = (int64_t)p->G * p->B * ((p->Skv + kDkdvKeys - 1) / kDkdvKeys);
    const int64_t heads = p->H / p->G;
    if (!walk_fits_32_bits(p->q_stride, heads, p->Sq) || !walk_fits_32_bits(p->do_stride, heads, p->Sq) ||
        heads * p->Sq * 16 >= ((int64_t)1 << 31))
        return false;
    return p->dtype == GPTOSS_ATTN_BF16 && effective_window(p) == 0 && !p->doc_start && p->q_offset == 0 &&
           !p->q_offset_dev && p->Sq == p->Skv && p->Sq % kTile == 0 && (blocks > 512 || (parts > 1 && p->Skv >= 2048));
}

// The hand-pipelined forward kernel (attn_fwd_pipe.h) takes the plain full-causal case (right-padded batch rows
// included): every key tile but the last of a row is interior, all four wavefronts have a head.
bool fwd_pipe_route(const gptoss_attn_params *p) {
    return p->dtype == GPTOSS_ATTN_BF16 && effective_window(p) == 0 && !p->doc_start && p->q_offset == 0 &&
           !p->q_offset_dev && p->Sq == p->Skv && p->Sq % kTile == 0 && (p->H / p->G) % 4 == 0;
}

// The one-pass forward of sliding-window layers (attn_fwd_window.h): a window of 32, 64, 96 or 128 keys on plain
// self-attention rows (no offset, no packed rows; right-padded batch rows are fine) whose padded length is a
// multiple of 32, all four wavefronts of a workgroup with a head of their own.
bool fwd_window_route(const gptoss_attn_params *p) {
    const int w = effective_window(p);
    // lane offsets are 32-bit: up to 160 rows of K / V, 32 of Q and O; the grid's y and z dimensions end at 65535
    const int64_t row_limit = (int64_t)1 << 22;
    if (p->k_stride.s >= row_limit || p->v_stride.s >= row_limit || p->q_stride.s >= row_limit || p->o_stride.s >= row_limit) return false;
    if ((int64_t)(p->H / p->G / 4) * p->B > 65535 || p->Sq / 32 > 65535) return false;
    return p->dtype == GPTOSS_ATTN_BF16 && w >= 32 && w <= 128 && w % 32 == 0 && !p->doc_start &&
           p->q_offset == 0 && !p->q_offset_dev && p->Sq == p->Skv && p->Sq % 32 == 0 && (p->H / p->G) % 4 == 0;
}

// workgroups of four independent wavefronts for the float32 kernels
int64_t f32_grid(int64_t waves) { return (waves + 3) / 4; }

// One launch.  hipLaunchKernel reports this launch's own status, so an error some earlier call of the
// thread left in the runtime's sticky state is neither reported here nor cleared.  A grid beyond the
// x-dimension limit is refused on the host.
template <typename Kernel>
int launch(Kernel kernel, int64_t workgroups, int threads, hipStream_t st, const KArgs &a, size_t dynamic_lds = 0) {
    if (workgroups <= 0 || workgroups > 0x7fffffff) return GPTOSS_ATTN_ERR_SHAPE;
    void *args[] = {const_cast<KArgs *>(&a)};
    const hipError_t e = hipLaunchKernel(reinterpret_cast<const void *>(kernel), dim3((unsigned)workgroups), dim3((unsigned)threads),
                                         args, dynamic_lds, st);
    return e == hipSuccess ? GPTOSS_ATTN_OK : static_cast<int>(e);
}

// The same for a three-dimensional grid of 256-thread workgroups (the caller has checked the y and z limits).
template <typename Kernel>
int launch3(Kernel kernel, dim3 grid, hipStream_t st, const KArgs &a) {
    if (grid.x == 0 || grid.y == 0 || grid.z == 0 || grid.y > 65535 || grid.z > 65535) return GPTOSS_ATTN_ERR_SHAPE;
    void *args[] = {const_cast<KArgs *>(&a)};
    const hipError_t e = hipLaunchKernel(reinterpret_cast<const void *>(kernel), grid, dim3(256), args, 0, st);
    return e == hipSuccess ? GPTOSS_ATTN_OK : static_cast<int>(e);
}

// ---- single-pass backward of sliding-window layers (attn_bwd_window.h) ------------------------
// Taken for bf16 self-attention (Sq == Skv, no offset, no packed rows) with a window of at most
// 128 and 2..16 query heads per KV head (WinCfg::kMaxGroup: the kernel's LDS holds dSinks slots for
// that many); everything else keeps the dK/dV + dQ kernel pair.
bool window_single_pass(const gptoss_attn_params *p) {
    const int r = p->G > 0 ? p->H / p->G : 0;
    const int window = effective_window(p);
    return p->dtype == GPTOSS_ATTN_BF16 && window > 0 && window <= WinCfg::kMaxWindow && !p->doc_start &&
           p->q_offset == 0 && !p->q_offset_dev && p->Sq == p->Skv && r >= 2 && r <= WinCfg::kMaxGroup;
}

constexpr int kMaxDevices = 64;

// Compute units of the current device (looked up once per device).
int compute_units() {
    static std::atomic<int> cus[kMaxDevices];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return 256;
    int n = cus[dev].load(std::memory_order_acquire);
    if (n <= 0) {
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
        cus[dev].store(n, std::memory_order_release);
    }
    return n;
}

// Query tiles per workgroup: about one workgroup per compute unit, between 2 and 16 tiles (each
// workgroup walks two tiles beyond its own, so short chunks repeat more work).
int window_chunk_tiles(const gptoss_attn_params *p, int cus) {
    const int64_t tiles = (int64_t)((p->Sq + kTile - 1) / kTile) * p->G * p->B;
    int64_t c = tiles / (cus > 0 ? cus : 256);
    return (int)(c < 2 ? 2 : (c > 16 ? 16 : c));
}

// A kernel that uses more than 64 KB of LDS has to be told so once per device.
int window_lds_attribute() {
    static std::atomic<bool> done[kMaxDevices];
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return static_cast<int>(e);
    const bool tracked = dev >= 0 && dev < kMaxDevices;
    if (!tracked || !done[dev].load(std::memory_order_acquire)) {
        e = hipFuncSetAttribute(reinterpret_cast<const void *>(attn_bwd_window_kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                WinCfg::kLdsBytes);
        if (e != hipSuccess) return static_cast<int>(e);
        if (tracked) done[dev].store(true, std::memory_order_release);
    }
    return GPTOSS_ATTN_OK;
}

// Scratch of the single-pass window backward: dSinks partial sums [B][chunk][H][2], then (rounded up
// to 16 bytes) the fp32 dK / dV shares of the two key tiles on each seam between chunks.
struct WindowScratch { int chunk_tiles, n_chunks; size_t sink_bytes, seam_bytes; };

WindowScratch window_scratch_for(const gptoss_attn_params *p, int chunk_tiles) {
    WindowScratch w;
    w.chunk_tiles = chunk_tiles;
    const int n_tiles = (p->Sq + kTile - 1) / kTile;
    w.n_chunks = (n_tiles + w.chunk_tiles - 1) / w.chunk_tiles;
    w.sink_bytes = (((size_t)p->B * w.n_chunks * p->H * WinCfg::NHELP * sizeof(float)) + 15) & ~(size_t)15;
    w.seam_bytes = (size_t)p->B * p->G * (w.n_chunks - 1) * 2 * 2 * (2 * kTile * kD) * sizeof(float);
    return w;
}

WindowScratch window_scratch(const gptoss_attn_params *p, int cus) { return window_scratch_for(p, window_chunk_tiles(p, cus)); }

// seam_sums: neighbouring chunks exchange fp32 shares through the scratch (needs window_scratch bytes);
// otherwise each chunk walks two query tiles past its end and nothing but the dSinks sums is kept.
int launch_window_bwd(const gptoss_attn_params *p, hipStream_t st, bool seam_sums) {
    int rc = window_lds_attribute();
    if (rc) return rc;
    KArgs a = make_args(p);
    const WindowScratch ws = window_scratch(p, compute_units());
    a.chunk_tiles = ws.chunk_tiles;
    a.dsink_partial = p->delta;
    if (seam_sums && ws.n_chunks > 1)
        a.boundary_partial = reinterpret_cast<float *>(reinterpret_cast<char *>(p->delta) + ws.sink_bytes);
    rc = launch(attn_bwd_window_kernel, (int64_t)a.G * a.B * ws.n_chunks, 64 * WinCfg::NWAVES, st, a, WinCfg::kLdsBytes);
    if (rc) return rc;
    // seam tiles and dSinks in one small launch
    const int64_t seam_chunks = a.boundary_partial ? (int64_t)a.B * a.G * (ws.n_chunks - 1) * 2 * 2 * kTile * 8 : 0;
    const int seam_blocks = (int)((seam_chunks + 255) / 256);
    const int sink_blocks = a.dsinks ? a.H : 0;
    if (seam_blocks + sink_blocks == 0) return GPTOSS_ATTN_OK;
    int n_chunks = ws.n_chunks, sb = seam_blocks;
    void *args[] = {&a, &n_chunks, &sb};
    const hipError_t e = hipLaunchKernel(reinterpret_cast<const void *>(attn_bwd_window_finish_kernel),
                                         dim3((unsigned)(seam_blocks + sink_blocks)), dim3(256), args, 0, st);
    return e == hipSuccess ? GPTOSS_ATTN_OK : static_cast<int>(e);
}

// workgroups of the forward / dQ launch: (KV head, chunk of HPB query heads, batch, query tile)
int64_t q_outer_grid(const KArgs &a, int hpb, int qb) {
    const int bm = 32 * qb * (4 / hpb);
    const int n_hc = (a.r + hpb - 1) / hpb;
    return (int64_t)a.G * n_hc * a.B * ((a.Sq + bm - 1) / bm);
}

// one launch of a synthetic instruction stream (mfma_rate.h): one workgroup per compute unit
template <int MIX>
int64_t launch_stream_probe(int waves_per_simd, int iters, float *sink, hipStream_t st) {
    const void *fn = reinterpret_cast<const void *>(stream_probe_kernel<MIX>);
    hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, kStreamProbeLdsBytes);
    if (e != hipSuccess) return -static_cast<int64_t>(e) - 1000;
    const int blocks = compute_units();
    void *args[] = {&sink, &iters};
    e = hipLaunchKernel(fn, dim3((unsigned)blocks), dim3(256u * waves_per_simd), args, kStreamProbeLdsBytes, st);
    if (e != hipSuccess) return -static_cast<int64_t>(e) - 1000;
    return (int64_t)blocks * 4 * waves_per_simd * iters * kStreamProbeMfmas;     // MFMA instructions the launch executes
}

}  // namespace

extern "C" {

int gptoss_attn_version(void) { return GPTOSS_ATTN_ABI_VERSION; }

const char *gptoss_attn_status_string(int status) {
    switch (status) {
        case GPTOSS_ATTN_OK: return "ok";
        case GPTOSS_ATTN_ERR_NULL_PARAMS: return "params pointer is NULL";
        case GPTOSS_ATTN_ERR_NULL_TENSOR: return "a required tensor pointer is NULL";
        case GPTOSS_ATTN_ERR_HEAD_DIM: return "head_dim must be 64";
        case GPTOSS_ATTN_ERR_HEADS: return "H and G must be positive and H divisible by G";
        case GPTOSS_ATTN_ERR_SHAPE: return "B, Sq, Skv must be positive; window, q_offset non-negative; positions and window at most 2^30; scale positive and finite; doc_start needs Sq == Skv and q_offset == 0; at most 2^31-1 workgroups";
        case GPTOSS_ATTN_ERR_DTYPE: return "unsupported dtype";
        case GPTOSS_ATTN_ERR_ALIGNMENT: return "tensor base or stride is not 16-byte aligned";
        case GPTOSS_ATTN_ERR_STRIDE: return "sequence stride smaller than head_dim or larger than 2^24 elements";
        case GPTOSS_ATTN_ERR_ABI: return "struct_size does not match this library";
        case GPTOSS_ATTN_ERR_WORKSPACE: return "the problem needs more scratch than the library's built-in array holds (gptoss_attn_static_scratch_bytes)";
        default: return status > 0 ? "HIP runtime error (status is the hipError_t)" : "unknown status";
    }
}

int gptoss_attn_validate(const gptoss_attn_params *p, int need_bwd) {
    if (!p) return GPTOSS_ATTN_ERR_NULL_PARAMS;
    if (p->struct_size != sizeof(gptoss_attn_params)) return GPTOSS_ATTN_ERR_ABI;
    if (p->dtype != GPTOSS_ATTN_BF16 && p->dtype != GPTOSS_ATTN_FP32) return GPTOSS_ATTN_ERR_DTYPE;
    if (p->D != kD) return GPTOSS_ATTN_ERR_HEAD_DIM;
    if (p->H <= 0 || p->G <= 0 || p->H % p->G) return GPTOSS_ATTN_ERR_HEADS;
    if (p->B <= 0 || p->Sq <= 0 || p->Skv <= 0 || p->window < 0 || (!p->q_offset_dev && p->q_offset < 0)) return GPTOSS_ATTN_ERR_SHAPE;
    // positions are 32-bit in the kernels and +-2^30 marks "no window" / "dead row"
    if ((int64_t)p->Sq + (p->q_offset_dev ? 0 : p->q_offset) > (1 << 30) || p->Skv > (1 << 30) || p->window > (1 << 30)) return GPTOSS_ATTN_ERR_SHAPE;
    if (!(p->scale > 0.0f) || !(p->scale < 3.0e38f)) return GPTOSS_ATTN_ERR_SHAPE;
    if (p->doc_start && (p->Sq != p->Skv || p->q_offset != 0 || p->q_offset_dev)) return GPTOSS_ATTN_ERR_SHAPE;
    if (p->q_offset_dev && (reinterpret_cast<uintptr_t>(p->q_offset_dev) & 3)) return GPTOSS_ATTN_ERR_ALIGNMENT;
    const int eb = p->dtype == GPTOSS_ATTN_FP32 ? 4 : 2;
    int rc;
    if ((rc = check_tensor(p->q, p->q_stride, eb, p->D))) return rc;
    if ((rc = check_tensor(p->k, p->k_stride, eb, p->D))) return rc;
    if ((rc = check_tensor(p->v, p->v_stride, eb, p->D))) return rc;
    if ((rc = check_tensor(p->o, p->o_stride, eb, p->D))) return rc;
    if (!p->lse) return GPTOSS_ATTN_ERR_NULL_TENSOR;
    if (need_bwd) {
        if ((rc = check_tensor(p->d_o, p->do_stride, eb, p->D))) return rc;
        if ((rc = check_tensor(p->dq, p->dq_stride, eb, p->D))) return rc;
        if ((rc = check_tensor(p->dk, p->dk_stride, eb, p->D))) return rc;
        if ((rc = check_tensor(p->dv, p->dv_stride, eb, p->D))) return rc;
        if (!p->delta) return GPTOSS_ATTN_ERR_NULL_TENSOR;
        if (!aligned16(p->delta)) return GPTOSS_ATTN_ERR_ALIGNMENT;   // the dK/dV partial sums use 16-byte accesses
    }
    return GPTOSS_ATTN_OK;
}

// Bytes of the row-statistics part of the scratch; dK/dV partials follow.
static size_t stats_bytes(const gptoss_attn_params *p) {
    return fp32_stats_bytes(p) + (size_t)16 * (size_t)p->B * (size_t)p->H * (size_t)p->Sq;
}

size_t gptoss_attn_workspace_bytes(const gptoss_attn_params *p) {
    if (!p || p->B <= 0 || p->H <= 0 || p->Sq <= 0) return 0;
    size_t n = stats_bytes(p);
    if (p->G > 0 && p->Skv > 0) {
        const int parts = dkdv_parts_for(p);
        if (parts > 1) n += (size_t)parts * 2 * sizeof(float) * (size_t)p->B * (size_t)p->G * (size_t)p->Skv * kD;
        if (window_single_pass(p)) {
            // gptoss_attn_bwd takes this route and lays its own scratch over the same bytes.  The layout
            // follows the compute-unit count of the device that is current at launch time; the size
            // returned is that of the shortest chunks (the most seams), which covers every device.
            const WindowScratch ws = window_scratch_for(p, 2);
            if (ws.sink_bytes + ws.seam_bytes > n) n = ws.sink_bytes + ws.seam_bytes;
        }
    }
    return n;
}

int gptoss_attn_fwd(const gptoss_attn_params *p, void *stream) {
    const int rc = gptoss_attn_validate(p, 0);
    if (rc) return rc;
    const KArgs a = make_args(p);
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (p->dtype == GPTOSS_ATTN_FP32)
        return launch(attn_f32_fwd_kernel, f32_grid((int64_t)a.B * a.H * ((a.Sq + 31) / 32)), 256, st, a);
    const int hpb = hpb_for(a.r), qb = query_blocks_for(a.window);
    const int64_t grid = q_outer_grid(a, hpb, qb);
    if (fwd_window_route(p)) {
        // two 32-row query blocks per workgroup (K / V rows staged once for both) where that still leaves every compute
        // unit several rounds of workgroups, else one
        const int64_t pairs = (int64_t)a.G * (a.r / 4) * a.B * ((a.Sq + 63) / 64);
        const bool by_pairs = a.Sq > 32 && pairs >= 8 * (int64_t)compute_units();
        const dim3 wgrid((unsigned)a.G, (unsigned)((a.r / 4) * a.B), (unsigned)(by_pairs ? (a.Sq + 63) / 64 : a.Sq / 32));
        switch (a.window / 32) {
            case 1: return launch3(attn_fwd_window_kernel<1>, wgrid, st, a);
            case 2: return launch3(attn_fwd_window_kernel<2>, wgrid, st, a);
            case 3: return launch3(attn_fwd_window_kernel<3>, wgrid, st, a);
            default: return launch3(attn_fwd_window_kernel<4>, wgrid, st, a);
        }
    }
    if (fwd_pipe_route(p)) return a.seqlens ? launch(attn_fwd_pipe_kernel<true>, grid, 256, st, a) : launch(attn_fwd_pipe_kernel<false>, grid, 256, st, a);
#define GPTOSS_LAUNCH_FWD(HPB, QB) launch(attn_fwd_kernel<HPB, QB>, grid, 256, st, a)
    if (qb == 2) return hpb == 4 ? GPTOSS_LAUNCH_FWD(4, 2) : hpb == 2 ? GPTOSS_LAUNCH_FWD(2, 2) : GPTOSS_LAUNCH_FWD(1, 2);
    return hpb == 4 ? GPTOSS_LAUNCH_FWD(4, 1) : hpb == 2 ? GPTOSS_LAUNCH_FWD(2, 1) : GPTOSS_LAUNCH_FWD(1, 1);
#undef GPTOSS_LAUNCH_FWD
}

int gptoss_attn_bwd_preprocess(const gptoss_attn_params *p, void *stream) {
    const int rc = gptoss_attn_validate(p, 1);
    if (rc) return rc;
    const KArgs a = make_args(p);
    hipStream_t st = static_cast<hipStream_t>(stream);
    const int64_t rows = (int64_t)a.B * a.H * a.Sq;
    int s = p->dtype == GPTOSS_ATTN_FP32 ? launch(attn_f32_delta_kernel, (rows + 15) / 16, 256, st, a)
                                         : launch(attn_bwd_delta_kernel, (rows + 127) / 128, 256, st, a);
    if (s == GPTOSS_ATTN_OK && a.dsinks) s = launch(attn_bwd_dsinks_kernel, a.H, 1024, st, a);
    return s;
}

// The dK/dV launch (and the sum of the partials when key blocks are cut).  whole_blocks: never cut a
// key block, so that nothing beyond the row statistics is kept in the scratch.
static int launch_dkdv(const gptoss_attn_params *p, void *stream, bool whole_blocks) {
    const int rc = gptoss_attn_validate(p, 1);
    if (rc) return rc;
    KArgs a = make_args(p);
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (p->dtype == GPTOSS_ATTN_FP32)
        return launch(attn_f32_dkdv_kernel, f32_grid((int64_t)a.B * a.G * ((a.Skv + 31) / 32)), 256, st, a);
    a.dkdv_parts = whole_blocks ? 1 : dkdv_parts_for(p);
    a.dkdv_partial = reinterpret_cast<float *>(reinterpret_cast<char *>(p->delta) + stats_bytes(p));
    if (dkdv64_route(p, a.dkdv_parts)) {
        const int64_t grid64 = (int64_t)a.G * a.B * a.dkdv_parts * ((a.Skv + Dkdv64::BN - 1) / Dkdv64::BN);
        const int s = a.seqlens ? launch(attn_bwd_dkdv64_kernel<true>, grid64, 256, st, a) : launch(attn_bwd_dkdv64_kernel<false>, grid64, 256, st, a);
        if (s || a.dkdv_parts == 1) return s;
        return launch(attn_bwd_dkdv_reduce_kernel, ((int64_t)2 * a.B * a.G * a.Skv * 8 + 255) / 256, 256, st, a);
    }
    const int64_t grid = (int64_t)a.G * a.B * a.dkdv_parts * ((a.Skv + kDkdvKeys - 1) / kDkdvKeys);
    const int s = a.doc_start ? launch(attn_bwd_dkdv_kernel<kDkdvWaves, kDkdvNB, true>, grid, 64 * kDkdvWaves, st, a)
                              : launch(attn_bwd_dkdv_kernel<kDkdvWaves, kDkdvNB, false>, grid, 64 * kDkdvWaves, st, a);
    if (s || a.dkdv_parts == 1) return s;
    const int64_t chunks = (int64_t)2 * a.B * a.G * a.Skv * 8;
    return launch(attn_bwd_dkdv_reduce_kernel, (chunks + 255) / 256, 256, st, a);
}

int gptoss_attn_bwd_dkdv(const gptoss_attn_params *p, void *stream) { return launch_dkdv(p, stream, false); }

// The dQ launch; fuse_delta: the kernel also produces the row statistics (see attn_bwd_dq_kernel).
static int launch_dq(const gptoss_attn_params *p, void *stream, int fuse_delta) {
    const int rc = gptoss_attn_validate(p, 1);
    if (rc) return rc;
    const KArgs a = make_args(p);
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (p->dtype == GPTOSS_ATTN_FP32)
        return launch(attn_f32_dq_kernel, f32_grid((int64_t)a.B * a.H * ((a.Sq + 31) / 32)), 256, st, a);
    const int hpb = hpb_for(a.r);
    int qb = query_blocks_for(a.window);
    // short problems: 64-row workgroups (two per compute unit) would be few and uneven (the key loops grow with the row
    // index); 32-row wavefronts make twice as many, three per SIMD (measured, full causal, B = 1: dQ 0.077 -> 0.066 ms
    // at S = 2048, 0.240 -> 0.218 at S = 4096, equal from S = 8192 on, 6 % slower at S = 16384)
    if (qb == 2 && q_outer_grid(a, hpb, 2) <= 4 * (int64_t)compute_units()) qb = 1;
    const int64_t grid = q_outer_grid(a, hpb, qb);
#define GPTOSS_LAUNCH_DQ(HPB, QB) \
    (fuse_delta ? launch(attn_bwd_dq_kernel<HPB, QB, true>, grid, 256, st, a) : launch(attn_bwd_dq_kernel<HPB, QB, false>, grid, 256, st, a))
    if (qb == 2) return hpb == 4 ? GPTOSS_LAUNCH_DQ(4, 2) : hpb == 2 ? GPTOSS_LAUNCH_DQ(2, 2) : GPTOSS_LAUNCH_DQ(1, 2);
    return hpb == 4 ? GPTOSS_LAUNCH_DQ(4, 1) : hpb == 2 ? GPTOSS_LAUNCH_DQ(2, 1) : GPTOSS_LAUNCH_DQ(1, 1);
#undef GPTOSS_LAUNCH_DQ
}

int gptoss_attn_bwd_dq(const gptoss_attn_params *p, void *stream) { return launch_dq(p, stream, 0); }

// The whole backward.  bf16: the dQ kernel computes the row statistics on the way (no separate
// pass over O and dO), then dSinks and dK/dV read them from the scratch buffer.  The results are
// bit-identical to gptoss_attn_bwd_preprocess + gptoss_attn_bwd_dkdv + gptoss_attn_bwd_dq.
static int bwd_all(const gptoss_attn_params *p, void *stream, bool whole_blocks) {
    int rc = gptoss_attn_validate(p, 1);
    if (rc) return rc;
    if (p->dtype == GPTOSS_ATTN_FP32) {
        rc = gptoss_attn_bwd_preprocess(p, stream);
        if (rc) return rc;
        rc = launch_dkdv(p, stream, whole_blocks);
        if (rc) return rc;
        return gptoss_attn_bwd_dq(p, stream);
    }
    if (window_single_pass(p)) return launch_window_bwd(p, static_cast<hipStream_t>(stream), !whole_blocks);
    rc = launch_dq(p, stream, 1);
    if (rc) return rc;
    if (p->dsinks) {
        const KArgs a = make_args(p);
        rc = launch(attn_bwd_dsinks_kernel, a.H, 1024, static_cast<hipStream_t>(stream), a);
        if (rc) return rc;
    }
    return launch_dkdv(p, stream, whole_blocks);
}

int gptoss_attn_bwd(const gptoss_attn_params *p, void *stream) { return bwd_all(p, stream, false); }

// ---- the backward for callers that cannot allocate ------------------------------------------
// Same kernels as gptoss_attn_bwd; the row statistics live in a device array that is part of the
// library image instead of a caller-provided workspace.  Each GPU has its own copy of the array
// at its own address, looked up once per device.
namespace {
constexpr size_t kStaticScratchBytes = GPTOSS_ATTN_STATIC_SCRATCH_BYTES;
}
static __device__ __align__(256) float scratch[kStaticScratchBytes / sizeof(float)];
static std::atomic<float *> scratch_ptr[kMaxDevices];     // device address of `scratch`, per device; NULL = not looked up yet

static int static_scratch(float **out) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return static_cast<int>(e);
    if (dev < 0 || dev >= kMaxDevices) return GPTOSS_ATTN_ERR_WORKSPACE;
    float *ptr = scratch_ptr[dev].load(std::memory_order_acquire);
    if (!ptr) {
        // with the device current, the symbol resolves to this device's copy; two threads racing
        // here look up the same address
        e = hipGetSymbolAddress(reinterpret_cast<void **>(&ptr), HIP_SYMBOL(scratch));
        if (e != hipSuccess) return static_cast<int>(e);
        if (!ptr) return GPTOSS_ATTN_ERR_WORKSPACE;
        scratch_ptr[dev].store(ptr, std::memory_order_release);
    }
    *out = ptr;
    return GPTOSS_ATTN_OK;
}

size_t gptoss_attn_static_scratch_bytes(void) { return kStaticScratchBytes; }

int gptoss_attn_bwd_static(const gptoss_attn_params *p, void *stream) {
    if (!p) return GPTOSS_ATTN_ERR_NULL_PARAMS;
    if (p->struct_size != sizeof(gptoss_attn_params)) return GPTOSS_ATTN_ERR_ABI;
    gptoss_attn_params q = *p;
    q.delta = reinterpret_cast<float *>(static_cast<uintptr_t>(256));   // stands in for the scratch while the other arguments are checked
    int rc = gptoss_attn_validate(&q, 1);
    if (rc) return rc;
    if (stats_bytes(&q) > kStaticScratchBytes) return GPTOSS_ATTN_ERR_WORKSPACE;
    rc = static_scratch(&q.delta);
    if (rc) return rc;
    return bwd_all(&q, stream, true);
}

// ---- measurement aid (mfma_rate.h) -----------------------------------------------------------
int64_t gptoss_attn_mfma_rate_probe(const void *operands, size_t operand_bytes, int iters, float *sink, size_t sink_floats,
                                    void *stream) {
    if (!operands || !sink || operand_bytes < 16 || iters <= 0 || !aligned16(operands)) return GPTOSS_ATTN_ERR_NULL_TENSOR;
    const int64_t blocks = (int64_t)2 * compute_units();       // two workgroups of four wavefronts per compute unit
    if ((size_t)blocks * 256 > sink_floats || operand_bytes / 16 > 0xffffffffu) return GPTOSS_ATTN_ERR_SHAPE;
    const u32x4 *ops = static_cast<const u32x4 *>(operands);
    uint32_t n_vec = (uint32_t)(operand_bytes / 16);
    void *args[] = {&ops, &n_vec, &iters, &sink};
    const hipError_t e = hipLaunchKernel(reinterpret_cast<const void *>(mfma_rate_kernel), dim3((unsigned)blocks), dim3(256), args, 0,
                                         static_cast<hipStream_t>(stream));
    if (e != hipSuccess) return -static_cast<int64_t>(e) - 1000;
    return blocks * 4 * (int64_t)iters * kMfmaRatePerIter;      // MFMA instructions the launch executes
}

int64_t gptoss_attn_stream_probe(int mix, int waves_per_simd, int iters, float *sink, size_t sink_floats, void *stream) {
    if (!sink || iters <= 0 || mix < 0 || mix >= kStreamMixes || waves_per_simd < 1 || waves_per_simd > 3) return GPTOSS_ATTN_ERR_SHAPE;
    if ((size_t)compute_units() * 256 * waves_per_simd > sink_floats) return GPTOSS_ATTN_ERR_SHAPE;
    hipStream_t st = static_cast<hipStream_t>(stream);
    switch (mix) {
        case kStreamMfmaOnly: return launch_stream_probe<kStreamMfmaOnly>(waves_per_simd, iters, sink, st);
        case kStreamFwdUniform: return launch_stream_probe<kStreamFwdUniform>(waves_per_simd, iters, sink, st);
        case kStreamFwdClumped: return launch_stream_probe<kStreamFwdClumped>(waves_per_simd, iters, sink, st);
        case kStreamDqUniform: return launch_stream_probe<kStreamDqUniform>(waves_per_simd, iters, sink, st);
        case kStreamDqClumped: return launch_stream_probe<kStreamDqClumped>(waves_per_simd, iters, sink, st);
        default: return launch_stream_probe<kStreamDkdvUniform>(waves_per_simd, iters, sink, st);
    }
}

}  // extern "C"
