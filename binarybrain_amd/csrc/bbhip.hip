// Host side of the C ABI declared in include/bbhip.h: argument checks, scratch management and kernel launches.
// The kernels themselves are in lut_kernels.hpp; the arithmetic they share in lut_math.hpp.

#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <map>
#include <mutex>
#include <string>
#include <vector>

#include "../../include/bbhip.h"
#include "lut_kernels.hpp"
#include "vector_kernels.hpp"
#include "conv_kernels.hpp"
#include "tail_kernels.hpp"
#include "bn_kernels.hpp"
#include "modulation_kernels.hpp"
#include "pooling_kernels.hpp"

using namespace bbhip;

// Scratch of bbhip_fp32_StochasticLut_Forward_NoAlloc: the transformed tables of one call (centred coefficients and, for
// binarized inputs, corner values).  One copy per GPU, held until the process ends; every call on a GPU shares it.
constexpr size_t kNoAllocScratchBytes = 8u << 20;
static __device__ __align__(256) unsigned char scratch[kNoAllocScratchBytes];

namespace {

// ------------------------------------------------------------------------------------------------
//  errors
// ------------------------------------------------------------------------------------------------
thread_local std::string g_last_error;

int fail(char const *fmt, ...)
{
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof(buf), fmt, ap);
    va_end(ap);
    g_last_error = buf;
    return 1;
}

#define BBHIP_TRY(expr)                                                                              \
    do {                                                                                             \
        hipError_t e_ = (expr);                                                                      \
        if (e_ != hipSuccess) { return fail("%s: %s (%s:%d)", #expr, hipGetErrorString(e_), __FILE__, __LINE__); } \
    } while (0)

#define BBHIP_REQUIRE(cond)                                                                          \
    do {                                                                                             \
        if (!(cond)) { return fail("%s: rejected argument: %s", __func__, #cond); }                  \
    } while (0)

#define BBHIP_LAUNCH_CHECK() BBHIP_TRY(hipGetLastError())

// ------------------------------------------------------------------------------------------------
//  global switches
// ------------------------------------------------------------------------------------------------
bool g_host_only = false;
int  g_dx_mode   = 0;
thread_local int g_input_node_hint = 0;      // bbhip_HintInputNodeSize: rows of the next forward call's input, 0 = unknown
// bbhip_HintPackedInput: a caller-owned buffer for the packed copy of the next LUT call's binarized fp32 input
struct PackedInputHint { uint32_t *bits; int rows, row_words, holds_input; };
thread_local PackedInputHint g_packed_hint = {nullptr, 0, 0, 0};
// hints are for the next LUT call only: every entry spends them
// bbhip_HintPreparedTables: a caller-owned place for the tables that a LUT call derives from W (centred coefficients, corner values)
struct PreparedTablesHint { float *buf; size_t bytes; int holds_tables; };
thread_local PreparedTablesHint g_tables_hint = {nullptr, 0, 0};
// bbhip_HintPackedOutput: a caller-owned buffer that receives the binarized output of the next forward call as packed bits
struct PackedOutputHint { uint32_t *bits; int rows, row_words; };
thread_local PackedOutputHint g_packed_out_hint = {nullptr, 0, 0};
// bbhip_HintTableGradientOverwrite: the next backward call writes dW instead of adding to it
thread_local int g_dw_overwrite_hint = 0;
static inline void clear_hints(void)
{
    g_dw_overwrite_hint = 0;
    g_input_node_hint = 0; g_packed_hint = PackedInputHint{nullptr, 0, 0, 0}; g_tables_hint = PreparedTablesHint{nullptr, 0, 0};
    g_packed_out_hint = PackedOutputHint{nullptr, 0, 0};
}
static inline bool tables_fit(PreparedTablesHint const &t, size_t bytes)
{
    return t.buf != nullptr && t.bytes >= bytes && (reinterpret_cast<uintptr_t>(t.buf) & 255u) == 0;
}

// ------------------------------------------------------------------------------------------------
//  optional kernel timer: HIP events around the dominant kernel of each entry point, on the launch stream
// ------------------------------------------------------------------------------------------------
enum TimedKernel : int { kTimeForward = 0, kTimeBackward = 1, kTimeBinary = 2, kTimeDx = 3, kTimeOther = 4, kTimedKinds = 5 };
struct TimedLaunch { hipEvent_t start, stop; int which; };
bool g_timer_on = false;
std::mutex g_timed_mtx;                      // guards g_timed: calls may come from several host threads
std::vector<TimedLaunch> g_timed;

struct ScopedTimer {
    hipStream_t st; bool on; TimedLaunch t;
    ScopedTimer(int which, hipStream_t s, bool allowed = true) : st(s), on(g_timer_on && allowed)
    {
        if (!on) { return; }
        t.which = which;
        if (hipEventCreate(&t.start) != hipSuccess || hipEventCreate(&t.stop) != hipSuccess) { on = false; return; }
        (void)hipEventRecord(t.start, st);
    }
    ~ScopedTimer()
    {
        if (!on) { return; }
        (void)hipEventRecord(t.stop, st);
        std::lock_guard<std::mutex> lk(g_timed_mtx);
        g_timed.push_back(t);
    }
};

// integer tunable from the environment: unset, empty or negative = the default
int env_int(char const *name, int def)
{
    char const *s = getenv(name);
    if (!s || !*s) { return def; }
    int v = atoi(s);
    return v >= 0 ? v : def;
}

// on/off switch from the environment: 0 (or 2, the older spelling) = off, any other number = on, unset = the default
bool env_switch(char const *name, bool def)
{
    char const *s = getenv(name);
    if (!s || !*s) { return def; }
    int v = atoi(s);
    return !(v == 0 || v == 2);
}

// two-valued inputs (packed bits, fp32 binarized at 0.5): the kernels that look the LUT output up among the node's corner values
bool use_corner_values(int xmode)
{
    static bool const on = env_switch("BBHIP_CORNER", true);
    return on && (xmode == kXBit || xmode == kXBinary);
}

bool pack_binarized_input(void) { static bool const on = env_switch("BBHIP_PACK", true); return on; }
// the corner-value forward kernel derives a node's tables in the wavefront where no packing launch carries the preparation (0 = a table launch)
bool inline_tables(void) { static bool const on = env_switch("BBHIP_INLINE_TABLES", true); return on; }
// packed rows in the dx kernel read with one scalar load per row and pass where pitch and alignment allow (0 = vector loads + read-lanes)
bool term_from_corner_values(void) { static bool const on = env_switch("BBHIP_TERM_NODES", true); return on; }
bool dx_indexed(void) { static bool const on = env_switch("BBHIP_DX_INDEXED", true); return on; }
bool dx_wide_rows(void) { static bool const on = env_switch("BBHIP_DX_WIDE", true); return on; }
int dx_wide_max_rows(void) { static int const v = env_int("BBHIP_DX_WIDE_ROWS", 1024); return v; }

// frames per unit; both are rounded to wavefront multiples where used
int fwd_nodes_per_wave(void) { static int v = env_int("BBHIP_FWD_NODES", 2); return v >= 2 ? 2 : 1; }
// Frames per forward unit.  fp32 rows are gathered through L2, and a 256-frame piece of every input row is what one XCD's L2
// holds; packed-bit rows are 32 times smaller, so their units are longer and a unit's set-up (wiring, table) weighs less.
// Longer units are halved while they would leave the launch with fewer than 2048 workgroups.
int fwd_chunk_frames_env(void) { static int env = env_int("BBHIP_FWD_CHUNK", 0); return env > 0 ? ((env + 63) / 64) * 64 : 0; }
int fwd_chunk_frames(int xmode, int frame_size, int tile_count)
{
    if (fwd_chunk_frames_env() > 0) { return fwd_chunk_frames_env(); }
    int chunk = (xmode == kXBit) ? 2048 : 256;
    while (chunk > 256 && (long long)((frame_size + chunk - 1) / chunk) * tile_count < 2048) {
        // ... but not past the number of units whose batch-norm partial sums the wavefronts add up themselves while the launch still
        // has a thousand workgroups: halving would bring the finalize launches back (5.6 us each) for a few idle compute units
        int const units = (frame_size + chunk - 1) / chunk;
        if (units <= kInlineStatUnits && 2 * units > kInlineStatUnits && (long long)units * tile_count >= 1024) { break; }
        chunk /= 2;
    }
    return chunk;
}
int bwd_slab_frames(void)  { static int v = env_int("BBHIP_BWD_SLAB", 0);  return ((v + 63) / 64) * 64; }       // 0: chosen per call
// dx units: frames per unit and wavefront-steps per pass over the work list.  128 frames in passes of two steps where the
// gathered rows are fp32 (what L2 holds); packed-bit rows leave room for 256 frames in passes of four, which halves the
// per-term set-up per frame.  0: not set in the environment.
int dx_chunk_frames_env(void) { static int v = env_int("BBHIP_DX_CHUNK", 0); return ((v + 63) / 64) * 64; }
int dx_pass_steps_env(void)   { static int v = env_int("BBHIP_DX_STEPS", 0); return (v <= 0) ? 0 : (v <= 1) ? 1 : (v <= 2) ? 2 : 4; }
// dx work lists split over the four wavefronts of a workgroup (DxArgs::split): where one wavefront per (input node, unit) would
// leave the launch with fewer than 4096 workgroups and the lists are long enough to share.  BBHIP_DX_SPLIT = 0 / 1 forces it.
bool dx_split_lists(int max_fan, long long workgroups)
{
    static int const env = env_int("BBHIP_DX_SPLIT", 2);
    if (env == 0 || env == 1) { return env == 1; }
    return max_fan >= 16 && workgroups < 4096;
}
// BinaryLut6 units of 128 words: 8192 input rows x 512 bytes is what an XCD's 4 MiB L2 holds (1.2 GB fetched per launch at
// the benchmark shape; 192-word units fetch 1.9 GB, 256-word units 2.3 GB).  With the per-wavefront set-up at its
// present cost the shorter units are also the fastest (241 us; 192 words 278 us, 256 words 332 us, 64 words 282 us).
int bin_chunk_words(void)  { static int v = env_int("BBHIP_BIN_CHUNK", 128); return (((v > 0 ? v : 128) + 63) / 64) * 64; }
int bin_nodes_per_wave(void) { static int v = env_int("BBHIP_BIN_NODES", 0); return v >= 4 ? 4 : v >= 2 ? 2 : v == 1 ? 1 : 0; }     // 0: chosen per call

// ------------------------------------------------------------------------------------------------
//  scratch arena: one growing device buffer per device, reused by every call
// ------------------------------------------------------------------------------------------------
constexpr int kMaxDevices = 64;
// Blocks that a growing arena has left behind stay allocated: kernels already queued and HIP graphs captured earlier hold
// their addresses.  bbhip_ReleaseScratch frees everything.
struct Arena { void *ptr = nullptr; size_t cap = 0; std::vector<void *> retired; };
Arena g_arena[kMaxDevices];

// Scratch for one call.  Either the library's arena (grown with hipMalloc where needed, never while the stream is being
// captured) or, for the entry point that must not allocate, a fixed block handed in by the caller of run_forward.
struct Scratch { char *fixed = nullptr; size_t fixed_cap = 0; };

int arena_get(size_t bytes, char **out, hipStream_t st, Scratch const *fixed = nullptr)
{
    if (fixed && fixed->fixed) {
        if (bytes > fixed->fixed_cap) { return fail("scratch of %zu bytes needed, the fixed block holds %zu", bytes, fixed->fixed_cap); }
        *out = fixed->fixed;
        return 0;
    }
    int dev = 0;
    BBHIP_TRY(hipGetDevice(&dev));
    if (dev < 0 || dev >= kMaxDevices) { return fail("device index %d out of range", dev); }
    Arena &a = g_arena[dev];
    if (a.cap < bytes) {
        hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
        if (hipStreamIsCapturing(st, &cap) == hipSuccess && cap != hipStreamCaptureStatusNone) {
            return fail("the scratch arena would have to grow from %zu to %zu bytes during stream capture: "
                        "run the call once outside the capture, or bbhip_ReserveScratch first", a.cap, bytes);
        }
        (void)hipGetLastError();
        size_t want = bytes + bytes / 2 + (1u << 20);
        void *p = nullptr;
        BBHIP_TRY(hipMalloc(&p, want));
        if (a.ptr) { a.retired.push_back(a.ptr); }
        a.ptr = p;
        a.cap = want;
    }
    *out = static_cast<char *>(a.ptr);
    return 0;
}

inline size_t align256(size_t v) { return (v + 255) & ~(size_t)255; }

inline int ceil_div(int a, int b) { return (a + b - 1) / b; }

// ------------------------------------------------------------------------------------------------
//  dispatch helpers
// ------------------------------------------------------------------------------------------------
#define BBHIP_SWITCH_N(n, EXPR)                       \
    switch (n) {                                      \
    case 2: { constexpr int N = 2; EXPR; } break;     \
    case 3: { constexpr int N = 3; EXPR; } break;     \
    case 4: { constexpr int N = 4; EXPR; } break;     \
    case 5: { constexpr int N = 5; EXPR; } break;     \
    case 6: { constexpr int N = 6; EXPR; } break;     \
    default: return fail("LUT width n=%d not in 2..6", n); \
    }

template <int N>
void launch_table_prep(float const *W, float *C, int node_size, int lut_binarize, hipStream_t st, float *V = nullptr, float bias = 0.0f,
                       float *clamp_W = nullptr, float clamp_lo = 0.0f, float clamp_hi = 0.0f)
{
    int const total = node_size * (1 << N);
    hipLaunchKernelGGL(table_prep_kernel<N>, dim3(ceil_div(total, kBlock)), dim3(kBlock), 0, st, W, C, node_size, lut_binarize, V, bias, clamp_W, clamp_lo, clamp_hi);
}

template <int N, int XMODE, int YMODE, int KIND>
void launch_forward(FwdArgs const &a, int npw, hipStream_t st)
{
    dim3 const grid(a.chunk_count * a.tiles.count), block(kBlock);
    if constexpr (XMODE == kXBit || XMODE == kXBinary) {
        // two-valued inputs: the corner-value kernel wherever the caller prepared the values (one node per wavefront)
        if (a.V != nullptr) {
            if constexpr (XMODE == kXBit && YMODE == kYBinarize && KIND == 1) {
                if (a.own_index != nullptr) {      // corner indices kept by the statistics launch of the same call
                    hipLaunchKernelGGL((lut_forward_corner_kernel<N, XMODE, YMODE, KIND, false, kOwnMemory>), grid, block, 0, st, a);
                    return;
                }
            }
            if constexpr (XMODE == kXBit) {
                // 32-byte scalar loads where they stay inside the row pitch and never straddle a unit
                if (a.x_stride % 8 == 0 && a.chunk % 256 == 0 && (reinterpret_cast<uintptr_t>(a.x) & 3u) == 0) {
                    hipLaunchKernelGGL((lut_forward_corner_kernel<N, XMODE, YMODE, KIND, true>), grid, block, 0, st, a);
                    return;
                }
            }
            hipLaunchKernelGGL((lut_forward_corner_kernel<N, XMODE, YMODE, KIND>), grid, block, 0, st, a);
            return;
        }
    }
    if (npw == 2) { hipLaunchKernelGGL((lut_forward_kernel<N, XMODE, YMODE, KIND, 2>), grid, block, 0, st, a); }
    else          { hipLaunchKernelGGL((lut_forward_kernel<N, XMODE, YMODE, KIND, 1>), grid, block, 0, st, a); }
}

// xmode / ymode / kind are runtime values here; the combinations that exist are enumerated explicitly
template <int N>
int dispatch_forward(int xmode, int ymode, int kind, FwdArgs const &a, int npw, hipStream_t st)
{
#define BBHIP_FWD_CASE(X, Y, K) if (xmode == X && ymode == Y && kind == K) { launch_forward<N, X, Y, K>(a, npw, st); return 0; }
    BBHIP_FWD_CASE(kXClamp,  kYClamp,    0)
    BBHIP_FWD_CASE(kXBinary, kYClamp,    0)
    BBHIP_FWD_CASE(kXBit,    kYClamp,    0)
    BBHIP_FWD_CASE(kXBit,    kYBit,      0)
    BBHIP_FWD_CASE(kXBinary, kYBinarize, 0)
    BBHIP_FWD_CASE(kXClamp,  kYClamp,    1)
    BBHIP_FWD_CASE(kXBinary, kYBinarize, 1)
    BBHIP_FWD_CASE(kXBit,    kYBit,      1)
    BBHIP_FWD_CASE(kXBit,    kYBinarize, 0)         // fp32 frames of binary mode, packed by the library
    BBHIP_FWD_CASE(kXBit,    kYBinarize, 1)
    BBHIP_FWD_CASE(kXClamp,  kYClamp,    2)
    BBHIP_FWD_CASE(kXBinary, kYClamp,    2)
    BBHIP_FWD_CASE(kXBit,    kYClamp,    2)
    BBHIP_FWD_CASE(kXClamp,  kYClamp,    3)
    BBHIP_FWD_CASE(kXBinary, kYClamp,    3)
    BBHIP_FWD_CASE(kXBit,    kYClamp,    3)
#undef BBHIP_FWD_CASE
    return fail("forward variant (x=%d, y=%d, kind=%d) not built", xmode, ymode, kind);
}

template <int N>
int dispatch_backward(int xmode, int kind, int dxmode, BwdArgs const &a, hipStream_t st)
{
    dim3 const grid(a.tt.blocks + a.slab_count * a.tiles.count), block(kBlock);
    if (xmode == kXBit && kind == 1 && dxmode == kDxNone && a.V != nullptr) {       // batch-norm window from the corner values
        hipLaunchKernelGGL((lut_backward_kernel<N, kXBit, 1, kDxNone, true>), grid, block, 0, st, a);
        return 0;
    }
#define BBHIP_BWD_CASE(X, K, M) if (xmode == X && kind == K && dxmode == M) { hipLaunchKernelGGL((lut_backward_kernel<N, X, K, M>), grid, block, 0, st, a); return 0; }
    BBHIP_BWD_CASE(kXClamp,  0, kDxAtomic) BBHIP_BWD_CASE(kXClamp,  0, kDxTmp)
    BBHIP_BWD_CASE(kXBinary, 0, kDxAtomic) BBHIP_BWD_CASE(kXBinary, 0, kDxTmp)
    BBHIP_BWD_CASE(kXBit,    0, kDxAtomic) BBHIP_BWD_CASE(kXBit,    0, kDxTmp)
    BBHIP_BWD_CASE(kXClamp,  1, kDxAtomic) BBHIP_BWD_CASE(kXClamp,  1, kDxTmp)
    BBHIP_BWD_CASE(kXBinary, 1, kDxAtomic) BBHIP_BWD_CASE(kXBinary, 1, kDxTmp)
    BBHIP_BWD_CASE(kXBit,    1, kDxAtomic) BBHIP_BWD_CASE(kXBit,    1, kDxTmp)
    BBHIP_BWD_CASE(kXClamp,  0, kDxNone) BBHIP_BWD_CASE(kXClamp,  1, kDxNone)
    BBHIP_BWD_CASE(kXBinary, 0, kDxNone) BBHIP_BWD_CASE(kXBinary, 1, kDxNone)
    BBHIP_BWD_CASE(kXBit,    0, kDxNone) BBHIP_BWD_CASE(kXBit,    1, kDxNone)
#undef BBHIP_BWD_CASE
    return fail("backward variant (x=%d, kind=%d, dx=%d) not built", xmode, kind, dxmode);
}

template <int N, int U>
int dispatch_dx_u(int xmode, DxArgs const &a, hipStream_t st)
{
    dim3 const grid(a.fin_blocks + a.chunk_count * a.tiles.count), block(kBlock);
    if (use_corner_values(xmode)) {         // the term table then holds corner values
        if (xmode == kXBit) { hipLaunchKernelGGL((lut_dx_corner_kernel<N, kXBit, U>),    grid, block, 0, st, a); }
        else                { hipLaunchKernelGGL((lut_dx_corner_kernel<N, kXBinary, U>), grid, block, 0, st, a); }
        return 0;
    }
    switch (xmode) {
    case kXClamp:  hipLaunchKernelGGL((lut_dx_kernel<N, kXClamp, U>),  grid, block, 0, st, a); return 0;
    case kXBinary: hipLaunchKernelGGL((lut_dx_kernel<N, kXBinary, U>), grid, block, 0, st, a); return 0;
    case kXBit:    hipLaunchKernelGGL((lut_dx_kernel<N, kXBit, U>),    grid, block, 0, st, a); return 0;
    }
    return fail("dx variant (x=%d) not built", xmode);
}

template <int N>
int dispatch_dx(int xmode, int steps, DxArgs const &a, hipStream_t st)
{
    switch (steps) {
    case 1: return dispatch_dx_u<N, 1>(xmode, a, st);
    case 2: return dispatch_dx_u<N, 2>(xmode, a, st);
    case 4: return dispatch_dx_u<N, 4>(xmode, a, st);
    }
    return fail("dx kernel with %d wavefront-steps per pass not built", steps);
}

// ------------------------------------------------------------------------------------------------
//  forward driver
// ------------------------------------------------------------------------------------------------
struct ForwardCall {
    int n;
    void const *x; void *y; int const *idx; float const *W;
    int node_size, frame_size, x_stride, y_stride;
    int xmode, ymode;
    int lut_binarize; float bias;
    // batch-norm
    int bn;                      // 0 none, 1 training, 2 inference
    float *mean, *rstd, *running_mean, *running_var;
    float gamma, beta, momentum;
    // non-null: W (the same buffer) is clamped in place to [clamp_lo, clamp_hi] by the table-preparation launch
    float *clamp_W; float clamp_lo, clamp_hi;
};

// the kernels address a frame inside its node row with a 32-bit byte offset
constexpr int kMaxFrames = 1 << 29;
// most scratch that a forward call takes for the corner indices that its statistics launch keeps for its output launch (run_forward)
constexpr size_t kOwnIndexMaxBytes = (size_t)1 << 30;

int check_forward(ForwardCall const &c)
{
    if (!(c.x && c.y && c.idx && c.W))               { return fail("forward: null buffer"); }
    if (!(c.node_size > 0 && c.frame_size > 0))      { return fail("forward: node_size=%d frame_size=%d must be positive", c.node_size, c.frame_size); }
    if (c.frame_size > kMaxFrames)                   { return fail("forward: frame_size=%d above %d (32-bit byte offsets within a row)", c.frame_size, kMaxFrames); }
    int const x_need = (c.xmode == kXBit) ? (c.frame_size + 31) / 32 : c.frame_size;
    int const y_need = (c.ymode == kYBit) ? (c.frame_size + 31) / 32 : c.frame_size;
    if (c.x_stride < x_need || c.y_stride < y_need)  { return fail("forward: frame stride (x %d, y %d) shorter than the frames (%d, %d)", c.x_stride, c.y_stride, x_need, y_need); }
    if ((long long)c.node_size * (1 << c.n) > 0x7fffffffLL) { return fail("forward: node_size too large"); }
    if (c.bn == 1 && !(c.mean && c.rstd && c.running_mean && c.running_var)) { return fail("forward: null statistics buffer"); }
    if (c.bn == 2 && !(c.running_mean && c.running_var))                      { return fail("forward: null statistics buffer"); }
    return 0;
}

// nodes per workgroup of the batch-norm finalize kernels: the more units there are to add per node, the more of the
// workgroup's threads share one node
int stat_nodes_per_block(int unit_count) { return unit_count >= 512 ? 4 : unit_count >= 64 ? 16 : 64; }

// row pitch (words) of the library's packed copy of `frame_size` binarized frames
int packed_row_words(int frame_size)
{
    int words = (((frame_size + 31) / 32) + 7) & ~7;
    if ((words * 4) % 2048 == 0) { words += 96; }          // keep the row pitch off the multiples of 2 KiB
    return words;
}

// fp32 frames -> packed bits (bit = x > 0.5) for `node_size` rows
int launch_binarize_pack(float const *x, int x_stride, uint32_t *bits, int bit_stride, int node_size, int frame_size, hipStream_t st)
{
    for (int n0 = 0; n0 < node_size; n0 += 65535) {        // grid.y is limited to 65535 rows per launch
        int const rows = (node_size - n0 < 65535) ? node_size - n0 : 65535;
        float const *src = x + (size_t)n0 * x_stride;
        uint32_t *dst = bits + (size_t)n0 * bit_stride;
        if (x_stride % 4 == 0 && (reinterpret_cast<uintptr_t>(x) & 15u) == 0) {
            hipLaunchKernelGGL(binarize_pack4_kernel, dim3(ceil_div(bit_stride * 8, kBlock), rows), dim3(kBlock), 0, st,
                               src, dst, frame_size, x_stride, bit_stride);
        }
        else {
            hipLaunchKernelGGL(binarize_pack_kernel, dim3(ceil_div(bit_stride * 32, kBlock), rows), dim3(kBlock), 0, st,
                               src, dst, frame_size, x_stride, bit_stride);
        }
    }
    BBHIP_LAUNCH_CHECK();
    return 0;
}

// packing and table preparation; one launch for both where the packing takes the 16-byte path
template <int N>
int launch_pack_and_prep(float const *x, int x_stride, uint32_t *bits, int bit_stride, int rows, int frame_size,
                         float const *W, float *C, float *V, int node_size, int lut_binarize, float bias, hipStream_t st,
                         float *clamp_W = nullptr, float clamp_lo = 0.0f, float clamp_hi = 0.0f)
{
    int const row_blocks = ceil_div(bit_stride * 8, kBlock);
    long long const pack_blocks = (long long)rows * row_blocks, prep_blocks = ceil_div(node_size * (1 << N), kBlock);
    if (x_stride % 4 == 0 && (reinterpret_cast<uintptr_t>(x) & 15u) == 0 && pack_blocks + prep_blocks <= 0x7fffffffLL) {
        PackPrepArgs a{};
        a.x = x; a.bits = bits; a.frame_size = frame_size; a.x_stride = x_stride; a.y_stride = bit_stride;
        a.row_blocks = make_tile_divisor(row_blocks); a.pack_blocks = (int)pack_blocks;
        a.W = W; a.C = C; a.V = V; a.node_size = node_size; a.lut_binarize = lut_binarize; a.bias = bias;
        a.clamp_W = clamp_W; a.clamp_lo = clamp_lo; a.clamp_hi = clamp_hi;
        hipLaunchKernelGGL(binarize_pack4_prep_kernel<N>, dim3((unsigned)(pack_blocks + prep_blocks)), dim3(kBlock), 0, st, a);
        BBHIP_LAUNCH_CHECK();
        return 0;
    }
    if (launch_binarize_pack(x, x_stride, bits, bit_stride, rows, frame_size, st)) { return 1; }
    launch_table_prep<N>(W, C, node_size, lut_binarize, st, V, bias, clamp_W, clamp_lo, clamp_hi);
    BBHIP_LAUNCH_CHECK();
    return 0;
}

template <int N>
int run_forward(ForwardCall const &call, int input_rows, hipStream_t st, Scratch const *fixed = nullptr,
                PackedInputHint packed = PackedInputHint{nullptr, 0, 0, 0}, PreparedTablesHint tables = PreparedTablesHint{nullptr, 0, 0},
                PackedOutputHint packed_out = PackedOutputHint{nullptr, 0, 0})
{
    constexpr int NN = 1 << N;
    // input_rows: what the caller said about the input's row count (bbhip_HintInputNodeSize), 0 = nothing.
    // fp32 frames that the layer binarizes at 0.5 are packed to bits once where the row count is known; from here on the
    // call is a packed-bit call (same outputs)
    ForwardCall c = call;
    bool const bits_wanted = (c.xmode == kXBinary) && input_rows > 0 && use_corner_values(kXBinary) && pack_binarized_input();
    // the packed copy goes to the caller's buffer where one was offered and fits (rows of whole 32-byte groups), else to the arena
    bool const to_caller = bits_wanted && packed.bits != nullptr && packed.rows == input_rows && packed.row_words >= (c.frame_size + 31) / 32 &&
                           packed.row_words % 8 == 0 && (reinterpret_cast<uintptr_t>(packed.bits) & 31u) == 0;
    // ... unless the caller says that the buffer already holds the packed copy of this input (the packed output of the layer
    // before, or of an earlier call on the same input): nothing to pack
    bool const have_bits = to_caller && packed.holds_input;
    bool const pack = bits_wanted && !have_bits;
    if (bits_wanted) { c.xmode = kXBit; c.x_stride = to_caller ? packed.row_words : packed_row_words(c.frame_size); c.x = have_bits ? packed.bits : nullptr; }
    bool const corner     = use_corner_values(c.xmode);
    int const npw         = corner ? 1 : fwd_nodes_per_wave();
    int const tile_count  = ceil_div(c.node_size, kWavesPerBlk * npw);
    // Batch-norm training pass of a small batch on the corner-value kernel: one unit per node, so that the wavefront that writes a
    // node's output can sum the node's statistics itself (kStatInline) and the statistics launch falls away — at up to 1024 frames
    // a launch costs more than the second evaluation of the unit does.  BBHIP_FWD_CHUNK set in the environment keeps its say.
    bool const one_unit   = (c.bn == 1) && corner && c.frame_size <= 1024 && fwd_chunk_frames_env() == 0;
    int const chunk       = one_unit ? 1024 : fwd_chunk_frames(c.xmode, c.frame_size, tile_count);
    int const chunk_count = ceil_div(c.frame_size, chunk);
    if ((long long)chunk_count * tile_count > 0x7fffffffLL) { return fail("forward: grid too large"); }

    size_t const c_bytes    = align256((size_t)c.node_size * NN * sizeof(float));
    size_t const v_bytes    = corner ? c_bytes : 0;
    size_t const stat_bytes = (c.bn == 1) ? align256((size_t)chunk_count * c.node_size * 2 * sizeof(float)) : 0;
    size_t const bits_bytes = (pack && !to_caller) ? align256((size_t)input_rows * c.x_stride * sizeof(uint32_t)) : 0;
    // fp32 frames of binary mode whose row count nobody told (nothing to pack ahead), batch-norm training pass in two launches: the
    // statistics launch keeps the corner index that it forms of every (node, frame), a byte each, and the output launch reads those
    // instead of gathering the fp32 frames again (FwdArgs::own_index_out).  Up to kOwnIndexMaxBytes of scratch.
    int const own_words = ceil_div(c.frame_size, 256) * kWave;
    bool const own_index = (c.xmode == kXBinary) && corner && pack_binarized_input() && c.bn == 1 && !one_unit && chunk_count > 1 &&
                           chunk % 256 == 0 && c.ymode == kYBinarize && fixed == nullptr &&
                           (size_t)c.node_size * own_words * sizeof(uint32_t) <= kOwnIndexMaxBytes;
    size_t const own_bytes = own_index ? align256((size_t)c.node_size * own_words * sizeof(uint32_t)) : 0;
    char *base = nullptr;
    if (arena_get(c_bytes + v_bytes + stat_bytes + bits_bytes + own_bytes, &base, st, fixed)) { return 1; }
    float *C        = reinterpret_cast<float *>(base);
    float *V        = corner ? reinterpret_cast<float *>(base + c_bytes) : nullptr;
    float *stat     = reinterpret_cast<float *>(base + c_bytes + v_bytes);
    // the tables go to the caller's buffer where one was offered and fits: the backward call of the same step can take them from there
    bool const tables_to_caller = tables_fit(tables, c_bytes + v_bytes);
    if (tables_to_caller) {
        C = tables.buf;
        V = corner ? reinterpret_cast<float *>(reinterpret_cast<char *>(tables.buf) + c_bytes) : nullptr;
    }
    if (pack) {
        uint32_t *bits = to_caller ? packed.bits : reinterpret_cast<uint32_t *>(base + c_bytes + v_bytes + stat_bytes);
        if (launch_pack_and_prep<N>(reinterpret_cast<float const *>(call.x), call.x_stride, bits, c.x_stride, input_rows, c.frame_size,
                                    c.W, C, V, c.node_size, c.lut_binarize, c.bias, st, c.clamp_W, c.clamp_lo, c.clamp_hi)) { return 1; }
        c.x = bits;
    }
    // plain output of a call with one unit per node on the polynomial kernel: the wavefronts prepare their node's table
    // themselves (FwdArgs::W_inline), clamp it in place where the entry asks for that, and the table launch falls away
    bool const inline_table = (c.bn == 0) && !corner && chunk_count == 1 && LutMatrixQ<N>::kUsable && !tables_to_caller;
    // the corner-value kernel derives a node's tables in the wavefront in any case where no packing launch is there to carry the
    // preparation: the first launch of the call does it and stores them for the launches (and the backward call) that follow
    bool const inline_corner = corner && !pack && inline_tables();
    if (!pack && !inline_table && !inline_corner) {
        launch_table_prep<N>(c.W, C, c.node_size, c.lut_binarize, st, V, c.bias, c.clamp_W, c.clamp_lo, c.clamp_hi);
        BBHIP_LAUNCH_CHECK();
    }

    FwdArgs a{};
    if (inline_table) { a.W_inline = c.W; a.lut_binarize = c.lut_binarize; a.clamp_W = c.clamp_W; a.clamp_lo = c.clamp_lo; a.clamp_hi = c.clamp_hi; }
    if (inline_corner) {
        a.W_inline = c.W; a.lut_binarize = c.lut_binarize; a.C_out = C; a.V_out = V;
        a.clamp_W = c.clamp_W; a.clamp_lo = c.clamp_lo; a.clamp_hi = c.clamp_hi;
    }
    a.x = c.x; a.y = c.y; a.idx = c.idx; a.C = C; a.V = V;
    a.node_size = c.node_size; a.frame_size = c.frame_size;
    a.x_stride = c.x_stride; a.y_stride = c.y_stride;
    a.chunk = chunk; a.chunk_count = chunk_count; a.tiles = make_tile_divisor(tile_count);
    a.bias = c.bias; a.gamma = c.gamma; a.beta = c.beta;

    int kind = 0;
    if (c.bn == 1 && corner && chunk_count == 1) {
        // one unit per node and the cheap corner-value kernel: its wavefronts sum the statistics of their node themselves
        // before they write its output, which saves the statistics launch (the evaluation it repeats costs less than that)
        a.stat_mode = kStatInline; a.momentum = c.momentum;
        a.mean_out = c.mean; a.rstd_out = c.rstd; a.running_mean = c.running_mean; a.running_var = c.running_var;
        kind = 1;
    }
    else if (c.bn == 1) {
        a.stat_partial = stat;
        if (own_index) { a.own_index_out = reinterpret_cast<uint32_t *>(base + c_bytes + v_bytes + stat_bytes + bits_bytes); a.own_stride = own_words; }
        if (dispatch_forward<N>(c.xmode, kYClamp, 2, a, npw, st)) { return 1; }
        BBHIP_LAUNCH_CHECK();
        if (inline_corner) { a.W_inline = nullptr; a.C_out = nullptr; a.V_out = nullptr; a.clamp_W = nullptr; }      // stored by that launch
        if (own_index) {
            // the output launch reads the kept indices, a coalesced word per lane and four steps: longer units than the gathers of
            // fp32 frames want (a unit's set-up weighs less), halved while they would leave the launch short of workgroups
            a.own_index = a.own_index_out; a.own_index_out = nullptr; a.stat_units = chunk_count;
            c.xmode = kXBit;
            int own_chunk = 2048;
            while (own_chunk > 256 && (long long)ceil_div(c.frame_size, own_chunk) * tile_count < 2048) { own_chunk /= 2; }
            a.chunk = own_chunk; a.chunk_count = ceil_div(c.frame_size, own_chunk);
        }
        if (chunk_count <= kInlineStatUnits) {
            // few units: every wavefront of the output pass adds up the partial sums of its node itself, and the wavefront of a
            // node's first unit stores the statistics; a launch that does it once per node would cost more than that
            a.stat_mode = kStatPartial; a.momentum = c.momentum;
            a.mean_out = c.mean; a.rstd_out = c.rstd; a.running_mean = c.running_mean; a.running_var = c.running_var;
        }
        else {
            int const npb = stat_nodes_per_block(chunk_count);
            hipLaunchKernelGGL(bn_forward_finalize_kernel, dim3(ceil_div(c.node_size, npb)), dim3(kBlock), 0, st,
                               stat, C, NN, c.mean, c.rstd, c.running_mean, c.running_var, c.momentum,
                               c.node_size, chunk_count, c.frame_size, npb);
            BBHIP_LAUNCH_CHECK();
            a.mean = c.mean; a.rstd = c.rstd;
        }
        kind = 1;
    }
    else if (c.bn == 2) {
        a.stat_mode = kStatRunning; a.mean = c.running_mean; a.rstd = c.running_var;       // rstd = 1 / sqrt(var) in the kernel
        kind = 1;
    }
    // the binarized fp32 output as packed bits as well, where the caller offered a buffer that fits (rows of whole 32-byte groups)
    if (c.ymode == kYBinarize && packed_out.bits != nullptr && packed_out.rows == c.node_size && packed_out.row_words >= (c.frame_size + 31) / 32 &&
        packed_out.row_words % 8 == 0 && (reinterpret_cast<uintptr_t>(packed_out.bits) & 31u) == 0) {
        a.y_bits = packed_out.bits; a.y_bits_stride = packed_out.row_words;
    }
    {
        ScopedTimer tm(kTimeForward, st, fixed == nullptr);     // (event creation may allocate: not on the path that must not)
        if (dispatch_forward<N>(c.xmode, c.ymode, kind, a, npw, st)) { return 1; }
    }
    BBHIP_LAUNCH_CHECK();
    return 0;
}

int forward_entry(ForwardCall const &c, void *stream, Scratch const *fixed = nullptr)
{
    // the hints are spent by this call, whatever becomes of it; a buffer for the packed copy also says how many rows the input has
    PackedInputHint const packed = fixed ? PackedInputHint{nullptr, 0, 0, 0} : g_packed_hint;
    int const input_rows = fixed ? 0 : (packed.bits ? packed.rows : g_input_node_hint);
    PreparedTablesHint const tables = fixed ? PreparedTablesHint{nullptr, 0, 0} : g_tables_hint;
    PackedOutputHint const packed_out = fixed ? PackedOutputHint{nullptr, 0, 0} : g_packed_out_hint;
    clear_hints();
    if (check_forward(c)) { return 1; }
    hipStream_t st = static_cast<hipStream_t>(stream);
    BBHIP_SWITCH_N(c.n, return run_forward<N>(c, input_rows, st, fixed, packed, tables, packed_out));
    return 0;
}

// ------------------------------------------------------------------------------------------------
//  backward driver
// ------------------------------------------------------------------------------------------------
struct BackwardCall {
    int n;
    void const *x; float const *dy; float *dx; float *dx_tmp;
    int const *idx; int const *rev; float const *W; float *dW;
    int rev_stride, input_node_size, output_node_size, frame_size;
    int x_stride, frame_stride, tmp_frame_size, tmp_frame_stride;
    int xmode, lut_binarize; float bias;
    int bn;
    float const *mean, *rstd; float *dmean_tmp, *dvar_tmp;
    float gamma, beta;
};

int check_backward(BackwardCall const &c, int dxmode)
{
    if (!(c.x && c.dy && c.dx && c.idx && c.W && c.dW)) { return fail("backward: null buffer"); }
    if (!(c.input_node_size > 0 && c.output_node_size > 0 && c.frame_size > 0)) { return fail("backward: sizes must be positive"); }
    if (c.frame_size > kMaxFrames)                   { return fail("backward: frame_size=%d above %d (32-bit byte offsets within a row)", c.frame_size, kMaxFrames); }
    int const x_need = (c.xmode == kXBit) ? (c.frame_size + 31) / 32 : c.frame_size;
    if (c.x_stride < x_need || c.frame_stride < c.frame_size) { return fail("backward: frame stride shorter than the frames"); }
    if ((long long)c.output_node_size * (1 << c.n) > 0x7fffffffLL) { return fail("backward: node_size too large"); }
    if (dxmode == kDxNone) {
        if (!c.rev)                                      { return fail("backward: deterministic dx needs reverse_index (or bbhip_SetDxMode(1))"); }
        if (c.rev_stride < 1)                            { return fail("backward: reverse_index_stride=%d", c.rev_stride); }
    }
    if (dxmode == kDxTmp) {
        if (!(c.dx_tmp && c.rev))                        { return fail("backward: scratch-buffer dx needs dx_tmp and reverse_index"); }
        if (c.tmp_frame_size <= 0)                       { return fail("backward: tmp_frame_size=%d must be positive", c.tmp_frame_size); }
        int const span = c.tmp_frame_size < c.frame_size ? c.tmp_frame_size : c.frame_size;
        if (c.tmp_frame_stride < span)                   { return fail("backward: tmp_frame_stride=%d shorter than tmp_frame_size", c.tmp_frame_stride); }
        if (c.rev_stride < 1)                            { return fail("backward: reverse_index_stride=%d", c.rev_stride); }
    }
    if (c.bn && !(c.mean && c.rstd && c.dmean_tmp && c.dvar_tmp)) { return fail("backward: null statistics buffer"); }
    return 0;
}

template <int N>
int run_backward(BackwardCall const &call, hipStream_t st, PackedInputHint packed = PackedInputHint{nullptr, 0, 0, 0},
                 PreparedTablesHint tables = PreparedTablesHint{nullptr, 0, 0}, int dw_overwrite = 0)
{
    constexpr int NN = 1 << N;
    int dxmode = (g_dx_mode == 1) ? kDxAtomic : (g_dx_mode == 2) ? kDxTmp : kDxNone;
    // The term table of the deterministic dx kernel has one slot per (input node, position in the longest fan-out list).  With
    // evenly used inputs that is about the number of connections; wiring in which a few inputs feed very many nodes would make
    // it (and the launch that fills it) grow with input nodes x longest list while only output nodes x n records are ever
    // read.  Such a call takes the reference's scheme where the caller gave it a dx_tmp buffer, else the atomic one: same
    // results to rounding, but in the atomic case not reproducible bit for bit.
    if (dxmode == kDxNone && call.rev != nullptr && call.rev_stride >= 1) {
        long long const slots = (long long)call.input_node_size * (long long)(call.rev_stride - 1);
        long long const links = (long long)call.output_node_size * call.n;
        if (slots > 8 * links + 65536) { dxmode = (call.dx_tmp != nullptr && call.tmp_frame_size > 0) ? kDxTmp : kDxAtomic; }
    }
    if (check_backward(call, dxmode)) { return 1; }

    // fp32 frames that the layer binarizes at 0.5 are packed to bits once (reading them once costs less than the three
    // kernels of this pass gain from packed rows); from here on the call is a packed-bit call
    BackwardCall c = call;
    bool const pack = (c.xmode == kXBinary) && dxmode == kDxNone && use_corner_values(kXBinary) && pack_binarized_input();
    // a caller that kept the packed copy of this input from the forward call hands it back: nothing to pack
    bool const have_bits = pack && packed.bits != nullptr && packed.holds_input && packed.rows == c.input_node_size &&
                           packed.row_words >= (c.frame_size + 31) / 32 && packed.row_words % 8 == 0 &&
                           (reinterpret_cast<uintptr_t>(packed.bits) & 31u) == 0;
    if (pack) { c.xmode = kXBit; c.x_stride = have_bits ? packed.row_words : packed_row_words(c.frame_size); c.x = nullptr; }   // else: a place in the arena below

    int const tile_count = ceil_div(c.output_node_size, kWavesPerBlk);
    int const range      = (dxmode == kDxTmp) ? (c.tmp_frame_size < c.frame_size ? c.tmp_frame_size : c.frame_size) : c.frame_size;
    int const range_count = ceil_div(c.frame_size, range);

    // slab length: a wavefront multiple.  Long slabs amortise the cross-lane reduction that ends each of them (4096 frames
    // unless that leaves fewer than eight workgroups per compute unit), and long enough that the per-slab partial tables
    // stay below 256 MiB
    int slab = bwd_slab_frames();
    if (slab == 0) {
        // The kernel keeps five workgroups per compute unit: a launch runs in ceil(workgroups / 1280) rounds of them, and a slab costs
        // its frames plus about 384 frames' worth of set-up and reduction (fitted to 112 / 121 / 122 us at slabs of 4096 / 2048 / 1024
        // frames for 4096 nodes x 8192 frames).  The slab length with the least rounds x cost: 4096 there (two rounds), 2048 for
        // 216 nodes x 230 400 frames (five rounds against three twice as long) and for 36 nodes (one round), 512 / 256 for the layers
        // of the classifier at 1024 frames.
        auto cost = [&](int frames) {
            long long const groups = (long long)tile_count * range_count * ceil_div(range, frames);
            return ((groups + 1279) / 1280) * (long long)(frames + 384);
        };
        slab = 4096;
        for (int cand = 2048; cand >= 256; cand /= 2) { if (cost(cand) < cost(slab)) { slab = cand; } }
    }
    for (;;) {
        long long slabs = (long long)range_count * ceil_div(range, slab);
        if (slabs * c.output_node_size * NN * (long long)sizeof(float) <= (256LL << 20) || slab >= range) { break; }
        slab *= 2;
    }
    // total number of slabs over all ranges (the last range may be shorter)
    int slab_total = 0;
    for (int r = 0; r < range_count; ++r) {
        int const len = (r + 1 < range_count) ? range : (c.frame_size - r * range);
        slab_total += ceil_div(len, slab);
    }
    if ((long long)slab_total * tile_count > 0x7fffffffLL) { return fail("backward: grid too large"); }

    size_t const c_bytes    = align256((size_t)c.output_node_size * NN * sizeof(float));
    size_t const part_bytes = align256((size_t)slab_total * c.output_node_size * NN * sizeof(float));
    // batch-norm statistics pass: the forward kernel's unit structure (frame chunks, see below)
    bool const corner = c.bn && use_corner_values(c.xmode);     // the statistics pass looks the LUT output up among corner values
    int const stat_npw = corner ? 1 : fwd_nodes_per_wave();
    int const stat_chunk       = fwd_chunk_frames(c.xmode, c.frame_size, ceil_div(c.output_node_size, kWavesPerBlk * stat_npw));
    int const stat_chunk_count = ceil_div(c.frame_size, stat_chunk);
    size_t const stat_bytes = c.bn ? align256((size_t)stat_chunk_count * c.output_node_size * 2 * sizeof(float)) : 0;
    // Batch-norm backward of a small batch over packed rows: the statistics pass (passes of four steps over 32-byte groups of the rows)
    // keeps the corner index it forms of every (node, frame), a byte each, and the dx kernel looks a term's value up at that index
    // instead of reading the consumer's other five rows and forming the index again (lut_dx_indexed_kernel): a third of the vector
    // instructions per term.  That pays where dy and the indices stay close to the compute units (classifier step: dx of the three
    // layers 43.9 -> 38 us); at 4096 x 4096 x 8192 and at the conv block's 230 400 frames the dx kernel is bound by the gather of its
    // dy rows and the kept bytes only add traffic (128.5 vs 128.1 us, 121 vs 114 us, statistics pass + 6 us): up to 32 MiB of both.
    int const own_words = ceil_div(c.frame_size, 256) * kWave;
    bool const indexed = c.bn && dxmode == kDxNone && corner && term_from_corner_values() && c.xmode == kXBit && dx_indexed() &&
                         dx_pass_steps_env() == 0 && (dx_chunk_frames_env() == 0 || dx_chunk_frames_env() % 256 == 0) &&
                         c.x_stride % 8 == 0 && stat_chunk % 256 == 0 &&
                         (size_t)c.output_node_size * c.frame_size * 5 <= ((size_t)32 << 20);
    size_t const own_bytes = indexed ? align256((size_t)c.output_node_size * own_words * sizeof(uint32_t)) : 0;
    size_t const term_count = (dxmode == kDxNone) ? (size_t)c.input_node_size * (size_t)(c.rev_stride - 1) * (kTermHead + (indexed ? NN : NN / 2)) : 0;
    size_t const dtab_bytes = align256(term_count * sizeof(int));
    size_t const dyh_bytes  = (dxmode == kDxNone && c.bn) ? align256((size_t)c.output_node_size * c.frame_stride * sizeof(float)) : 0;
    size_t const v_bytes = corner ? c_bytes : 0;
    size_t const bits_bytes = (pack && !have_bits) ? align256((size_t)c.input_node_size * c.x_stride * sizeof(uint32_t)) : 0;
    char *base = nullptr;
    if (arena_get(c_bytes + part_bytes + stat_bytes + dtab_bytes + dyh_bytes + v_bytes + bits_bytes + own_bytes, &base, st)) { return 1; }
    uint32_t *own = indexed ? reinterpret_cast<uint32_t *>(base + c_bytes + part_bytes + stat_bytes + dtab_bytes + dyh_bytes + v_bytes + bits_bytes) : nullptr;
    float *V    = corner ? reinterpret_cast<float *>(base + c_bytes + part_bytes + stat_bytes + dtab_bytes + dyh_bytes) : nullptr;
    float *C    = reinterpret_cast<float *>(base);
    float *part = reinterpret_cast<float *>(base + c_bytes);
    float *stat = reinterpret_cast<float *>(base + c_bytes + part_bytes);
    int   *term = reinterpret_cast<int *>(base + c_bytes + part_bytes + stat_bytes);
    float *dyh  = reinterpret_cast<float *>(base + c_bytes + part_bytes + stat_bytes + dtab_bytes);

    // centred coefficients: needed where the LUT output is recomputed (batch-norm) or per-connection gradients are formed;
    // a caller that kept the tables of this step's forward call (same W, same kind of input) hands them back: nothing to prepare
    bool const have_tables = tables.holds_tables && tables_fit(tables, c_bytes + v_bytes);
    if (have_tables) {
        C = tables.buf;
        V = corner ? reinterpret_cast<float *>(reinterpret_cast<char *>(tables.buf) + c_bytes) : nullptr;
    }
    bool const prep = (c.bn || dxmode != kDxNone) && !have_tables;
    if (have_bits) {
        c.x = packed.bits;
        if (prep) {
            launch_table_prep<N>(c.W, C, c.output_node_size, c.lut_binarize, st, V, c.bias);
            BBHIP_LAUNCH_CHECK();
        }
    }
    else if (pack) {
        uint32_t *bits = reinterpret_cast<uint32_t *>(base + c_bytes + part_bytes + stat_bytes + dtab_bytes + dyh_bytes + v_bytes);
        float const *src = reinterpret_cast<float const *>(call.x);
        if (prep) {
            if (launch_pack_and_prep<N>(src, call.x_stride, bits, c.x_stride, c.input_node_size, c.frame_size,
                                        c.W, C, V, c.output_node_size, c.lut_binarize, c.bias, st)) { return 1; }
        }
        else if (launch_binarize_pack(src, call.x_stride, bits, c.x_stride, c.input_node_size, c.frame_size, st)) { return 1; }
        c.x = bits;
    }
    else if (prep) {
        launch_table_prep<N>(c.W, C, c.output_node_size, c.lut_binarize, st, V, c.bias);
        BBHIP_LAUNCH_CHECK();
    }
    // the term table of the dx kernel is built by extra workgroups at the end of the table-gradient launch
    TermArgs tt{};
    if (dxmode == kDxNone && term_count > 0) {
        size_t const records = (size_t)c.input_node_size * (size_t)(c.rev_stride - 1);
        size_t const per_block = (size_t)kWavesPerBlk * kTermRecordsPerWave;
        size_t const blocks = (((records + per_block - 1) / per_block) + 7) & ~(size_t)7;            // whole rounds over the XCDs
        if (records > 0x7fffffffULL || blocks + (size_t)slab_total * tile_count > 0x7fffffffULL) { return fail("backward: grid too large"); }
        tt.fan = make_tile_divisor(c.rev_stride - 1);
        tt.W = c.W; tt.idx = c.idx; tt.rev = c.rev; tt.term = term;
        tt.x_base = (unsigned long long)(uintptr_t)c.x; tt.x_row_pitch_bytes = (unsigned long long)c.x_stride * 4ULL;
        tt.dy_base = (unsigned long long)(uintptr_t)(c.bn ? (void const *)dyh : (void const *)c.dy);
        tt.dy_row_pitch_bytes = (unsigned long long)c.frame_stride * 4ULL;
        tt.lut_binarize = c.lut_binarize; tt.rev_stride = c.rev_stride; tt.input_node_size = c.input_node_size;
        tt.blocks = (int)blocks;
        tt.corner = use_corner_values(c.xmode) ? 1 : 0;
        tt.lo = 0.5f - c.bias; tt.hi = 0.5f + c.bias;
        // node by node: coefficient records always, value records where the nodes' corner values are at hand (batch-norm backward)
        if (term_from_corner_values() && (corner || tt.corner == 0)) {
            tt.V = corner ? V : nullptr; tt.node_size = c.output_node_size;
            tt.blocks = (ceil_div(c.output_node_size, kWavesPerBlk) + 7) & ~7;
            if (indexed) {      // ... and point at the rows of kept corner indices instead of the input rows
                tt.indexed = 1;
                tt.x_base = (unsigned long long)(uintptr_t)own; tt.x_row_pitch_bytes = (unsigned long long)own_words * 4ULL;
            }
        }
    }

    BwdArgs a{};
    a.x = c.x; a.dy = c.dy; a.idx = c.idx; a.C = C; a.V = V;
    a.dw_partial = part;
    a.mean = c.mean; a.rstd = c.rstd; a.dmean = c.dmean_tmp; a.dvar = c.dvar_tmp;
    a.node_size = c.output_node_size; a.frame_size = c.frame_size;
    a.x_stride = c.x_stride; a.dy_stride = c.frame_stride;
    a.slab = slab; a.tiles = make_tile_divisor(tile_count);
    a.bias = c.bias; a.gamma = c.gamma; a.beta = c.beta; a.inv_frames = 1.0f / (float)c.frame_size;

    if (c.bn) {
        // phase 0: per-node sums over ALL frames, then dmean / dvar.  It only recomputes the LUT output, so it runs in the
        // forward kernel (kind 3): frame chunks that keep the gathered rows in L2, partial sums from the matrix unit
        int const npw = stat_npw;
        int const stat_tiles = ceil_div(c.output_node_size, kWavesPerBlk * npw);
        if ((long long)stat_chunk_count * stat_tiles > 0x7fffffffLL) { return fail("backward: grid too large"); }
        FwdArgs f{};
        f.x = c.x; f.idx = c.idx; f.C = C; f.V = V; f.mean = c.mean; f.rstd = c.rstd; f.stat_partial = stat;
        f.dy = c.dy; f.dy_stride = c.frame_stride;
        f.node_size = c.output_node_size; f.frame_size = c.frame_size; f.x_stride = c.x_stride;
        f.chunk = stat_chunk; f.chunk_count = stat_chunk_count; f.tiles = make_tile_divisor(stat_tiles);
        f.bias = c.bias; f.gamma = c.gamma; f.beta = c.beta;
        if (indexed) { f.own_index_out = own; f.own_stride = own_words; }
        if (dispatch_forward<N>(c.xmode, kYClamp, 3, f, npw, st)) { return 1; }
        BBHIP_LAUNCH_CHECK();
        if (stat_chunk_count <= kInlineStatUnits) {
            a.stat_partial = stat; a.stat_count = stat_chunk_count;     // few units: the table-gradient wavefronts add them up themselves
        }
        else {
            int const npb = stat_nodes_per_block(stat_chunk_count);
            hipLaunchKernelGGL(bn_backward_finalize_kernel, dim3(ceil_div(c.output_node_size, npb)), dim3(kBlock), 0, st,
                               stat, c.mean, c.rstd, c.dmean_tmp, c.dvar_tmp, c.gamma, c.output_node_size, stat_chunk_count, c.frame_size, npb);
            BBHIP_LAUNCH_CHECK();
        }
    }

    if (dxmode == kDxAtomic) {
        size_t const count = (size_t)c.input_node_size * c.frame_stride;
        hipLaunchKernelGGL(fill_kernel, dim3((unsigned)((count + kBlock * 4 - 1) / (kBlock * 4))), dim3(kBlock), 0, st, c.dx, 0.0f, count);
        BBHIP_LAUNCH_CHECK();
    }

    int slab_first = 0;
    for (int r = 0; r < range_count; ++r) {
        a.f_base     = r * range;
        a.f_limit    = (a.f_base + range < c.frame_size) ? a.f_base + range : c.frame_size;
        a.slab_first = slab_first;
        a.slab_count = ceil_div(a.f_limit - a.f_base, slab);
        if (dxmode == kDxAtomic)    { a.dx = c.dx;     a.dx_stride = c.frame_stride; }
        else if (dxmode == kDxTmp)  { a.dx = c.dx_tmp; a.dx_stride = c.tmp_frame_stride; }
        else                        { a.dx = dyh;      a.dx_stride = c.frame_stride; }
        a.tt = (r == 0) ? tt : TermArgs{};
        {
            ScopedTimer tm(kTimeBackward, st);
            if (dispatch_backward<N>(c.xmode, c.bn ? 1 : 0, dxmode, a, st)) { return 1; }
        }
        BBHIP_LAUNCH_CHECK();
        if (dxmode == kDxTmp) {
            dim3 const grid(ceil_div(a.f_limit - a.f_base, kBlock), c.input_node_size < 65535 ? c.input_node_size : 65535);
            hipLaunchKernelGGL(dx_gather_kernel, grid, dim3(kBlock), 0, st, c.dx_tmp, c.dx, c.rev, c.rev_stride,
                               c.input_node_size, a.f_base, a.f_limit, c.frame_stride, c.tmp_frame_stride);
            BBHIP_LAUNCH_CHECK();
        }
        slab_first += a.slab_count;
    }

    if (dxmode == kDxNone) {
        bool const bit_corner = (c.xmode == kXBit) && use_corner_values(c.xmode);
        int const steps  = dx_pass_steps_env() ? dx_pass_steps_env() : (bit_corner ? 4 : 2);        // wavefront-steps per pass: {1, 2, 4}
        // Packed rows with up to about a thousand input nodes (the layers of a convolution: tens to hundreds of channels x taps, very
        // many frames): the words of a pass are read with one scalar load per row — the rows then stay in the scalar cache.  With
        // more rows they do not, and the vector loads are faster (dx kernel at 324 / 512 / 1024 / 2048 rows: 94 / 107 / 138 / 141 us
        // against 104 / 127 / 147 / 135 us; 4096 rows: 385 against 319 us per step).
        bool const wide = bit_corner && dx_wide_rows() && steps == 4 && c.input_node_size <= dx_wide_max_rows() && c.x_stride % 8 == 0 &&
                          (reinterpret_cast<uintptr_t>(c.x) % 32u) == 0;
        int frames = dx_chunk_frames_env() ? dx_chunk_frames_env() : (bit_corner ? 256 : 128);
        if (wide && dx_chunk_frames_env() == 0) {
            // ... and such layers have few wavefronts' worth of input nodes and many frames: units of 1024 frames, so that a
            // wavefront's set-up (its list, its share of it) serves four passes, halved while the launch would fall short of workgroups
            // (conv block 0.602 -> 0.590 ms; the same units for a 4096-row layer: 0.338 -> 0.358 ms, hence only here)
            frames = 1024;
            while (frames > 256 && (long long)ceil_div(c.frame_size, frames) * ceil_div(c.input_node_size, kWavesPerBlk) < 2048) { frames /= 2; }
        }
        int const chunk  = ((frames + kWave * steps - 1) / (kWave * steps)) * (kWave * steps);
        int const chunk_count = ceil_div(c.frame_size, chunk);
        // few input nodes with long work lists: the four wavefronts of a workgroup share one input node (DxArgs::split)
        bool const split   = dx_split_lists(c.rev_stride - 1, (long long)chunk_count * ceil_div(c.input_node_size, kWavesPerBlk));
        int const in_tiles = split ? c.input_node_size : ceil_div(c.input_node_size, kWavesPerBlk);
        if ((long long)chunk_count * in_tiles > 0x7fffffffLL) { return fail("backward: grid too large"); }
        DxArgs d{};
        d.x = c.x; d.dy = c.bn ? dyh : c.dy; d.dx = c.dx; d.rev = c.rev; d.term = term;
        d.rev_stride = c.rev_stride; d.input_node_size = c.input_node_size; d.frame_size = c.frame_size;
        d.x_stride = c.x_stride; d.dy_stride = c.frame_stride; d.dx_stride = c.frame_stride;
        d.chunk = chunk; d.chunk_count = chunk_count; d.tiles = make_tile_divisor(in_tiles);
        d.bias = c.bias; d.split = split ? 1 : 0;
        // folding the slab sums into dW rides at the end of this launch
        d.fin_partial = part; d.fin_dW = c.dW; d.fin_node_size = c.output_node_size; d.fin_slab_count = slab_total;
        d.fin_overwrite = dw_overwrite;
        d.fin_blocks = (ceil_div(c.output_node_size * NN, kBlock) + 7) & ~7;
        if ((long long)d.fin_blocks + (long long)chunk_count * in_tiles > 0x7fffffffLL) { return fail("backward: grid too large"); }
        d.own_stride = own_words;
        {
            ScopedTimer tm(kTimeDx, st);
            if (indexed) {
                dim3 const grid(d.fin_blocks + d.chunk_count * d.tiles.count), block(kBlock);
                hipLaunchKernelGGL((lut_dx_indexed_kernel<N>), grid, block, 0, st, d);
            }
            else if (wide) {
                dim3 const grid(d.fin_blocks + d.chunk_count * d.tiles.count), block(kBlock);
                hipLaunchKernelGGL((lut_dx_corner_kernel<N, kXBit, 4, true>), grid, block, 0, st, d);
            }
            else if (dispatch_dx<N>(c.xmode, steps, d, st)) { return 1; }
        }
        BBHIP_LAUNCH_CHECK();
        return 0;
    }

    int const total = c.output_node_size * NN;
    hipLaunchKernelGGL(dw_finalize_kernel<N>, dim3(ceil_div(total, kBlock)), dim3(kBlock), 0, st, part, c.dW, c.output_node_size, slab_total, dw_overwrite);
    BBHIP_LAUNCH_CHECK();
    return 0;
}

int backward_entry(BackwardCall const &c, void *stream)
{
    PackedInputHint const packed = g_packed_hint;
    PreparedTablesHint const tables = g_tables_hint;
    int const dw_overwrite = g_dw_overwrite_hint;
    clear_hints();                                  // hints are for the next LUT call only
    hipStream_t st = static_cast<hipStream_t>(stream);
    BBHIP_SWITCH_N(c.n, return run_backward<N>(c, st, packed, tables, dw_overwrite));
    return 0;
}

// ------------------------------------------------------------------------------------------------
//  caching allocator
// ------------------------------------------------------------------------------------------------
struct LocalHeap {
    std::mutex mtx;
    std::map<void *, size_t>      used;
    std::multimap<size_t, void *> spare;
    size_t allocated = 0, reserved = 0, max_alloc = 0;

    void *alloc(size_t size)
    {
        if (size == 0) { size = 1; }
        size = (size + 255) & ~(size_t)255;
        std::lock_guard<std::mutex> lk(mtx);
        auto it = spare.lower_bound(size);
        if (it != spare.end() && it->first <= size + size / 2) {        // best fit within 1.5x
            void *p = it->second;
            size_t sz = it->first;
            spare.erase(it);
            used[p] = sz;
            allocated += sz;
            if (allocated > max_alloc) { max_alloc = allocated; }
            return p;
        }
        void *p = nullptr;
        if (hipMalloc(&p, size) != hipSuccess) {
            (void)hipGetLastError();
            collect_locked();
            if (hipMalloc(&p, size) != hipSuccess) { (void)hipGetLastError(); return nullptr; }
        }
        used[p] = size;
        allocated += size;
        reserved += size;
        if (allocated > max_alloc) { max_alloc = allocated; }
        return p;
    }

    void release(void *p)
    {
        if (!p) { return; }
        std::lock_guard<std::mutex> lk(mtx);
        auto it = used.find(p);
        if (it == used.end()) { return; }
        size_t sz = it->second;
        used.erase(it);
        allocated -= sz;
        spare.emplace(sz, p);
        if (reserved > max_alloc + max_alloc / 2) { collect_locked(); }   // keep the reserve within 1.5x of the high-water mark
    }

    void collect_locked(void)
    {
        for (auto &kv : spare) { (void)hipFree(kv.second); reserved -= kv.first; }
        spare.clear();
    }
};

LocalHeap &heap(void) { static LocalHeap h; return h; }

int check_im2col(Im2ColArgs const &a, bool bit, char const *name)
{
    if (!(a.x && a.y)) { return fail("%s: null buffer", name); }
    if (!(a.c > 0 && a.h > 0 && a.w > 0 && a.fh > 0 && a.fw > 0 && a.oh > 0 && a.ow > 0 && a.input_frame_size > 0)) {
        return fail("%s: sizes must be positive", name);
    }
    if (!(a.x_stride > 0 && a.y_stride > 0 && a.x_offset >= 0 && a.y_offset >= 0)) { return fail("%s: bad stride or offset", name); }
    if (a.border_mode < 0 || a.border_mode > 4) { return fail("%s: border_mode=%d not in 0..4", name, a.border_mode); }
    // border modes fold an out-of-range tap back once: it must land inside the image
    if (a.border_mode != 0 &&
        (a.x_offset >= a.w || a.y_offset >= a.h || a.fw - 1 - a.x_offset + (a.ow - 1) * a.x_stride > 2 * a.w - 2 ||
         a.fh - 1 - a.y_offset + (a.oh - 1) * a.y_stride > 2 * a.h - 2)) {
        return fail("%s: filter reaches a full image size beyond the border", name);
    }
    long long const out_frames = (long long)a.input_frame_size * a.oh * a.ow;
    if (out_frames > 0x7fffffffLL) { return fail("%s: %lld output frames do not fit an int", name, out_frames); }
    long long const in_need  = bit ? (a.input_frame_size + 31) / 32 : a.input_frame_size;
    long long const out_need = bit ? (out_frames + 31) / 32 : out_frames;
    if (a.input_frame_stride < in_need || a.output_frame_stride < out_need) { return fail("%s: frame stride shorter than the frames", name); }
    if ((long long)a.c * a.h * a.w > 0x7fffffffLL || (long long)a.c * a.fh * a.fw > 0x7fffffffLL) { return fail("%s: too many nodes", name); }
    return 0;
}

constexpr int kAdamBlocksPerTensor = 1024;

template <int OP>
int vector_op(float *dst, float const *src0, float const *src1, float a, float b, float c, float d, int size, void *stream, char const *name)
{
    if (!(dst != nullptr && src0 != nullptr && (src1 != nullptr || !vec_binary<OP>()) && size >= 0)) {
        return fail("%s: rejected argument (null pointer or negative size)", name);
    }
    if (size == 0) { return 0; }
    int const aligned = ((reinterpret_cast<uintptr_t>(dst) | reinterpret_cast<uintptr_t>(src0) |
                          (vec_binary<OP>() ? reinterpret_cast<uintptr_t>(src1) : 0)) & 15) == 0;
    size_t const blocks = ((size_t)size + kVecBlock * 4 - 1) / (kVecBlock * 4);
    ScopedTimer tm(kTimeOther, static_cast<hipStream_t>(stream));
    hipLaunchKernelGGL(vector_op_kernel<OP>, dim3((unsigned)blocks), dim3(kVecBlock), 0, static_cast<hipStream_t>(stream),
                       dst, src0, src1, a, b, c, d, (size_t)size, aligned);
    BBHIP_LAUNCH_CHECK();
    return 0;
}

}  // namespace


// ================================================================================================
//  exported entry points
// ================================================================================================
extern "C" {

int bbhip_GetDeviceCount(void)
{
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess) { (void)hipGetLastError(); return 0; }
    return n;
}

int bbhip_GetDevice(void)
{
    int d = 0;
    if (hipGetDevice(&d) != hipSuccess) { (void)hipGetLastError(); return -1; }
    return d;
}

void bbhip_SetDevice(int device) { if (hipSetDevice(device) != hipSuccess) { fail("hipSetDevice(%d) failed", device); (void)hipGetLastError(); } }
void bbhip_SetHostOnly(int host_only) { g_host_only = host_only != 0; }
int  bbhip_IsHostOnly(void) { return g_host_only ? 1 : 0; }
int  bbhip_IsDeviceAvailable(void) { return (!g_host_only && bbhip_GetDeviceCount() > 0) ? 1 : 0; }
const char *bbhip_GetLastErrorString(void) { return g_last_error.c_str(); }

void  *bbhip_LocalHeap_Malloc(size_t size) { return heap().alloc(size); }
void   bbhip_LocalHeap_Free(void *ptr) { heap().release(ptr); }
size_t bbhip_LocalHeap_GetMaxAllocSize(void) { return heap().max_alloc; }
size_t bbhip_LocalHeap_GetAllocatedSize(void) { return heap().allocated; }
void   bbhip_LocalHeap_GarbageCollect(void) { std::lock_guard<std::mutex> lk(heap().mtx); heap().collect_locked(); }

int bbhip_Malloc(void **ptr, size_t size)
{
    BBHIP_REQUIRE(ptr != nullptr);
    *ptr = heap().alloc(size);
    if (!*ptr) { return fail("bbhip_Malloc: out of device memory (%zu bytes)", size); }
    return 0;
}

int bbhip_Free(void *ptr) { heap().release(ptr); return 0; }

int bbhip_MallocHost(void **ptr, size_t size)
{
    BBHIP_REQUIRE(ptr != nullptr);
    BBHIP_TRY(hipHostMalloc(ptr, size ? size : 1, hipHostMallocDefault));
    return 0;
}

int bbhip_FreeHost(void *ptr)
{
    if (ptr) { BBHIP_TRY(hipHostFree(ptr)); }
    return 0;
}

int bbhip_Memcpy(void *dst, void const *src, size_t size, int kind)
{
    BBHIP_REQUIRE(kind >= 1 && kind <= 3);
    if (size == 0) { return 0; }
    BBHIP_REQUIRE(dst != nullptr && src != nullptr);
    hipMemcpyKind const k = (kind == 1) ? hipMemcpyHostToDevice : (kind == 2) ? hipMemcpyDeviceToHost : hipMemcpyDeviceToDevice;
    BBHIP_TRY(hipMemcpy(dst, src, size, k));
    return 0;
}

int bbhip_Memset(void *dev_ptr, int value, size_t size)
{
    if (size == 0) { return 0; }
    BBHIP_REQUIRE(dev_ptr != nullptr);
    BBHIP_TRY(hipMemset(dev_ptr, value, size));
    return 0;
}

int bbhip_DeviceSynchronize(void)
{
    BBHIP_TRY(hipDeviceSynchronize());
    return 0;
}

void bbhip_KernelTimer_Enable(int enable) { g_timer_on = enable != 0; }

int bbhip_KernelTimer_Read(int which, float *total_ms, int *launches)
{
    BBHIP_REQUIRE(which >= 0 && which < kTimedKinds && total_ms != nullptr && launches != nullptr);
    // take the launches of this kind out of the list first; whatever happens below, none of them stays behind with
    // destroyed events
    std::vector<TimedLaunch> mine;
    {
        std::lock_guard<std::mutex> lk(g_timed_mtx);
        std::vector<TimedLaunch> keep;
        for (auto &t : g_timed) { (t.which == which ? mine : keep).push_back(t); }
        g_timed.swap(keep);
    }
    float total = 0.0f;
    int count = 0;
    hipError_t first_error = hipSuccess;
    for (auto &t : mine) {
        float ms = 0.0f;
        hipError_t e = hipEventSynchronize(t.stop);
        if (e == hipSuccess) { e = hipEventElapsedTime(&ms, t.start, t.stop); }
        (void)hipEventDestroy(t.start);
        (void)hipEventDestroy(t.stop);
        if (e != hipSuccess) { if (first_error == hipSuccess) { first_error = e; } continue; }
        total += ms;
        ++count;
    }
    *total_ms = total;
    *launches = count;
    if (first_error != hipSuccess) { return fail("bbhip_KernelTimer_Read: %s", hipGetErrorString(first_error)); }
    return 0;
}

int bbhip_ReserveScratch(size_t bytes)
{
    char *p = nullptr;
    return arena_get(bytes, &p, nullptr);
}

int bbhip_ReleaseScratch(void)
{
    int dev = 0;
    BBHIP_TRY(hipGetDevice(&dev));
    if (dev < 0 || dev >= kMaxDevices) { return fail("device index %d out of range", dev); }
    BBHIP_TRY(hipDeviceSynchronize());
    Arena &a = g_arena[dev];
    for (void *p : a.retired) { (void)hipFree(p); }
    a.retired.clear();
    if (a.ptr) { (void)hipFree(a.ptr); }
    a.ptr = nullptr;
    a.cap = 0;
    return 0;
}

size_t bbhip_GetScratchSize(void)
{
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) { (void)hipGetLastError(); return 0; }
    return g_arena[dev].cap;
}

int bbhip_GetSwitch(char const *name)
{
    if (!name) { return -1; }
    if (!strcmp(name, "corner")) { return use_corner_values(kXBit) ? 1 : 0; }
    if (!strcmp(name, "pack"))   { return pack_binarized_input() ? 1 : 0; }
    if (!strcmp(name, "dx_wide")) { return dx_wide_rows() ? 1 : 0; }
    if (!strcmp(name, "inline_tables")) { return inline_tables() ? 1 : 0; }
    return -1;
}

void bbhip_SetDxMode(int mode) { g_dx_mode = (mode == 1 || mode == 2) ? mode : 0; }
void bbhip_HintInputNodeSize(int input_node_size) { g_input_node_hint = input_node_size > 0 ? input_node_size : 0; }
int  bbhip_PackedRowWords(int frame_size) { return frame_size > 0 ? packed_row_words(frame_size) : 0; }
void bbhip_HintPreparedTables(float *dev_tables, size_t bytes, int holds_tables)
{
    g_tables_hint = (dev_tables != nullptr && bytes > 0) ? PreparedTablesHint{dev_tables, bytes, holds_tables != 0} : PreparedTablesHint{nullptr, 0, 0};
}

size_t bbhip_PreparedTablesBytes(int n, int node_size)
{
    if (n < 2 || n > 6 || node_size <= 0) { return 0; }
    return 2 * align256((size_t)node_size * ((size_t)1 << n) * sizeof(float));
}

void bbhip_HintTableGradientOverwrite(int overwrite) { g_dw_overwrite_hint = overwrite != 0; }

void bbhip_HintPackedOutput(int *dev_bits, int rows, int row_words)
{
    g_packed_out_hint = (dev_bits != nullptr && rows > 0 && row_words > 0) ? PackedOutputHint{reinterpret_cast<uint32_t *>(dev_bits), rows, row_words}
                                                                           : PackedOutputHint{nullptr, 0, 0};
}

void bbhip_HintPackedInput(int *dev_bits, int rows, int row_words, int holds_input)
{
    g_packed_hint = (dev_bits != nullptr && rows > 0 && row_words > 0)
                  ? PackedInputHint{reinterpret_cast<uint32_t *>(dev_bits), rows, row_words, holds_input != 0}
                  : PackedInputHint{nullptr, 0, 0, 0};
}
int  bbhip_GetDxMode(void) { return g_dx_mode; }

int bbhip_fp32_Vector_set(float *dev_dst, float a, int size, void *stream)
{
    clear_hints();                                 // a hint is for the next LUT forward call only
    BBHIP_REQUIRE(dev_dst != nullptr && size >= 0);
    if (size == 0) { return 0; }
    hipLaunchKernelGGL(fill_kernel, dim3(ceil_div(size, kBlock * 4)), dim3(kBlock), 0, static_cast<hipStream_t>(stream), dev_dst, a, (size_t)size);
    BBHIP_LAUNCH_CHECK();
    return 0;
}

int bbhip_fp32_Vector_clamp(float *dev_dst, float const *dev_src, float lo, float hi, int size, void *stream)
{
    clear_hints();                                 // a hint is for the next LUT forward call only
    BBHIP_REQUIRE(dev_dst != nullptr && dev_src != nullptr && size >= 0);
    if (size == 0) { return 0; }
    hipLaunchKernelGGL(clamp_kernel, dim3(ceil_div(size, kBlock)), dim3(kBlock), 0, static_cast<hipStream_t>(stream), dev_dst, dev_src, lo, hi, size);
    BBHIP_LAUNCH_CHECK();
    return 0;
}

int bbhip_fp32_Vector_add_ex(float *dev_dst, float const *dev_src0, float const *dev_src1, float a, float b, float c, int size, void *stream)
{
    clear_hints();
    return vector_op<kVecAddEx>(dev_dst, dev_src0, dev_src1, a, b, c, 0.0f, size, stream, __func__);
}

int bbhip_fp32_Vector_mul_ex(float *dev_dst, float const *dev_src0, float const *dev_src1, float a, float b, int size, void *stream)
{
    clear_hints();
    return vector_op<kVecMulEx>(dev_dst, dev_src0, dev_src1, a, b, 0.0f, 0.0f, size, stream, __func__);
}

int bbhip_fp32_Vector_div_ex(float *dev_dst, float const *dev_src0, float const *dev_src1, float a, float b, float c, float d, int size, void *stream)
{
    clear_hints();
    return vector_op<kVecDivEx>(dev_dst, dev_src0, dev_src1, a, b, c, d, size, stream, __func__);
}

int bbhip_fp32_Vector_sqrt(float *dev_dst, float const *dev_src, int size, void *stream)
{
    clear_hints();
    return vector_op<kVecSqrt>(dev_dst, dev_src, nullptr, 0.0f, 0.0f, 0.0f, 0.0f, size, stream, __func__);
}

int bbhip_fp32_Vector_exp(float *dev_dst, float const *dev_src, int size, void *stream)
{
    clear_hints();
    return vector_op<kVecExp>(dev_dst, dev_src, nullptr, 0.0f, 0.0f, 0.0f, 0.0f, size, stream, __func__);
}

int bbhip_fp32_Vector_min(float *dev_dst, float const *dev_src0, float const *dev_src1, int size, void *stream)
{
    clear_hints();
    return vector_op<kVecMin>(dev_dst, dev_src0, dev_src1, 0.0f, 0.0f, 0.0f, 0.0f, size, stream, __func__);
}

int bbhip_fp32_Vector_min_v(float *dev_dst, float const *dev_src, float a, int size, void *stream)
{
    clear_hints();
    return vector_op<kVecMinV>(dev_dst, dev_src, nullptr, a, 0.0f, 0.0f, 0.0f, size, stream, __func__);
}

int bbhip_fp32_Vector_max(float *dev_dst, float const *dev_src0, float const *dev_src1, int size, void *stream)
{
    clear_hints();
    return vector_op<kVecMax>(dev_dst, dev_src0, dev_src1, 0.0f, 0.0f, 0.0f, 0.0f, size, stream, __func__);
}

int bbhip_fp32_Vector_max_v(float *dev_dst, float const *dev_src, float a, int size, void *stream)
{
    clear_hints();
    return vector_op<kVecMaxV>(dev_dst, dev_src, nullptr, a, 0.0f, 0.0f, 0.0f, size, stream, __func__);
}

namespace {
int adam_entry(bool zero_grads, int size, int const *dev_size_table, float *const *dev_params_buf_table, float *const *dev_grads_buf_table,
               float *const *dev_m_buf_table, float *const *dev_v_buf_table, float lr_t, float beta1, float beta2, void *stream)
{
    clear_hints();                                 // a hint is for the next LUT forward call only
    BBHIP_REQUIRE(size >= 0 && size <= 65535);
    if (size == 0) { return 0; }
    BBHIP_REQUIRE(dev_size_table != nullptr && dev_params_buf_table != nullptr && dev_grads_buf_table != nullptr &&
                  dev_m_buf_table != nullptr && dev_v_buf_table != nullptr);
    // the element counts live on the device: a fixed number of blocks per tensor strides over its elements
    ScopedTimer tm(kTimeOther, static_cast<hipStream_t>(stream));
    dim3 const grid(kAdamBlocksPerTensor, (unsigned)size), block(kVecBlock);
    if (zero_grads) {
        hipLaunchKernelGGL(adam_kernel<true>, grid, block, 0, static_cast<hipStream_t>(stream),
                           dev_size_table, dev_params_buf_table, dev_grads_buf_table, dev_m_buf_table, dev_v_buf_table,
                           lr_t, 1.0f - beta1, 1.0f - beta2);
    }
    else {
        hipLaunchKernelGGL(adam_kernel<false>, grid, block, 0, static_cast<hipStream_t>(stream),
                           dev_size_table, dev_params_buf_table, dev_grads_buf_table, dev_m_buf_table, dev_v_buf_table,
                           lr_t, 1.0f - beta1, 1.0f - beta2);
    }
    BBHIP_LAUNCH_CHECK();
    return 0;
}
}  // namespace

int bbhip_fp32_OptimizerAdam(int size, int const *dev_size_table, float *const *dev_params_buf_table, float *const *dev_grads_buf_table,
                             float *const *dev_m_buf_table, float *const *dev_v_buf_table, float lr_t, float beta1, float beta2, void *stream)
{
    return adam_entry(false, size, dev_size_table, dev_params_buf_table, dev_grads_buf_table, dev_m_buf_table, dev_v_buf_table, lr_t, beta1, beta2, stream);
}

int bbhip_fp32_OptimizerAdam_Update(int size, int const *dev_size_table, float *const *dev_params_buf_table, float *const *dev_grads_buf_table,
                                    float *const *dev_m_buf_table, float *const *dev_v_buf_table, float lr_t, float beta1, float beta2, void *stream)
{
    return adam_entry(true, size, dev_size_table, dev_params_buf_table, dev_grads_buf_table, dev_m_buf_table, dev_v_buf_table, lr_t, beta1, beta2, stream);
}

int bbhip_fp32_Im2Col_Forward(float const *dev_x_buf, float *dev_y_buf, int x_stride, int y_stride, int x_offset, int y_offset,
                              int input_frame_size, int input_frame_stride, int input_w_size, int input_h_size, int input_c_size,
                              int output_w_size, int output_h_size, int output_frame_stride, int filter_w_size, int filter_h_size,
                              int border_mode, float border_value, void *stream)
{
    clear_hints();                                 // a hint is for the next LUT forward call only
    Im2ColArgs a{dev_x_buf, dev_y_buf, x_stride, y_stride, x_offset, y_offset, input_frame_size, input_frame_stride, input_w_size,
                 input_h_size, input_c_size, output_w_size, output_h_size, output_frame_stride, filter_w_size, filter_h_size,
                 border_mode, border_value, 0, 0};
    if (check_im2col(a, false, __func__)) { return 1; }
    if ((long long)a.oh * a.ow > 0x7fffffffLL) { return fail("%s: output plane too large", __func__); }
    a.q_tiles = ceil_div(a.oh * a.ow, kTile);
    a.f_tiles  = ceil_div(a.input_frame_size, kTile);
    long long const blocks = (long long)a.c * a.fh * a.fw * a.q_tiles * a.f_tiles;
    if (blocks > 0x7fffffffLL) { return fail("%s: grid too large", __func__); }
    ScopedTimer tm(kTimeOther, static_cast<hipStream_t>(stream));
    hipLaunchKernelGGL(im2col_forward_kernel, dim3((unsigned)blocks), dim3(kConvBlock), 0, static_cast<hipStream_t>(stream), a);
    BBHIP_LAUNCH_CHECK();
    return 0;
}

int bbhip_bit_Im2Col_Forward(int const *dev_x_buf, int *dev_y_buf, int x_stride, int y_stride, int x_offset, int y_offset,
                             int input_frame_size, int input_frame_stride, int input_w_size, int input_h_size, int input_c_size,
                             int output_w_size, int output_h_size, int output_frame_stride, int filter_w_size, int filter_h_size,
                             int border_mode, void *stream)
{
    clear_hints();                                 // a hint is for the next LUT forward call only
    Im2ColArgs a{dev_x_buf, dev_y_buf, x_stride, y_stride, x_offset, y_offset, input_frame_size, input_frame_stride, input_w_size,
                 input_h_size, input_c_size, output_w_size, output_h_size, output_frame_stride, filter_w_size, filter_h_size,
                 border_mode, 0.0f, 0, 0};
    if (check_im2col(a, true, __func__)) { return 1; }
    long long const out_frames = (long long)a.input_frame_size * a.oh * a.ow;
    int const words = (int)((out_frames + 31) / 32);
    long long const total = (long long)a.c * a.fh * a.fw * words;
    long long const blocks = (total + kConvBlock - 1) / kConvBlock;
    if (blocks > 0x7fffffffLL) { return fail("%s: grid too large", __func__); }
    ScopedTimer tm(kTimeOther, static_cast<hipStream_t>(stream));
    hipLaunchKernelGGL(im2col_forward_bit_kernel, dim3((unsigned)blocks), dim3(kConvBlock), 0, static_cast<hipStream_t>(stream), a, words, total);
    BBHIP_LAUNCH_CHECK();
    return 0;
}

int bbhip_fp32_Im2Col_Backward(float const *dev_dy_buf, float *dev_dx_buf, int x_stride, int y_stride, int x_offset, int y_offset,
                               int input_frame_size, int input_frame_stride, int input_w_size, int input_h_size, int input_c_size,
                               int output_w_size, int output_h_size, int output_frame_stride, int filter_w_size, int filter_h_size,
                               void *stream)
{
    clear_hints();                                 // a hint is for the next LUT forward call only
    Im2ColArgs a{dev_dy_buf, dev_dx_buf, x_stride, y_stride, x_offset, y_offset, input_frame_size, input_frame_stride, input_w_size,
                 input_h_size, input_c_size, output_w_size, output_h_size, output_frame_stride, filter_w_size, filter_h_size,
                 0, 0.0f, 0, 0};
    if (check_im2col(a, false, __func__)) { return 1; }
    if ((long long)a.h * a.w > 0x7fffffffLL) { return fail("%s: image too large", __func__); }
    int const p_tiles = ceil_div(a.h * a.w, kTile);
    // 64 frames per block, or 16 when that leaves fewer than eight blocks per compute unit
    int const tf = ((long long)a.c * p_tiles * ceil_div(a.input_frame_size, 64) >= 2048) ? 64 : 16;
    a.f_tiles = ceil_div(a.input_frame_size, tf);
    long long const blocks = (long long)a.c * p_tiles * a.f_tiles;
    if (blocks > 0x7fffffffLL) { return fail("%s: grid too large", __func__); }
    ScopedTimer tm(kTimeOther, static_cast<hipStream_t>(stream));
    if (tf == 64) { hipLaunchKernelGGL(im2col_backward_kernel<64>, dim3((unsigned)blocks), dim3(kConvBlock), 0, static_cast<hipStream_t>(stream), a, p_tiles); }
    else          { hipLaunchKernelGGL(im2col_backward_kernel<16>, dim3((unsigned)blocks), dim3(kConvBlock), 0, static_cast<hipStream_t>(stream), a, p_tiles); }
    BBHIP_LAUNCH_CHECK();
    return 0;
}

static int check_col2im(void const *p, void const *q, int w, int h, int c, int narrow_stride, int frames, int wide_stride, bool bit, char const *name)
{
    if (!(p && q)) { return fail("%s: null buffer", name); }
    if (!(w > 0 && h > 0 && c > 0 && frames > 0)) { return fail("%s: sizes must be positive", name); }
    long long const narrow = (long long)frames * h * w;
    if (narrow > 0x7fffffffLL) { return fail("%s: %lld input frames do not fit an int", name, narrow); }
    if (narrow_stride < (bit ? (narrow + 31) / 32 : narrow) || wide_stride < (bit ? (frames + 31) / 32 : frames)) {
        return fail("%s: frame stride shorter than the frames", name);
    }
    if ((long long)c * h * w > 0x7fffffffLL) { return fail("%s: too many nodes", name); }
    return 0;
}

int bbhip_fp32_Col2Im_Forward(float const *dev_x_buf, float *dev_y_buf, int w_size, int h_size, int c_size, int input_frame_stride,
                              int output_frame_size, int output_frame_stride, void *stream)
{
    clear_hints();                                 // a hint is for the next LUT forward call only
    if (check_col2im(dev_x_buf, dev_y_buf, w_size, h_size, c_size, input_frame_stride, output_frame_size, output_frame_stride, false, __func__)) { return 1; }
    int const hw = h_size * w_size, xy_tiles = ceil_div(hw, kTile), f_tiles = ceil_div(output_frame_size, kTile);
    long long const blocks = (long long)c_size * xy_tiles * f_tiles;
    if (blocks > 0x7fffffffLL) { return fail("%s: grid too large", __func__); }
    ScopedTimer tm(kTimeOther, static_cast<hipStream_t>(stream));
    hipLaunchKernelGGL(col2im_kernel<true>, dim3((unsigned)blocks), dim3(kConvBlock), 0, static_cast<hipStream_t>(stream),
                       dev_x_buf, dev_y_buf, hw, c_size, input_frame_stride, output_frame_size, output_frame_stride, xy_tiles, f_tiles);
    BBHIP_LAUNCH_CHECK();
    return 0;
}

int bbhip_fp32_Col2Im_Backward(float const *dev_dy_buf, float *dev_dx_buf, int w_size, int h_size, int c_size, int input_frame_stride,
                               int output_frame_size, int output_frame_stride, void *stream)
{
    clear_hints();                                 // a hint is for the next LUT forward call only
    if (check_col2im(dev_dy_buf, dev_dx_buf, w_size, h_size, c_size, input_frame_stride, output_frame_size, output_frame_stride, false, __func__)) { return 1; }
    int const hw = h_size * w_size, xy_tiles = ceil_div(hw, kTile), f_tiles = ceil_div(output_frame_size, kTile);
    long long const blocks = (long long)c_size * xy_tiles * f_tiles;
    if (blocks > 0x7fffffffLL) { return fail("%s: grid too large", __func__); }
    ScopedTimer tm(kTimeOther, static_cast<hipStream_t>(stream));
    hipLaunchKernelGGL(col2im_kernel<false>, dim3((unsigned)blocks), dim3(kConvBlock), 0, static_cast<hipStream_t>(stream),
                       dev_dy_buf, dev_dx_buf, hw, c_size, input_frame_stride, output_frame_size, output_frame_stride, xy_tiles, f_tiles);
    BBHIP_LAUNCH_CHECK();
    return 0;
}

int bbhip_bit_Col2Im_Forward(int const *dev_x_buf, int *dev_y_buf, int w_size, int h_size, int c_size, int input_frame_stride,
                             int output_frame_size, int output_frame_stride, void *stream)
{
    clear_hints();                                 // a hint is for the next LUT forward call only
    if (check_col2im(dev_x_buf, dev_y_buf, w_size, h_size, c_size, input_frame_stride, output_frame_size, output_frame_stride, true, __func__)) { return 1; }
    int const hw = h_size * w_size, words = (output_frame_size + 31) / 32;
    long long const total = (long long)c_size * hw * words;
    long long const blocks = (total + kConvBlock - 1) / kConvBlock;
    if (blocks > 0x7fffffffLL) { return fail("%s: grid too large", __func__); }
    ScopedTimer tm(kTimeOther, static_cast<hipStream_t>(stream));
    hipLaunchKernelGGL(col2im_forward_bit_kernel, dim3((unsigned)blocks), dim3(kConvBlock), 0, static_cast<hipStream_t>(stream),
                       reinterpret_cast<uint32_t const *>(dev_x_buf), reinterpret_cast<uint32_t *>(dev_y_buf), hw, input_frame_stride,
                       output_frame_size, output_frame_stride, words, total);
    BBHIP_LAUNCH_CHECK();
    return 0;
}

static int launch_pool(PoolArgs const &a, bool backward, void *stream, char const *name)
{
    if (!(a.x && a.out && (a.dy || !backward))) { return fail("%s: null buffer", name); }
    if (!(a.w > 0 && a.h > 0 && a.c > 0 && a.frame_size > 0)) { return fail("%s: sizes must be positive", name); }
    if (a.ow != (a.w + 1) / 2 || a.oh != (a.h + 1) / 2) { return fail("%s: output size must be ceil(input / 2)", name); }
    if (a.frame_stride < a.frame_size) { return fail("%s: frame stride shorter than the frames", name); }
    // four frames per thread with 128-bit accesses where every row starts on 16 bytes
    uintptr_t const bits = reinterpret_cast<uintptr_t>(a.x) | reinterpret_cast<uintptr_t>(a.out) | reinterpret_cast<uintptr_t>(backward ? a.dy : a.x);
    bool const wide = (bits & 15u) == 0 && (a.frame_stride & 3) == 0;
    int const f_blocks = ceil_div(a.frame_size, kConvBlock * (wide ? 4 : 1));
    long long const blocks = (long long)a.c * a.oh * a.ow * f_blocks;
    if (blocks > 0x7fffffffLL) { return fail("%s: grid too large", name); }
    hipStream_t const st = static_cast<hipStream_t>(stream);
    ScopedTimer tm(kTimeOther, st);
    dim3 const grid((unsigned)blocks), block(kConvBlock);
    if (backward) { if (wide) { hipLaunchKernelGGL((stochastic_maxpool2x2_backward_kernel<4>), grid, block, 0, st, a, f_blocks); }
                    else      { hipLaunchKernelGGL((stochastic_maxpool2x2_backward_kernel<1>), grid, block, 0, st, a, f_blocks); } }
    else          { if (wide) { hipLaunchKernelGGL((stochastic_maxpool2x2_forward_kernel<4>), grid, block, 0, st, a, f_blocks); }
                    else      { hipLaunchKernelGGL((stochastic_maxpool2x2_forward_kernel<1>), grid, block, 0, st, a, f_blocks); } }
    BBHIP_LAUNCH_CHECK();
    return 0;
}

int bbhip_fp32_StochasticMaxPooling2x2_Forward(float const *dev_x_buf, float *dev_y_buf, int input_w_size, int input_h_size,
                                               int output_w_size, int output_h_size, int c_size, int frame_size, int frame_stride, void *stream)
{
    clear_hints();                                 // a hint is for the next LUT forward call only
    PoolArgs a{dev_x_buf, nullptr, dev_y_buf, input_w_size, input_h_size, output_w_size, output_h_size, c_size, frame_size, frame_stride};
    return launch_pool(a, false, stream, __func__);
}

int bbhip_fp32_StochasticMaxPooling2x2_Backward(float const *dev_x_buf, float const *dev_dy_buf, float *dev_dx_buf, int input_w_size,
                                                int input_h_size, int output_w_size, int output_h_size, int c_size, int frame_size,
                                                int frame_stride, void *stream)
{
    clear_hints();                                 // a hint is for the next LUT forward call only
    PoolArgs a{dev_x_buf, dev_dy_buf, dev_dx_buf, input_w_size, input_h_size, output_w_size, output_h_size, c_size, frame_size, frame_stride};
    return launch_pool(a, true, stream, __func__);
}

// The backward passes of AverageLut and MaxLut are input-centric.  A table that fits one LDS piece can be walked whole by every
// wavefront (no reverse wiring, one launch instead of two); that costs table entries x wavefronts comparisons, so it is taken only
// while that product stays below what the saved launch costs (the tail of a classifier at a training batch: 70 entries, 70 input
// nodes, 1024 frames).  Both ways add in table order: the same bits.
static bool walk_whole_table(int total, int input_node_size, int frame_size)
{
    if (total > kReversePiece) { return false; }
    return (long long)total * input_node_size * ceil_div(frame_size, kWave) <= 131072LL;
}

static int check_average_lut(void const *a, void const *b, int const *idx, int n, int node_size, int frame_size, int frame_stride, int row_items,
                             char const *name)
{
    if (!(a && b && idx)) { return fail("%s: null buffer", name); }
    if (!(n > 0 && node_size > 0 && frame_size > 0)) { return fail("%s: sizes must be positive", name); }
    if (frame_stride < row_items) { return fail("%s: frame stride shorter than the frames", name); }
    if ((long long)node_size * n > 0x7fffffffLL) { return fail("%s: connection table too large", name); }
    return 0;
}

static int average_lut_forward(float const *dev_x_buf, float *dev_y_buf, int const *dev_input_index, int n, int node_size, int frame_size,
                               int frame_stride, int binarize_input, int binarize_output, bool mean, void *stream, char const *name)
{
    clear_hints();                                 // a hint is for the next LUT forward call only
    if (check_average_lut(dev_x_buf, dev_y_buf, dev_input_index, n, node_size, frame_size, frame_stride, frame_size, name)) { return 1; }
    int const f_blocks = ceil_div(frame_size, kTailBlock);
    long long const blocks = (long long)node_size * f_blocks;
    if (blocks > 0x7fffffffLL) { return fail("%s: grid too large", name); }
    ScopedTimer tm(kTimeOther, static_cast<hipStream_t>(stream));
    hipLaunchKernelGGL(average_lut_forward_kernel, dim3((unsigned)blocks), dim3(kTailBlock), 0, static_cast<hipStream_t>(stream), dev_x_buf,
                       dev_y_buf, dev_input_index, n, frame_size, frame_stride, binarize_input, binarize_output, f_blocks,
                       mean ? 1.0f / (float)n : 1.0f);
    BBHIP_LAUNCH_CHECK();
    return 0;
}

int bbhip_fp32_AverageLut_Forward(float const *dev_x_buf, float *dev_y_buf, int const *dev_input_index, int n, int node_size, int frame_size,
                                  int frame_stride, int binarize_input, int binarize_output, void *stream)
{
    return average_lut_forward(dev_x_buf, dev_y_buf, dev_input_index, n, node_size, frame_size, frame_stride, binarize_input, binarize_output,
                               true, stream, __func__);
}

int bbhip_fp32_AverageLut_ForwardSum(float const *dev_x_buf, float *dev_y_buf, int const *dev_input_index, int n, int node_size, int frame_size,
                                     int frame_stride, int binarize_input, int binarize_output, void *stream)
{
    return average_lut_forward(dev_x_buf, dev_y_buf, dev_input_index, n, node_size, frame_size, frame_stride, binarize_input, binarize_output,
                               false, stream, __func__);
}

int bbhip_bit_AverageLut_Forward(int const *dev_x_buf, int *dev_y_buf, int const *dev_input_index, int n, int node_size, int frame_size,
                                 int frame_stride, void *stream)
{
    clear_hints();                                 // a hint is for the next LUT forward call only
    int const words = (frame_size > 0) ? ceil_div(frame_size, 32) : 0;
    if (check_average_lut(dev_x_buf, dev_y_buf, dev_input_index, n, node_size, frame_size, frame_stride, words, __func__)) { return 1; }
    int const w_blocks = ceil_div(words, kTailBlock);
    long long const blocks = (long long)node_size * w_blocks;
    if (blocks > 0x7fffffffLL) { return fail("%s: grid too large", __func__); }
    int planes = 1;
    while ((1 << planes) <= n && planes < 31) { ++planes; }      // planes = bits of n: counts 0..n fit
    dim3 const grid((unsigned)blocks), block(kTailBlock);
    hipStream_t const st = static_cast<hipStream_t>(stream);
    ScopedTimer tm(kTimeOther, st);
#define BBHIP_AVERAGE_BIT(P) hipLaunchKernelGGL(average_lut_forward_bit_kernel<P>, grid, block, 0, st, dev_x_buf, dev_y_buf, dev_input_index, n, words, frame_stride, w_blocks)
    switch (planes) {
    case 1: BBHIP_AVERAGE_BIT(1); break;
    case 2: BBHIP_AVERAGE_BIT(2); break;
    case 3: BBHIP_AVERAGE_BIT(3); break;
    case 4: BBHIP_AVERAGE_BIT(4); break;
    case 5: BBHIP_AVERAGE_BIT(5); break;
    case 6: BBHIP_AVERAGE_BIT(6); break;
    case 7: BBHIP_AVERAGE_BIT(7); break;
    case 8: BBHIP_AVERAGE_BIT(8); break;
    default:
        hipLaunchKernelGGL(average_lut_forward_bit_wide_kernel, grid, block, 0, st, dev_x_buf, dev_y_buf, dev_input_index, n, words, frame_stride, w_blocks);
    }
#undef BBHIP_AVERAGE_BIT
    BBHIP_LAUNCH_CHECK();
    return 0;
}

int bbhip_fp32_AverageLut_Backward(float const *dev_dy_buf, float *dev_dx_buf, int const *dev_input_index, int n, int input_node_size,
                                   int output_node_size, int frame_size, int frame_stride, void *stream)
{
    clear_hints();                                 // a hint is for the next LUT forward call only
    if (check_average_lut(dev_dy_buf, dev_dx_buf, dev_input_index, n, output_node_size, frame_size, frame_stride, frame_size, __func__)) { return 1; }
    if (input_node_size <= 0) { return fail("%s: sizes must be positive", __func__); }
    int const total = output_node_size * n;
    int const f_blocks = ceil_div(frame_stride, kTailBlock);
    long long const blocks = (long long)input_node_size * f_blocks;
    if (blocks > 0x7fffffffLL) { return fail("%s: grid too large", __func__); }
    hipStream_t const st = static_cast<hipStream_t>(stream);
    if (walk_whole_table(total, input_node_size, frame_size)) {
        ScopedTimer tm(kTimeOther, st);
        hipLaunchKernelGGL(average_lut_backward_small_kernel, dim3((unsigned)blocks), dim3(kTailBlock), 0, st, dev_dy_buf, dev_dx_buf, dev_input_index,
                           total, n, frame_size, frame_stride, f_blocks);
        BBHIP_LAUNCH_CHECK();
        return 0;
    }
    char *scratch = nullptr;
    size_t const offsets_bytes = align256(sizeof(int) * ((size_t)input_node_size + 1));
    if (arena_get(offsets_bytes + sizeof(int) * (size_t)total, &scratch, static_cast<hipStream_t>(stream))) { return 1; }
    int *offsets = reinterpret_cast<int *>(scratch), *list = reinterpret_cast<int *>(scratch + offsets_bytes);
    ScopedTimer tm(kTimeOther, static_cast<hipStream_t>(stream));
    hipLaunchKernelGGL(average_lut_reverse_kernel, dim3((unsigned)ceil_div(input_node_size + 1, kTailBlock)), dim3(kTailBlock), 0, st,
                       dev_input_index, total, n, input_node_size, offsets, list, 0);
    BBHIP_LAUNCH_CHECK();
    hipLaunchKernelGGL(average_lut_backward_kernel, dim3((unsigned)blocks), dim3(kTailBlock), 0, st, dev_dy_buf, dev_dx_buf, offsets, list, n,
                       frame_size, frame_stride, f_blocks);
    BBHIP_LAUNCH_CHECK();
    return 0;
}

int bbhip_fp32_MaxLut_Forward(float const *dev_x_buf, float *dev_y_buf, int const *dev_input_index, int n, int node_size, int frame_size,
                              int frame_stride, int binarize_input, int binarize_output, void *stream)
{
    clear_hints();                                 // a hint is for the next LUT forward call only
    if (check_average_lut(dev_x_buf, dev_y_buf, dev_input_index, n, node_size, frame_size, frame_stride, frame_size, __func__)) { return 1; }
    int const f_blocks = ceil_div(frame_size, kTailBlock);
    long long const blocks = (long long)node_size * f_blocks;
    if (blocks > 0x7fffffffLL) { return fail("%s: grid too large", __func__); }
    ScopedTimer tm(kTimeOther, static_cast<hipStream_t>(stream));
    hipLaunchKernelGGL(max_lut_forward_kernel, dim3((unsigned)blocks), dim3(kTailBlock), 0, static_cast<hipStream_t>(stream), dev_x_buf,
                       dev_y_buf, dev_input_index, n, frame_size, frame_stride, binarize_input, binarize_output, f_blocks);
    BBHIP_LAUNCH_CHECK();
    return 0;
}

int bbhip_bit_MaxLut_Forward(int const *dev_x_buf, int *dev_y_buf, int const *dev_input_index, int n, int node_size, int frame_size,
                             int frame_stride, void *stream)
{
    clear_hints();                                 // a hint is for the next LUT forward call only
    int const words = (frame_size > 0) ? ceil_div(frame_size, 32) : 0;
    if (check_average_lut(dev_x_buf, dev_y_buf, dev_input_index, n, node_size, frame_size, frame_stride, words, __func__)) { return 1; }
    int const w_blocks = ceil_div(words, kTailBlock);
    long long const blocks = (long long)node_size * w_blocks;
    if (blocks > 0x7fffffffLL) { return fail("%s: grid too large", __func__); }
    ScopedTimer tm(kTimeOther, static_cast<hipStream_t>(stream));
    hipLaunchKernelGGL(max_lut_forward_bit_kernel, dim3((unsigned)blocks), dim3(kTailBlock), 0, static_cast<hipStream_t>(stream), dev_x_buf,
                       dev_y_buf, dev_input_index, n, words, frame_stride, w_blocks);
    BBHIP_LAUNCH_CHECK();
    return 0;
}

// x: fp32 rows (bits == false) or packed rows of x_stride words; dy and dx: fp32 rows of dy_stride
static int launch_max_lut_backward(void const *x, bool bits, float const *dy, float *dx, int const *idx, int n, int input_node_size,
                                   int output_node_size, int frame_size, int x_stride, int dy_stride, int binarize_input, void *stream,
                                   char const *name)
{
    if (check_average_lut(dy, dx, idx, n, output_node_size, frame_size, dy_stride, frame_size, name)) { return 1; }
    if (x == nullptr) { return fail("%s: null buffer", name); }
    if (input_node_size <= 0) { return fail("%s: sizes must be positive", name); }
    if (x_stride < (bits ? ceil_div(frame_size, 32) : frame_size)) { return fail("%s: frame stride shorter than the frames", name); }
    int const total = output_node_size * n;
    int const f_blocks = ceil_div(dy_stride, kTailBlock);
    long long const blocks = (long long)input_node_size * f_blocks;
    if (blocks > 0x7fffffffLL) { return fail("%s: grid too large", name); }
    hipStream_t const st = static_cast<hipStream_t>(stream);
    if (walk_whole_table(total, input_node_size, frame_size)) {
        ScopedTimer tm(kTimeOther, st);
        if (bits) {
            hipLaunchKernelGGL(max_lut_backward_small_kernel<true>, dim3((unsigned)blocks), dim3(kTailBlock), 0, st, x, dy, dx, idx, total, n,
                               frame_size, x_stride, dy_stride, 0, f_blocks);
        }
        else {
            hipLaunchKernelGGL(max_lut_backward_small_kernel<false>, dim3((unsigned)blocks), dim3(kTailBlock), 0, st, x, dy, dx, idx, total, n,
                               frame_size, x_stride, dy_stride, binarize_input, f_blocks);
        }
        BBHIP_LAUNCH_CHECK();
        return 0;
    }
    char *scratch = nullptr;
    size_t const offsets_bytes = align256(sizeof(int) * ((size_t)input_node_size + 1));
    if (arena_get(offsets_bytes + sizeof(int) * (size_t)total, &scratch, st)) { return 1; }
    int *offsets = reinterpret_cast<int *>(scratch), *list = reinterpret_cast<int *>(scratch + offsets_bytes);
    ScopedTimer tm(kTimeOther, st);
    hipLaunchKernelGGL(average_lut_reverse_kernel, dim3((unsigned)ceil_div(input_node_size + 1, kTailBlock)), dim3(kTailBlock), 0, st,
                       idx, total, n, input_node_size, offsets, list, 1);
    BBHIP_LAUNCH_CHECK();
    if (bits) {
        hipLaunchKernelGGL(max_lut_backward_kernel<true>, dim3((unsigned)blocks), dim3(kTailBlock), 0, st, x, dy, dx, idx, offsets, list, n,
                           frame_size, x_stride, dy_stride, 0, f_blocks);
    }
    else {
        hipLaunchKernelGGL(max_lut_backward_kernel<false>, dim3((unsigned)blocks), dim3(kTailBlock), 0, st, x, dy, dx, idx, offsets, list, n,
                           frame_size, x_stride, dy_stride, binarize_input, f_blocks);
    }
    BBHIP_LAUNCH_CHECK();
    return 0;
}

int bbhip_fp32_MaxLut_Backward(float const *dev_x_buf, float const *dev_dy_buf, float *dev_dx_buf, int const *dev_input_index, int n,
                               int input_node_size, int output_node_size, int frame_size, int frame_stride, int binarize_input, void *stream)
{
    clear_hints();                                 // a hint is for the next LUT forward call only
    return launch_max_lut_backward(dev_x_buf, false, dev_dy_buf, dev_dx_buf, dev_input_index, n, input_node_size, output_node_size, frame_size,
                                   frame_stride, frame_stride, binarize_input, stream, __func__);
}

int bbhip_bit_fp32_MaxLut_Backward(int const *dev_x_buf, float const *dev_dy_buf, float *dev_dx_buf, int const *dev_input_index, int n,
                                   int input_node_size, int output_node_size, int frame_size, int x_frame_stride, int dy_frame_stride,
                                   void *stream)
{
    clear_hints();                                 // a hint is for the next LUT forward call only
    return launch_max_lut_backward(dev_x_buf, true, dev_dy_buf, dev_dx_buf, dev_input_index, n, input_node_size, output_node_size, frame_size,
                                   x_frame_stride, dy_frame_stride, 0, stream, __func__);
}

static int launch_reduce_forward(void const *x, bool bits, float *y, int input_node_size, int output_node_size, int frame_size,
                                 int x_stride, int y_stride, void *stream, char const *name)
{
    if (!(x && y)) { return fail("%s: null buffer", name); }
    if (!(input_node_size > 0 && output_node_size > 0 && frame_size > 0)) { return fail("%s: sizes must be positive", name); }
    if (input_node_size % output_node_size != 0) { return fail("%s: the input nodes must be a multiple of the output nodes", name); }
    if (x_stride < (bits ? ceil_div(frame_size, 32) : frame_size) || y_stride < frame_size) { return fail("%s: frame stride shorter than the frames", name); }
    int const f_blocks = ceil_div(frame_size, kTailBlock);
    long long const blocks = (long long)output_node_size * f_blocks;
    if (blocks > 0x7fffffffLL) { return fail("%s: grid too large", name); }
    hipStream_t const st = static_cast<hipStream_t>(stream);
    int const mux = input_node_size / output_node_size;
    ScopedTimer tm(kTimeOther, st);
    if (bits) { hipLaunchKernelGGL(reduce_forward_kernel<true>, dim3((unsigned)blocks), dim3(kTailBlock), 0, st, x, y, mux, output_node_size, frame_size, x_stride, y_stride, f_blocks); }
    else      { hipLaunchKernelGGL(reduce_forward_kernel<false>, dim3((unsigned)blocks), dim3(kTailBlock), 0, st, x, y, mux, output_node_size, frame_size, x_stride, y_stride, f_blocks); }
    BBHIP_LAUNCH_CHECK();
    return 0;
}

int bbhip_fp32_Reduce_Forward(float const *dev_x_buf, float *dev_y_buf, int input_node_size, int output_node_size, int frame_size,
                              int frame_stride, void *stream)
{
    clear_hints();                                 // a hint is for the next LUT forward call only
    return launch_reduce_forward(dev_x_buf, false, dev_y_buf, input_node_size, output_node_size, frame_size, frame_stride, frame_stride, stream, __func__);
}

int bbhip_bit_fp32_Reduce_Forward(int const *dev_x_buf, float *dev_y_buf, int input_node_size, int output_node_size, int frame_size,
                                  int x_frame_stride, int y_frame_stride, void *stream)
{
    clear_hints();                                 // a hint is for the next LUT forward call only
    return launch_reduce_forward(dev_x_buf, true, dev_y_buf, input_node_size, output_node_size, frame_size, x_frame_stride, y_frame_stride, stream, __func__);
}

int bbhip_fp32_Reduce_Backward(float const *dev_dy_buf, float *dev_dx_buf, int input_node_size, int output_node_size, int frame_size,
                               int frame_stride, void *stream)
{
    clear_hints();                                 // a hint is for the next LUT forward call only
    if (!(dev_dy_buf && dev_dx_buf)) { return fail("%s: null buffer", __func__); }
    if (!(input_node_size > 0 && output_node_size > 0 && frame_size > 0)) { return fail("%s: sizes must be positive", __func__); }
    if (input_node_size % output_node_size != 0) { return fail("%s: the input nodes must be a multiple of the output nodes", __func__); }
    if (frame_stride < frame_size) { return fail("%s: frame stride shorter than the frames", __func__); }
    int const f_blocks = ceil_div(frame_size, kTailBlock);
    long long const blocks = (long long)input_node_size * f_blocks;
    if (blocks > 0x7fffffffLL) { return fail("%s: grid too large", __func__); }
    ScopedTimer tm(kTimeOther, static_cast<hipStream_t>(stream));
    hipLaunchKernelGGL(reduce_backward_kernel, dim3((unsigned)blocks), dim3(kTailBlock), 0, static_cast<hipStream_t>(stream), dev_dy_buf, dev_dx_buf,
                       input_node_size / output_node_size, output_node_size, frame_size, frame_stride, f_blocks);
    BBHIP_LAUNCH_CHECK();
    return 0;
}

static int launch_mean_squared_error(float const *y, float const *t, float *dy, double *buf, int buf_size, int node_size, int frame_size,
                                     int frame_stride, float grad_scale, double loss_scale, bool loss, void *stream, char const *name)
{
    if (!(y && t && buf && (dy || !loss))) { return fail("%s: null buffer", name); }
    if (!(node_size > 0 && frame_size > 0 && buf_size > 0)) { return fail("%s: sizes must be positive", name); }
    if (frame_stride < frame_size) { return fail("%s: frame stride shorter than the frames", name); }
    int const groups = ceil_div(node_size, kMseNodes), f_blocks = ceil_div(frame_size, kTailBlock);
    long long const blocks = (long long)groups * f_blocks;
    if (blocks > 0x7fffffffLL) { return fail("%s: grid too large", name); }
    hipStream_t const st = static_cast<hipStream_t>(stream);
    char *scratch = nullptr;
    if (arena_get(sizeof(double) * (size_t)groups * (size_t)frame_size, &scratch, st)) { return 1; }
    double *partial = reinterpret_cast<double *>(scratch);
    ScopedTimer tm(kTimeOther, st);
    if (loss) {
        hipLaunchKernelGGL(mean_squared_error_kernel<true>, dim3((unsigned)blocks), dim3(kTailBlock), 0, st, y, t, dy, partial, grad_scale, loss_scale,
                           node_size, frame_size, frame_stride, f_blocks);
    }
    else {
        hipLaunchKernelGGL(mean_squared_error_kernel<false>, dim3((unsigned)blocks), dim3(kTailBlock), 0, st, y, t, dy, partial, grad_scale, loss_scale,
                           node_size, frame_size, frame_stride, f_blocks);
    }
    BBHIP_LAUNCH_CHECK();
    hipLaunchKernelGGL(mean_squared_error_sum_kernel, dim3((unsigned)ceil_div(buf_size < frame_size ? buf_size : frame_size, kTailBlock)), dim3(kTailBlock),
                       0, st, partial, buf, buf_size, groups, frame_size);
    BBHIP_LAUNCH_CHECK();
    return 0;
}

int bbhip_fp32_LossMeanSquaredError(float const *dev_y_buf, float const *dev_t_buf, float *dev_dy_buf, double *dev_loss_buf, int loss_buf_size,
                                    int node_size, int frame_size, int frame_stride, float grad_reduction, double loss_reduction, void *stream)
{
    clear_hints();                                 // a hint is for the next LUT forward call only
    return launch_mean_squared_error(dev_y_buf, dev_t_buf, dev_dy_buf, dev_loss_buf, loss_buf_size, node_size, frame_size, frame_stride,
                                     grad_reduction, loss_reduction, true, stream, __func__);
}

int bbhip_fp32_MetricsMeanSquaredError(float const *dev_y_buf, float const *dev_t_buf, double *dev_accuracy_buf, int accuracy_buf_size,
                                       int node_size, int frame_size, int frame_stride, void *stream)
{
    clear_hints();                                 // a hint is for the next LUT forward call only
    return launch_mean_squared_error(dev_y_buf, dev_t_buf, nullptr, dev_accuracy_buf, accuracy_buf_size, node_size, frame_size, frame_stride,
                                     0.0f, (double)node_size, false, stream, __func__);
}

int bbhip_fp32_LossSoftmaxCrossEntropy(float const *dev_y_buf, float const *dev_t_buf, float *dev_dy_buf, double *dev_loss_buf, float t_sum,
                                       int pix_size, int ch_size, int frame_size, int frame_stride, void *stream)
{
    clear_hints();                                 // a hint is for the next LUT forward call only
    if (!(dev_y_buf && dev_t_buf && dev_dy_buf && dev_loss_buf)) { return fail("%s: null buffer", __func__); }
    if (!(pix_size > 0 && ch_size > 0 && frame_size > 0)) { return fail("%s: sizes must be positive", __func__); }
    if (frame_stride < frame_size) { return fail("%s: frame stride shorter than the frames", __func__); }
    if ((long long)pix_size * ch_size > 0x7fffffffLL) { return fail("%s: node count too large", __func__); }
    int const f_blocks = ceil_div(frame_size, kTailBlock);
    long long const blocks = (long long)pix_size * f_blocks;
    if (blocks > 0x7fffffffLL) { return fail("%s: grid too large", __func__); }
    hipStream_t const st = static_cast<hipStream_t>(stream);
    double *partial = dev_loss_buf;
    if (pix_size > 1) {
        char *scratch = nullptr;
        if (arena_get(sizeof(double) * (size_t)pix_size * (size_t)frame_size, &scratch, st)) { return 1; }
        partial = reinterpret_cast<double *>(scratch);
    }
    ScopedTimer tm(kTimeOther, static_cast<hipStream_t>(stream));
    if (ch_size <= 16) {
        hipLaunchKernelGGL(softmax_cross_entropy_few_kernel<16>, dim3((unsigned)blocks), dim3(kTailBlock), 0, st, dev_y_buf, dev_t_buf, dev_dy_buf,
                           partial, t_sum, pix_size, ch_size, frame_size, frame_stride, f_blocks);
    }
    else {
        hipLaunchKernelGGL(softmax_cross_entropy_kernel, dim3((unsigned)blocks), dim3(kTailBlock), 0, st, dev_y_buf, dev_t_buf, dev_dy_buf, partial,
                           t_sum, pix_size, ch_size, frame_size, frame_stride, f_blocks);
    }
    BBHIP_LAUNCH_CHECK();
    if (pix_size > 1) {
        hipLaunchKernelGGL(loss_pixel_sum_kernel, dim3((unsigned)f_blocks), dim3(kTailBlock), 0, st, partial, dev_loss_buf, pix_size, frame_size);
        BBHIP_LAUNCH_CHECK();
    }
    return 0;
}

int bbhip_fp32_ClassifierTail_ForwardBackward(float const *dev_x_buf, float *dev_y_buf, float *dev_dx_buf, int const *dev_input_index,
                                              float const *dev_t_buf, float *dev_dy_buf, double *dev_loss_buf, int *dev_accuracy_buf,
                                              int *dev_category_buf, float t_sum, int n, int input_node_size, int ch_size, int frame_size,
                                              int frame_stride, int binarize_input, int output_sum, void *stream)
{
    clear_hints();
    if (!(dev_x_buf && dev_dx_buf && dev_input_index && dev_t_buf && dev_loss_buf)) { return fail("%s: null buffer", __func__); }
    if (!(n > 0 && input_node_size > 0 && ch_size > 0 && frame_size > 0)) { return fail("%s: sizes must be positive", __func__); }
    if (frame_stride < frame_size) { return fail("%s: frame stride shorter than the frames", __func__); }
    if (ch_size > 16) { return fail("%s: at most 16 classes (ch_size=%d): call the four entries one by one", __func__, ch_size); }
    if ((long long)ch_size * n > 0x7fffffffLL) { return fail("%s: connection table too large", __func__); }
    // per-input sums, logits and gradients of 64 frames, then the table: within 64 KiB of LDS
    size_t const lds = ((size_t)input_node_size + 2 * 16) * 64 * sizeof(float) + (((size_t)ch_size * n + 3) & ~(size_t)3) * sizeof(int);
    if (lds > 64u * 1024u) {
        return fail("%s: input_node_size=%d nodes and ch_size*n=%d table entries need %zu bytes of LDS, 65536 are there (192 nodes with 2048 entries, "
                    "216 with 512): call the four entries one by one", __func__, input_node_size, ch_size * n, lds);
    }
    hipStream_t const st = static_cast<hipStream_t>(stream);
    ScopedTimer tm(kTimeOther, st);
    hipLaunchKernelGGL(classifier_tail_kernel<16>, dim3((unsigned)ceil_div(frame_stride, 64)), dim3(64 * kClassifierTailWaves), lds, st, dev_x_buf, dev_y_buf, dev_dx_buf,
                       dev_input_index, dev_t_buf, dev_dy_buf, dev_loss_buf, dev_accuracy_buf, dev_category_buf, t_sum,
                       output_sum ? 1.0f : 1.0f / (float)n, n, input_node_size, ch_size, frame_size, frame_stride, binarize_input);
    BBHIP_LAUNCH_CHECK();
    return 0;
}

int bbhip_fp32_MetricsCategoricalAccuracy(float const *dev_y_buf, float const *dev_t_buf, int *dev_accuracy_buf, int *dev_category_buf,
                                          int pix_size, int ch_size, int frame_size, int frame_stride, void *stream)
{
    clear_hints();                                 // a hint is for the next LUT forward call only
    if (!(dev_y_buf && dev_t_buf && dev_accuracy_buf && dev_category_buf)) { return fail("%s: null buffer", __func__); }
    if (!(pix_size > 0 && ch_size > 0 && frame_size > 0)) { return fail("%s: sizes must be positive", __func__); }
    if (frame_stride < frame_size) { return fail("%s: frame stride shorter than the frames", __func__); }
    if ((long long)pix_size * ch_size > 0x7fffffffLL) { return fail("%s: node count too large", __func__); }
    ScopedTimer tm(kTimeOther, static_cast<hipStream_t>(stream));
    hipLaunchKernelGGL(categorical_accuracy_kernel, dim3((unsigned)ceil_div(frame_size, kTailBlock)), dim3(kTailBlock), 0,
                       static_cast<hipStream_t>(stream), dev_y_buf, dev_t_buf, dev_accuracy_buf, dev_category_buf, pix_size, ch_size, frame_size,
                       frame_stride);
    BBHIP_LAUNCH_CHECK();
    return 0;
}

// ---- StochasticBatchNormalization ----
// 128-bit accesses need rows that start on 16 bytes: both bases aligned and both strides a multiple of four floats
static bool bn_rows_aligned(void const *p0, void const *p1, void const *p2, int stride0, int stride1)
{
    uintptr_t const bits = reinterpret_cast<uintptr_t>(p0) | reinterpret_cast<uintptr_t>(p1) | reinterpret_cast<uintptr_t>(p2);
    return (bits & 15u) == 0 && (stride0 & 3) == 0 && (stride1 & 3) == 0;
}

static int check_bn(void const *x, void const *out, int node_size, int frame_size, int x_stride, int out_stride, char const *name)
{
    if (!(x && out)) { return fail("%s: null buffer", name); }
    if (!(node_size > 0 && frame_size > 0)) { return fail("%s: sizes must be positive", name); }
    if (x_stride < frame_size || out_stride < frame_size) { return fail("%s: frame stride shorter than the frames", name); }
    return 0;
}

static int launch_bn_rows(BnArgs const &a, int node_size, bool backward, void *stream)
{
    bool const wide = bn_rows_aligned(a.x, backward ? a.dy : a.out, a.out, a.x_stride, a.out_stride);
    bool const held = a.frame_size <= kBnBlock * kBnHeld * (wide ? 4 : 1);
    dim3 const grid((unsigned)node_size), block(held ? kBnBlock : kBnLongBlock);
    hipStream_t const st = static_cast<hipStream_t>(stream);
    ScopedTimer tm(kTimeOther, st);
#define BBHIP_BN_ROWS(W, HELD)                                                                                  \
    do {                                                                                                        \
        if (backward) { hipLaunchKernelGGL((bn_backward_kernel<W, HELD>), grid, block, 0, st, a); }             \
        else          { hipLaunchKernelGGL((bn_forward_training_kernel<W, HELD>), grid, block, 0, st, a); }     \
    } while (0)
    if (wide) { if (held) { BBHIP_BN_ROWS(4, true); } else { BBHIP_BN_ROWS(4, false); } }
    else      { if (held) { BBHIP_BN_ROWS(1, true); } else { BBHIP_BN_ROWS(1, false); } }
#undef BBHIP_BN_ROWS
    BBHIP_LAUNCH_CHECK();
    return 0;
}

static int launch_bn_apply(BnArgs const &a, int node_size, bool from_running, void *stream, char const *name)
{
    bool const wide = bn_rows_aligned(a.x, a.out, a.out, a.x_stride, a.out_stride);
    int const f_blocks = ceil_div(a.frame_size, kBnBlock * (wide ? 4 : 1));
    long long const blocks = (long long)node_size * f_blocks;
    if (blocks > 0x7fffffffLL) { return fail("%s: grid too large", name); }
    dim3 const grid((unsigned)blocks), block(kBnBlock);
    hipStream_t const st = static_cast<hipStream_t>(stream);
    ScopedTimer tm(kTimeOther, st);
    if (wide) {
        if (from_running) { hipLaunchKernelGGL((bn_apply_kernel<4, true>), grid, block, 0, st, a, f_blocks); }
        else              { hipLaunchKernelGGL((bn_apply_kernel<4, false>), grid, block, 0, st, a, f_blocks); }
    }
    else {
        if (from_running) { hipLaunchKernelGGL((bn_apply_kernel<1, true>), grid, block, 0, st, a, f_blocks); }
        else              { hipLaunchKernelGGL((bn_apply_kernel<1, false>), grid, block, 0, st, a, f_blocks); }
    }
    BBHIP_LAUNCH_CHECK();
    return 0;
}

int bbhip_fp32_StochasticBatchNormalization_ForwardTraining(float const *dev_x_buf, float *dev_y_buf, float *dev_mean_buf, float *dev_rstd_buf,
                                                            float *dev_running_mean_buf, float *dev_running_var_buf, float gamma, float beta,
                                                            float momentum, int node_size, int frame_size, int frame_stride, void *stream)
{
    clear_hints();                                 // a hint is for the next LUT forward call only
    if (check_bn(dev_x_buf, dev_y_buf, node_size, frame_size, frame_stride, frame_stride, __func__)) { return 1; }
    BBHIP_REQUIRE(dev_mean_buf != nullptr && dev_rstd_buf != nullptr && dev_running_mean_buf != nullptr && dev_running_var_buf != nullptr);
    BnArgs a{};
    a.x = dev_x_buf; a.out = dev_y_buf; a.mean = dev_mean_buf; a.rstd = dev_rstd_buf;
    a.running_mean = dev_running_mean_buf; a.running_var = dev_running_var_buf;
    a.gamma = gamma; a.beta = beta; a.momentum = momentum;
    a.frame_size = frame_size; a.x_stride = frame_stride; a.out_stride = frame_stride;
    return launch_bn_rows(a, node_size, false, stream);
}

int bbhip_fp32_StochasticBatchNormalization_ReForward(float const *dev_x_buf, float *dev_y_buf, float const *dev_mean_buf,
                                                      float const *dev_rstd_buf, float gamma, float beta, int node_size, int frame_size,
                                                      int frame_stride, void *stream)
{
    clear_hints();                                 // a hint is for the next LUT forward call only
    if (check_bn(dev_x_buf, dev_y_buf, node_size, frame_size, frame_stride, frame_stride, __func__)) { return 1; }
    BBHIP_REQUIRE(dev_mean_buf != nullptr && dev_rstd_buf != nullptr);
    BnArgs a{};
    a.x = dev_x_buf; a.out = dev_y_buf; a.mean = const_cast<float *>(dev_mean_buf); a.rstd = const_cast<float *>(dev_rstd_buf);
    a.gamma = gamma; a.beta = beta;
    a.frame_size = frame_size; a.x_stride = frame_stride; a.out_stride = frame_stride;
    return launch_bn_apply(a, node_size, false, stream, __func__);
}

int bbhip_fp32_StochasticBatchNormalization_ForwardInference(float const *dev_x_buf, float *dev_y_buf, float const *dev_running_mean_buf,
                                                             float const *dev_running_var_buf, float gamma, float beta, int node_size,
                                                             int frame_size, int frame_stride, void *stream)
{
    clear_hints();                                 // a hint is for the next LUT forward call only
    if (check_bn(dev_x_buf, dev_y_buf, node_size, frame_size, frame_stride, frame_stride, __func__)) { return 1; }
    BBHIP_REQUIRE(dev_running_mean_buf != nullptr && dev_running_var_buf != nullptr);
    BnArgs a{};
    a.x = dev_x_buf; a.out = dev_y_buf;
    a.running_mean = const_cast<float *>(dev_running_mean_buf); a.running_var = const_cast<float *>(dev_running_var_buf);
    a.gamma = gamma; a.beta = beta;
    a.frame_size = frame_size; a.x_stride = frame_stride; a.out_stride = frame_stride;
    return launch_bn_apply(a, node_size, true, stream, __func__);
}

int bbhip_fp32_StochasticBatchNormalization_Backward(float const *dev_x_buf, float const *dev_dy_buf, float *dev_dx_buf,
                                                     float const *dev_mean_buf, float const *dev_rstd_buf, float gamma,
                                                     float reciprocal_frame_size, int node_size, int frame_size, int frame_stride,
                                                     int x_frame_stride, void *stream)
{
    clear_hints();                                 // a hint is for the next LUT forward call only
    if (check_bn(dev_x_buf, dev_dx_buf, node_size, frame_size, x_frame_stride, frame_stride, __func__)) { return 1; }
    BBHIP_REQUIRE(dev_dy_buf != nullptr && dev_mean_buf != nullptr && dev_rstd_buf != nullptr);
    BnArgs a{};
    a.x = dev_x_buf; a.dy = dev_dy_buf; a.out = dev_dx_buf;
    a.mean = const_cast<float *>(dev_mean_buf); a.rstd = const_cast<float *>(dev_rstd_buf);
    a.gamma = gamma; a.reciprocal_frame_size = reciprocal_frame_size;
    a.frame_size = frame_size; a.x_stride = x_frame_stride; a.out_stride = frame_stride;
    return launch_bn_rows(a, node_size, true, stream);
}

// ---- RealToBinary, BinaryToReal, Binarize, HardTanh ----
// `wide`: four frames per thread with 128-bit accesses; f_blocks = workgroups per row
static int modulation_grid(int rows, int frame_size, bool wide, TileDivisor &f_blocks, unsigned &blocks, char const *name)
{
    int const per_row = ceil_div(frame_size, kModBlock * (wide ? 4 : 1));
    long long const total = (long long)rows * per_row;
    if (total > 0x7fffffffLL) { return fail("%s: grid too large", name); }
    f_blocks = make_tile_divisor(per_row);
    blocks = (unsigned)total;
    return 0;
}

static int launch_row_map(int op, float const *x, float const *dy, float *out, float p0, float p1, float p2, int node_size, int frame_size,
                          int frame_stride, void *stream, char const *name)
{
    if (!(x && out && (dy || op != kMapHardTanhBackward))) { return fail("%s: null buffer", name); }
    if (!(node_size > 0 && frame_size > 0)) { return fail("%s: sizes must be positive", name); }
    if (frame_stride < frame_size) { return fail("%s: frame stride shorter than the frames", name); }
    RowMapArgs a{};
    a.x = x; a.dy = dy; a.out = out; a.frame_size = frame_size; a.x_stride = frame_stride; a.out_stride = frame_stride;
    a.p0 = p0; a.p1 = p1; a.p2 = p2;
    bool const wide = bn_rows_aligned(x, dy ? dy : x, out, frame_stride, frame_stride);
    unsigned blocks;
    if (modulation_grid(node_size, frame_size, wide, a.f_blocks, blocks, name)) { return 1; }
    hipStream_t const st = static_cast<hipStream_t>(stream);
    ScopedTimer tm(kTimeOther, st);
    dim3 const grid(blocks), block(kModBlock);
#define BBHIP_ROW_MAP(OP)                                                                               \
    do {                                                                                                \
        if (wide) { hipLaunchKernelGGL((row_map_kernel<OP, 4>), grid, block, 0, st, a); }               \
        else      { hipLaunchKernelGGL((row_map_kernel<OP, 1>), grid, block, 0, st, a); }               \
    } while (0)
    switch (op) {
    case kMapBinarize:  BBHIP_ROW_MAP(kMapBinarize); break;
    case kMapHardTanh:  BBHIP_ROW_MAP(kMapHardTanh); break;
    default:            BBHIP_ROW_MAP(kMapHardTanhBackward); break;
    }
#undef BBHIP_ROW_MAP
    BBHIP_LAUNCH_CHECK();
    return 0;
}

int bbhip_fp32_Binarize_Forward(float const *dev_x_buf, float *dev_y_buf, float binary_th, float binary_low, float binary_high,
                                int node_size, int frame_size, int frame_stride, void *stream)
{
    clear_hints();                                 // a hint is for the next LUT forward call only
    return launch_row_map(kMapBinarize, dev_x_buf, nullptr, dev_y_buf, binary_th, binary_low, binary_high, node_size, frame_size, frame_stride,
                          stream, __func__);
}

int bbhip_fp32_bit_Binarize_Forward(float const *dev_x_buf, int *dev_y_buf, float binary_th, int node_size, int frame_size,
                                    int x_frame_stride, int y_frame_stride, void *stream)
{
    clear_hints();                                 // a hint is for the next LUT forward call only
    if (!(dev_x_buf && dev_y_buf)) { return fail("%s: null buffer", __func__); }
    if (!(node_size > 0 && frame_size > 0)) { return fail("%s: sizes must be positive", __func__); }
    if (x_frame_stride < frame_size || y_frame_stride < (frame_size + 31) / 32) { return fail("%s: frame stride shorter than the frames", __func__); }
    bool const wide = bn_rows_aligned(dev_x_buf, dev_x_buf, dev_x_buf, x_frame_stride, x_frame_stride);
    TileDivisor f_blocks;
    unsigned blocks;
    if (modulation_grid(node_size, frame_size, wide, f_blocks, blocks, __func__)) { return 1; }
    hipStream_t const st = static_cast<hipStream_t>(stream);
    ScopedTimer tm(kTimeOther, st);
    uint32_t *const y = reinterpret_cast<uint32_t *>(dev_y_buf);
    if (wide) { hipLaunchKernelGGL((binarize_bits_kernel<4>), dim3(blocks), dim3(kModBlock), 0, st, dev_x_buf, y, binary_th, frame_size, x_frame_stride, y_frame_stride, f_blocks); }
    else      { hipLaunchKernelGGL((binarize_bits_kernel<1>), dim3(blocks), dim3(kModBlock), 0, st, dev_x_buf, y, binary_th, frame_size, x_frame_stride, y_frame_stride, f_blocks); }
    BBHIP_LAUNCH_CHECK();
    return 0;
}

int bbhip_fp32_HardTanh_Forward(float const *dev_x_buf, float *dev_y_buf, float limit_min, float limit_max, int node_size, int frame_size,
                                int frame_stride, void *stream)
{
    clear_hints();                                 // a hint is for the next LUT forward call only
    return launch_row_map(kMapHardTanh, dev_x_buf, nullptr, dev_y_buf, limit_min, limit_max, 0.0f, node_size, frame_size, frame_stride, stream, __func__);
}

int bbhip_fp32_HardTanh_Backward(float const *dev_x_buf, float const *dev_dy_buf, float *dev_dx_buf, float limit_min, float limit_max,
                                 int node_size, int frame_size, int frame_stride, void *stream)
{
    clear_hints();                                 // a hint is for the next LUT forward call only
    return launch_row_map(kMapHardTanhBackward, dev_x_buf, dev_dy_buf, dev_dx_buf, limit_min, limit_max, 0.0f, node_size, frame_size, frame_stride,
                          stream, __func__);
}

static int launch_real_to_binary(float const *x, void *y, bool bit, unsigned depth_modulation_size, unsigned frame_modulation_size,
                                 float input_range_lo, float input_range_hi, unsigned point_size, unsigned x_depth_size, unsigned x_frame_size,
                                 unsigned x_frame_stride, unsigned y_frame_stride, int binarize, void *stream, char const *name)
{
    if (!(x && y)) { return fail("%s: null buffer", name); }
    if (!(depth_modulation_size > 0 && frame_modulation_size > 0 && point_size > 0 && x_depth_size > 0 && x_frame_size > 0)) {
        return fail("%s: sizes must be positive", name);
    }
    long long const y_frames = (long long)x_frame_size * frame_modulation_size;
    long long const y_planes = (long long)x_depth_size * depth_modulation_size;
    long long const y_nodes = (y_planes <= 0x7fffffffLL) ? y_planes * point_size : -1;
    if (y_frames > 0x7fffffffLL || y_nodes < 0 || y_nodes > 0x7fffffffLL) { return fail("%s: output too large", name); }
    if (x_frame_stride < x_frame_size || (long long)y_frame_stride < (bit ? (y_frames + 31) / 32 : y_frames)) {
        return fail("%s: frame stride shorter than the frames", name);
    }
    RealToBinaryArgs a{};
    a.x = x; a.y = y;
    a.x_frame_size = (int)x_frame_size; a.y_frame_size = (int)y_frames; a.x_stride = (int)x_frame_stride; a.y_stride = (int)y_frame_stride;
    a.points = make_tile_divisor((int)point_size); a.depth_modulation = make_tile_divisor((int)depth_modulation_size);
    a.lo = input_range_lo; a.x_scale = 1.0f / (input_range_hi - input_range_lo);
    a.depth_step = 1.0f / (float)depth_modulation_size; a.depth_step_recip = (float)depth_modulation_size;
    a.frame_step = 1.0f / (float)frame_modulation_size; a.frame_step_recip = (float)frame_modulation_size;
    a.binarize = binarize; a.threshold = binarize ? 0.5f : 0.0f;
    a.frame_modulation = make_tile_divisor((int)frame_modulation_size);
    // packed rows are assembled from whole threads either way; fp32 rows need 16-byte rows for the wide stores
    bool const wide = bit || ((reinterpret_cast<uintptr_t>(y) & 15u) == 0 && (y_frame_stride & 3u) == 0);
    unsigned blocks;
    if (modulation_grid((int)y_nodes, (int)y_frames, wide, a.f_blocks, blocks, name)) { return 1; }
    hipStream_t const st = static_cast<hipStream_t>(stream);
    ScopedTimer tm(kTimeOther, st);
    dim3 const grid(blocks), block(kModBlock);
    if (bit)       { hipLaunchKernelGGL((real_to_binary_kernel<true, 4>), grid, block, 0, st, a); }
    else if (wide) { hipLaunchKernelGGL((real_to_binary_kernel<false, 4>), grid, block, 0, st, a); }
    else           { hipLaunchKernelGGL((real_to_binary_kernel<false, 1>), grid, block, 0, st, a); }
    BBHIP_LAUNCH_CHECK();
    return 0;
}

int bbhip_fp32_RealToBinary_Forward(float const *dev_x_buf, float *dev_y_buf, unsigned depth_modulation_size, unsigned frame_modulation_size,
                                    float input_range_lo, float input_range_hi, unsigned point_size, unsigned x_depth_size,
                                    unsigned x_frame_size, unsigned x_frame_stride, unsigned y_frame_stride, int binarize, void *stream)
{
    clear_hints();                                 // a hint is for the next LUT forward call only
    return launch_real_to_binary(dev_x_buf, dev_y_buf, false, depth_modulation_size, frame_modulation_size, input_range_lo, input_range_hi,
                                 point_size, x_depth_size, x_frame_size, x_frame_stride, y_frame_stride, binarize, stream, __func__);
}

int bbhip_fp32_bit_RealToBinary_Forward(float const *dev_x_buf, int *dev_y_buf, unsigned depth_modulation_size, unsigned frame_modulation_size,
                                        float input_range_lo, float input_range_hi, unsigned point_size, unsigned x_depth_size,
                                        unsigned x_frame_size, unsigned x_frame_stride, unsigned y_frame_stride, int binarize, void *stream)
{
    clear_hints();                                 // a hint is for the next LUT forward call only
    return launch_real_to_binary(dev_x_buf, dev_y_buf, true, depth_modulation_size, frame_modulation_size, input_range_lo, input_range_hi,
                                 point_size, x_depth_size, x_frame_size, x_frame_stride, y_frame_stride, binarize, stream, __func__);
}

static int check_binary_to_real(void const *a, void const *b, int node_mux_size, int frame_mux_size, int y_node_size, long long x_stride_frames,
                                int y_frame_size, int y_frame_stride, char const *name)
{
    if (!(a && b)) { return fail("%s: null buffer", name); }
    if (!(node_mux_size > 0 && frame_mux_size > 0 && y_node_size > 0 && y_frame_size > 0)) { return fail("%s: sizes must be positive", name); }
    if ((long long)y_frame_size * frame_mux_size > 0x7fffffffLL || (long long)node_mux_size * y_node_size > 0x7fffffffLL) {
        return fail("%s: input too large", name);
    }
    if ((long long)node_mux_size * frame_mux_size >= (1 << 24)) { return fail("%s: more than 2^24 inputs fold into an output", name); }
    if (y_frame_stride < y_frame_size || x_stride_frames < (long long)y_frame_size * frame_mux_size) {
        return fail("%s: frame stride shorter than the frames", name);
    }
    return 0;
}

static int launch_binary_to_real_forward(void const *x, bool bit, float *y, int node_mux_size, int frame_mux_size, int y_node_size,
                                         int x_frame_stride, int y_frame_size, int y_frame_stride, void *stream, char const *name)
{
    if (check_binary_to_real(x, y, node_mux_size, frame_mux_size, y_node_size, (long long)x_frame_stride * (bit ? 32 : 1), y_frame_size,
                             y_frame_stride, name)) { return 1; }
    BinaryToRealArgs a{};
    a.x = x; a.out = y; a.node_mux_size = node_mux_size; a.frame_mux_size = frame_mux_size; a.y_node_size = y_node_size;
    a.x_stride = x_frame_stride; a.y_frame_size = y_frame_size; a.y_stride = y_frame_stride;
    a.denominator = (float)(node_mux_size * frame_mux_size);
    unsigned blocks;
    if (modulation_grid(y_node_size, y_frame_size, false, a.f_blocks, blocks, name)) { return 1; }
    hipStream_t const st = static_cast<hipStream_t>(stream);
    ScopedTimer tm(kTimeOther, st);
    if (bit) { hipLaunchKernelGGL((binary_to_real_forward_kernel<true>), dim3(blocks), dim3(kModBlock), 0, st, a); }
    else     { hipLaunchKernelGGL((binary_to_real_forward_kernel<false>), dim3(blocks), dim3(kModBlock), 0, st, a); }
    BBHIP_LAUNCH_CHECK();
    return 0;
}

int bbhip_fp32_BinaryToReal_Forward(float const *dev_x_buf, float *dev_y_buf, int node_mux_size, int frame_mux_size, int y_node_size,
                                    int x_frame_stride, int y_frame_size, int y_frame_stride, void *stream)
{
    clear_hints();                                 // a hint is for the next LUT forward call only
    return launch_binary_to_real_forward(dev_x_buf, false, dev_y_buf, node_mux_size, frame_mux_size, y_node_size, x_frame_stride, y_frame_size,
                                         y_frame_stride, stream, __func__);
}

int bbhip_bit_fp32_BinaryToReal_Forward(int const *dev_x_buf, float *dev_y_buf, int node_mux_size, int frame_mux_size, int y_node_size,
                                        int x_frame_stride, int y_frame_size, int y_frame_stride, void *stream)
{
    clear_hints();                                 // a hint is for the next LUT forward call only
    return launch_binary_to_real_forward(dev_x_buf, true, dev_y_buf, node_mux_size, frame_mux_size, y_node_size, x_frame_stride, y_frame_size,
                                         y_frame_stride, stream, __func__);
}

int bbhip_fp32_BinaryToReal_Backward(float const *dev_dy_buf, float *dev_dx_buf, int node_mux_size, int frame_mux_size, int y_node_size,
                                     int x_frame_stride, int y_frame_size, int y_frame_stride, void *stream)
{
    clear_hints();                                 // a hint is for the next LUT forward call only
    if (check_binary_to_real(dev_dy_buf, dev_dx_buf, node_mux_size, frame_mux_size, y_node_size, x_frame_stride, y_frame_size, y_frame_stride,
                             __func__)) { return 1; }
    BinaryToRealArgs a{};
    a.dy = dev_dy_buf; a.out = dev_dx_buf; a.node_mux_size = node_mux_size; a.frame_mux_size = frame_mux_size; a.y_node_size = y_node_size;
    a.x_stride = x_frame_stride; a.y_frame_size = y_frame_size; a.y_stride = y_frame_stride;
    // the host loop's gain (include/bb/BinaryToReal.h:342): output nodes / (input nodes * frames folded), in fp32
    a.gain = (float)y_node_size / ((float)(node_mux_size * y_node_size) * (float)frame_mux_size);
    a.frame_mux = make_tile_divisor(frame_mux_size);
    int const x_frame_size = y_frame_size * frame_mux_size;
    bool const wide = (reinterpret_cast<uintptr_t>(dev_dx_buf) & 15u) == 0 && (x_frame_stride & 3) == 0;
    unsigned blocks;
    if (modulation_grid(node_mux_size * y_node_size, x_frame_size, wide, a.f_blocks, blocks, __func__)) { return 1; }
    hipStream_t const st = static_cast<hipStream_t>(stream);
    ScopedTimer tm(kTimeOther, st);
    if (wide) { hipLaunchKernelGGL((binary_to_real_backward_kernel<4>), dim3(blocks), dim3(kModBlock), 0, st, a, x_frame_size); }
    else      { hipLaunchKernelGGL((binary_to_real_backward_kernel<1>), dim3(blocks), dim3(kModBlock), 0, st, a, x_frame_size); }
    BBHIP_LAUNCH_CHECK();
    return 0;
}

// ---- MaxPooling, UpSampling ----
// rows = the rows of the launch's index space, an image of (row_h, row_w) pixels per channel; items = frames or words per row
static int window_grid(WindowArgs &a, int c, int row_h, int row_w, int items, int per_thread, unsigned &blocks, char const *name)
{
    long long const rows = (long long)c * row_h * row_w;
    int const per_row = ceil_div(items, kPoolBlock * per_thread);
    if (rows > 0x7fffffffLL || rows * per_row > 0x7fffffffLL) { return fail("%s: grid too large", name); }
    a.f_blocks = make_tile_divisor(per_row);
    a.row_w = make_tile_divisor(row_w);
    a.row_h = make_tile_divisor(row_h);
    blocks = (unsigned)(rows * per_row);
    return 0;
}

// packed rows: (row, word) pairs numbered through, f_blocks = words per row
static int window_grid_flat(WindowArgs &a, int c, int row_h, int row_w, int words, unsigned &blocks, long long &total, char const *name)
{
    long long const rows = (long long)c * row_h * row_w;
    total = rows * words;
    if (rows > 0x7fffffffLL || total > 0x7fffffffLL) { return fail("%s: grid too large", name); }
    a.f_blocks = make_tile_divisor(words);
    a.row_w = make_tile_divisor(row_w);
    a.row_h = make_tile_divisor(row_h);
    blocks = (unsigned)((total + kPoolBlock - 1) / kPoolBlock);
    return 0;
}

static int check_pooling(void const *p0, void const *p1, void const *p2, int fh, int fw, int w, int h, int ow, int oh, int c, int frame_size,
                         char const *name)
{
    if (!(p0 && p1 && p2)) { return fail("%s: null buffer", name); }
    if (!(fh > 0 && fw > 0 && w > 0 && h > 0 && c > 0 && frame_size > 0)) { return fail("%s: sizes must be positive", name); }
    if (ow != (w + fw - 1) / fw || oh != (h + fh - 1) / fh) { return fail("%s: output size must be ceil(input / filter)", name); }
    if ((long long)c * h * w > 0x7fffffffLL) { return fail("%s: image too large", name); }
    return 0;
}

int bbhip_fp32_MaxPooling_Forward(float const *dev_x_buf, float *dev_y_buf, int *dev_argmax_buf, int filter_h_size, int filter_w_size,
                                  int input_w_size, int input_h_size, int output_w_size, int output_h_size, int c_size, int frame_size,
                                  int frame_stride, void *stream)
{
    clear_hints();                                 // a hint is for the next LUT forward call only
    if (check_pooling(dev_x_buf, dev_y_buf, dev_argmax_buf, filter_h_size, filter_w_size, input_w_size, input_h_size, output_w_size, output_h_size,
                      c_size, frame_size, __func__)) { return 1; }
    if (frame_stride < frame_size) { return fail("%s: frame stride shorter than the frames", __func__); }
    WindowArgs a{};
    a.x = dev_x_buf; a.out = dev_y_buf; a.argmax_out = dev_argmax_buf;
    a.fh = filter_h_size; a.fw = filter_w_size; a.w = input_w_size; a.h = input_h_size; a.ow = output_w_size; a.oh = output_h_size;
    a.frame_size = frame_size; a.x_stride = frame_stride; a.out_stride = frame_stride;
    bool const wide = bn_rows_aligned(dev_x_buf, dev_y_buf, dev_argmax_buf, frame_stride, frame_stride);
    bool const two = filter_h_size == 2 && filter_w_size == 2;
    unsigned blocks;
    if (window_grid(a, c_size, output_h_size, output_w_size, frame_size, wide ? 4 : 1, blocks, __func__)) { return 1; }
    hipStream_t const st = static_cast<hipStream_t>(stream);
    ScopedTimer tm(kTimeOther, st);
    dim3 const grid(blocks), block(kPoolBlock);
    if (wide) { if (two) { hipLaunchKernelGGL((max_pooling_forward_kernel<4, true>), grid, block, 0, st, a); }
                else     { hipLaunchKernelGGL((max_pooling_forward_kernel<4, false>), grid, block, 0, st, a); } }
    else      { if (two) { hipLaunchKernelGGL((max_pooling_forward_kernel<1, true>), grid, block, 0, st, a); }
                else     { hipLaunchKernelGGL((max_pooling_forward_kernel<1, false>), grid, block, 0, st, a); } }
    BBHIP_LAUNCH_CHECK();
    return 0;
}

int bbhip_bit_MaxPooling_Forward(int const *dev_x_buf, int *dev_y_buf, int filter_h_size, int filter_w_size, int input_w_size,
                                 int input_h_size, int output_w_size, int output_h_size, int c_size, int frame_size, int frame_stride,
                                 void *stream)
{
    clear_hints();                                 // a hint is for the next LUT forward call only
    if (check_pooling(dev_x_buf, dev_y_buf, dev_y_buf, filter_h_size, filter_w_size, input_w_size, input_h_size, output_w_size, output_h_size,
                      c_size, frame_size, __func__)) { return 1; }
    int const words = (frame_size + 31) / 32;
    if (frame_stride < words) { return fail("%s: frame stride shorter than the frames", __func__); }
    WindowArgs a{};
    a.x = dev_x_buf; a.out = dev_y_buf;
    a.fh = filter_h_size; a.fw = filter_w_size; a.w = input_w_size; a.h = input_h_size; a.ow = output_w_size; a.oh = output_h_size;
    a.frame_size = frame_size; a.x_stride = frame_stride; a.out_stride = frame_stride;
    unsigned blocks;
    long long total;
    if (window_grid_flat(a, c_size, output_h_size, output_w_size, words, blocks, total, __func__)) { return 1; }
    hipStream_t const st = static_cast<hipStream_t>(stream);
    ScopedTimer tm(kTimeOther, st);
    hipLaunchKernelGGL(max_pooling_bit_forward_kernel, dim3(blocks), dim3(kPoolBlock), 0, st, a, words, total);
    BBHIP_LAUNCH_CHECK();
    return 0;
}

int bbhip_fp32_MaxPooling_Backward(int const *dev_argmax_buf, float const *dev_dy_buf, float *dev_dx_buf, int filter_h_size, int filter_w_size,
                                   int input_w_size, int input_h_size, int output_w_size, int output_h_size, int c_size, int frame_size,
                                   int frame_stride, void *stream)
{
    clear_hints();                                 // a hint is for the next LUT forward call only
    if (check_pooling(dev_argmax_buf, dev_dy_buf, dev_dx_buf, filter_h_size, filter_w_size, input_w_size, input_h_size, output_w_size,
                      output_h_size, c_size, frame_size, __func__)) { return 1; }
    if (frame_stride < frame_size) { return fail("%s: frame stride shorter than the frames", __func__); }
    WindowArgs a{};
    a.argmax_in = dev_argmax_buf; a.dy = dev_dy_buf; a.out = dev_dx_buf;
    a.fh = filter_h_size; a.fw = filter_w_size; a.w = input_w_size; a.h = input_h_size; a.ow = output_w_size; a.oh = output_h_size;
    a.frame_size = frame_size; a.x_stride = frame_stride; a.out_stride = frame_stride;
    bool const wide = bn_rows_aligned(dev_argmax_buf, dev_dy_buf, dev_dx_buf, frame_stride, frame_stride);
    unsigned blocks;
    if (window_grid(a, c_size, output_h_size, output_w_size, frame_size, wide ? 4 : 1, blocks, __func__)) { return 1; }
    hipStream_t const st = static_cast<hipStream_t>(stream);
    ScopedTimer tm(kTimeOther, st);
    if (wide) { hipLaunchKernelGGL((max_pooling_backward_kernel<4>), dim3(blocks), dim3(kPoolBlock), 0, st, a); }
    else      { hipLaunchKernelGGL((max_pooling_backward_kernel<1>), dim3(blocks), dim3(kPoolBlock), 0, st, a); }
    BBHIP_LAUNCH_CHECK();
    return 0;
}

int bbhip_bit_fp32_MaxPooling_Backward(int const *dev_x_buf, float const *dev_dy_buf, float *dev_dx_buf, int filter_h_size, int filter_w_size,
                                       int input_w_size, int input_h_size, int output_w_size, int output_h_size, int c_size, int frame_size,
                                       int forward_frame_stride, int backward_frame_stride, void *stream)
{
    clear_hints();                                 // a hint is for the next LUT forward call only
    if (check_pooling(dev_x_buf, dev_dy_buf, dev_dx_buf, filter_h_size, filter_w_size, input_w_size, input_h_size, output_w_size, output_h_size,
                      c_size, frame_size, __func__)) { return 1; }
    if (forward_frame_stride < (frame_size + 31) / 32 || backward_frame_stride < frame_size) { return fail("%s: frame stride shorter than the frames", __func__); }
    WindowArgs a{};
    a.x = dev_x_buf; a.dy = dev_dy_buf; a.out = dev_dx_buf;
    a.fh = filter_h_size; a.fw = filter_w_size; a.w = input_w_size; a.h = input_h_size; a.ow = output_w_size; a.oh = output_h_size;
    a.frame_size = frame_size; a.x_stride = forward_frame_stride; a.out_stride = backward_frame_stride;
    unsigned blocks;
    if (window_grid(a, c_size, output_h_size, output_w_size, frame_size, 1, blocks, __func__)) { return 1; }
    hipStream_t const st = static_cast<hipStream_t>(stream);
    ScopedTimer tm(kTimeOther, st);
    hipLaunchKernelGGL(max_pooling_bit_backward_kernel, dim3(blocks), dim3(kPoolBlock), 0, st, a);
    BBHIP_LAUNCH_CHECK();
    return 0;
}

static int launch_up_sampling(void const *x, float const *dy, void *out, bool bit, bool backward, int input_w_size, int input_h_size, int c_size,
                              int filter_w_size, int filter_h_size, int fill, int frame_size, int frame_stride, void *stream, char const *name)
{
    if (!((backward ? (void const *)dy : x) && out)) { return fail("%s: null buffer", name); }
    if (!(filter_h_size > 0 && filter_w_size > 0 && input_w_size > 0 && input_h_size > 0 && c_size > 0 && frame_size > 0)) {
        return fail("%s: sizes must be positive", name);
    }
    long long const out_pixels = (long long)c_size * input_h_size * filter_h_size * input_w_size * filter_w_size;
    if ((long long)input_h_size * filter_h_size > 0x7fffffffLL || (long long)input_w_size * filter_w_size > 0x7fffffffLL || out_pixels > 0x7fffffffLL) {
        return fail("%s: image too large", name);
    }
    int const items = bit ? (frame_size + 31) / 32 : frame_size;
    if (frame_stride < items) { return fail("%s: frame stride shorter than the frames", name); }
    WindowArgs a{};
    a.x = x; a.dy = dy; a.out = out;
    a.fh = filter_h_size; a.fw = filter_w_size; a.w = input_w_size; a.h = input_h_size; a.fill = fill;
    a.frame_size = frame_size; a.x_stride = frame_stride; a.out_stride = frame_stride;
    bool const wide = !bit && bn_rows_aligned(backward ? (void const *)dy : x, out, out, frame_stride, frame_stride);
    unsigned blocks;
    hipStream_t const st = static_cast<hipStream_t>(stream);
    if (backward) {
        if (window_grid(a, c_size, input_h_size, input_w_size, items, wide ? 4 : 1, blocks, name)) { return 1; }
        ScopedTimer tm(kTimeOther, st);
        if (wide) { hipLaunchKernelGGL((up_sampling_backward_kernel<4>), dim3(blocks), dim3(kPoolBlock), 0, st, a); }
        else      { hipLaunchKernelGGL((up_sampling_backward_kernel<1>), dim3(blocks), dim3(kPoolBlock), 0, st, a); }
    }
    else {
        long long total = 0;
        if (bit) { if (window_grid_flat(a, c_size, input_h_size * filter_h_size, input_w_size * filter_w_size, items, blocks, total, name)) { return 1; } }
        else if (window_grid(a, c_size, input_h_size * filter_h_size, input_w_size * filter_w_size, items, wide ? 4 : 1, blocks, name)) { return 1; }
        ScopedTimer tm(kTimeOther, st);
        if (bit)       { hipLaunchKernelGGL((up_sampling_forward_kernel<true, 1>), dim3(blocks), dim3(kPoolBlock), 0, st, a, items, total); }
        else if (wide) { hipLaunchKernelGGL((up_sampling_forward_kernel<false, 4>), dim3(blocks), dim3(kPoolBlock), 0, st, a, items, total); }
        else           { hipLaunchKernelGGL((up_sampling_forward_kernel<false, 1>), dim3(blocks), dim3(kPoolBlock), 0, st, a, items, total); }
    }
    BBHIP_LAUNCH_CHECK();
    return 0;
}

int bbhip_fp32_UpSampling_Forward(float const *dev_x_buf, float *dev_y_buf, int input_w_size, int input_h_size, int c_size, int filter_w_size,
                                  int filter_h_size, int fill, int frame_size, int frame_stride, void *stream)
{
    clear_hints();                                 // a hint is for the next LUT forward call only
    return launch_up_sampling(dev_x_buf, nullptr, dev_y_buf, false, false, input_w_size, input_h_size, c_size, filter_w_size, filter_h_size, fill,
                              frame_size, frame_stride, stream, __func__);
}

int bbhip_bit_UpSampling_Forward(int const *dev_x_buf, int *dev_y_buf, int input_w_size, int input_h_size, int c_size, int filter_w_size,
                                 int filter_h_size, int fill, int frame_size, int frame_stride, void *stream)
{
    clear_hints();                                 // a hint is for the next LUT forward call only
    return launch_up_sampling(dev_x_buf, nullptr, dev_y_buf, true, false, input_w_size, input_h_size, c_size, filter_w_size, filter_h_size, fill,
                              frame_size, frame_stride, stream, __func__);
}

int bbhip_fp32_UpSampling_Backward(float const *dev_dy_buf, float *dev_dx_buf, int input_w_size, int input_h_size, int c_size, int filter_w_size,
                                   int filter_h_size, int fill, int frame_size, int frame_stride, void *stream)
{
    clear_hints();                                 // a hint is for the next LUT forward call only
    return launch_up_sampling(nullptr, dev_dy_buf, dev_dx_buf, false, true, input_w_size, input_h_size, c_size, filter_w_size, filter_h_size, fill,
                              frame_size, frame_stride, stream, __func__);
}

// ---- Shuffle ----
static int launch_shuffle(int const *src, int *dst, unsigned unit_size, unsigned group_size, unsigned node_size, unsigned frame_size,
                          unsigned frame_stride, void *stream, char const *name)
{
    if (!(src && dst)) { return fail("%s: null buffer", name); }
    if (unit_size == 0 || node_size == 0 || frame_size == 0 || frame_stride == 0) { return fail("%s: sizes must be positive", name); }
    if ((unsigned long long)unit_size * group_size != node_size) { return fail("%s: node_size must be a multiple of the unit size", name); }
    if (node_size > 0x7fffffffu || frame_stride > 0x7fffffffu) { return fail("%s: buffer too large", name); }
    bool const wide = (frame_stride & 3u) == 0 && (((uintptr_t)src | (uintptr_t)dst) & 15u) == 0;
    unsigned const pieces = wide ? frame_stride / 4 : frame_stride;
    long long const total = (long long)node_size * pieces;
    if (total > 0x7fffffffLL) { return fail("%s: grid too large", name); }
    ShuffleArgs a{};
    a.src = reinterpret_cast<uint32_t const *>(src); a.dst = reinterpret_cast<uint32_t *>(dst);
    a.pieces = make_tile_divisor((int)pieces); a.unit = make_tile_divisor((int)unit_size);
    a.group_size = (int)group_size; a.stride = (int)frame_stride;
    hipStream_t const st = static_cast<hipStream_t>(stream);
    ScopedTimer tm(kTimeOther, st);
    dim3 const grid((unsigned)((total + kPoolBlock - 1) / kPoolBlock)), block(kPoolBlock);
    if (wide) { hipLaunchKernelGGL(row_shuffle_kernel<4>, grid, block, 0, st, a, total); }
    else      { hipLaunchKernelGGL(row_shuffle_kernel<1>, grid, block, 0, st, a, total); }
    BBHIP_LAUNCH_CHECK();
    return 0;
}

int bbhip_Shuffle_Forward(int const *dev_x_buf, int *dev_y_buf, unsigned int y_unit_size, unsigned int node_size, unsigned int frame_size,
                          unsigned int frame_stride, void *stream)
{
    clear_hints();                                 // a hint is for the next LUT forward call only
    if (y_unit_size == 0) { return fail("%s: sizes must be positive", __func__); }
    return launch_shuffle(dev_x_buf, dev_y_buf, y_unit_size, node_size / y_unit_size, node_size, frame_size, frame_stride, stream, __func__);
}

int bbhip_Shuffle_Backward(int const *dev_dy_buf, int *dev_dx_buf, unsigned int y_unit_size, unsigned int node_size, unsigned int frame_size,
                           unsigned int frame_stride, void *stream)
{
    clear_hints();                                 // a hint is for the next LUT forward call only
    if (y_unit_size == 0 || node_size % y_unit_size != 0) { return fail("%s: node_size must be a multiple of the unit size", __func__); }
    return launch_shuffle(dev_dy_buf, dev_dx_buf, node_size / y_unit_size, y_unit_size, node_size, frame_size, frame_stride, stream, __func__);
}

int bbhip_fp32_ConvBitToReal(int const *dev_x_buf, float *dev_y_buf, float value0, float value1,
                             int node_size, int frame_size, int x_frame_stride, int y_frame_stride, void *stream)
{
    clear_hints();                                 // a hint is for the next LUT forward call only
    BBHIP_REQUIRE(dev_x_buf != nullptr && dev_y_buf != nullptr);
    BBHIP_REQUIRE(node_size > 0 && node_size <= 65535 * 1024 && frame_size > 0);
    BBHIP_REQUIRE(x_frame_stride >= (frame_size + 31) / 32 && y_frame_stride >= frame_size);
    // grid.y is limited to 65535 rows per launch
    for (int n0 = 0; n0 < node_size; n0 += 65535) {
        int const rows = (node_size - n0 < 65535) ? node_size - n0 : 65535;
        hipLaunchKernelGGL(conv_bit_to_real_kernel, dim3(ceil_div(frame_size, kBlock), rows), dim3(kBlock), 0, static_cast<hipStream_t>(stream),
                           reinterpret_cast<uint32_t const *>(dev_x_buf) + (size_t)n0 * x_frame_stride,
                           dev_y_buf + (size_t)n0 * y_frame_stride, value0, value1, frame_size, x_frame_stride, y_frame_stride);
        BBHIP_LAUNCH_CHECK();
    }
    return 0;
}

// ---- StochasticLut ---------------------------------------------------------------------------------

int bbhip_fp32_StochasticLut_Forward(int n, float const *dev_x_buf, float *dev_y_buf, int const *dev_input_index,
                                     float const *dev_W, int node_size, int frame_size, int frame_stride,
                                     int input_binary, int lut_binarize, float unbinarize_bias, void *stream)
{
    ForwardCall c{};
    c.n = n; c.x = dev_x_buf; c.y = dev_y_buf; c.idx = dev_input_index; c.W = dev_W;
    c.node_size = node_size; c.frame_size = frame_size; c.x_stride = frame_stride; c.y_stride = frame_stride;
    c.xmode = input_binary ? kXBinary : kXClamp; c.ymode = kYClamp;
    c.lut_binarize = lut_binarize; c.bias = unbinarize_bias;
    return forward_entry(c, stream);
}

int bbhip_fp32_StochasticLut_ForwardClampW(int n, float const *dev_x_buf, float *dev_y_buf, int const *dev_input_index,
                                           float *dev_W, int node_size, int frame_size, int frame_stride,
                                           int input_binary, int lut_binarize, float unbinarize_bias,
                                           float w_lo, float w_hi, void *stream)
{
    BBHIP_REQUIRE(w_lo <= w_hi);
    ForwardCall c{};
    c.n = n; c.x = dev_x_buf; c.y = dev_y_buf; c.idx = dev_input_index; c.W = dev_W;
    c.node_size = node_size; c.frame_size = frame_size; c.x_stride = frame_stride; c.y_stride = frame_stride;
    c.xmode = input_binary ? kXBinary : kXClamp; c.ymode = kYClamp;
    c.lut_binarize = lut_binarize; c.bias = unbinarize_bias;
    c.clamp_W = dev_W; c.clamp_lo = w_lo; c.clamp_hi = w_hi;
    return forward_entry(c, stream);
}

int bbhip_fp32_StochasticLut_Forward_NoAlloc(int n, float const *dev_x_buf, float *dev_y_buf, int const *dev_input_index,
                                             float const *dev_W, int node_size, int frame_size, int frame_stride,
                                             int input_binary, int lut_binarize, float unbinarize_bias, void *stream)
{
    // device address of the file-scope scratch array, looked up once per device with that device current (the array's
    // name is only a host-side handle; each GPU holds its own copy at its own address)
    static void      *scratch_ptr[kMaxDevices] = {};
    static std::mutex scratch_mtx;
    int dev = 0;
    BBHIP_TRY(hipGetDevice(&dev));
    if (dev < 0 || dev >= kMaxDevices) { return fail("device index %d out of range", dev); }
    void *base = nullptr;
    {
        std::lock_guard<std::mutex> lk(scratch_mtx);
        if (!scratch_ptr[dev]) {
            void *p = nullptr;
            BBHIP_TRY(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
            scratch_ptr[dev] = p;
        }
        base = scratch_ptr[dev];
    }
    if (n < 2 || n > 6) { return fail("LUT width n=%d not in 2..6", n); }
    // both tables of a call must fit: [node_size][2^n] floats each, rounded to 256 bytes
    size_t const table = align256((size_t)(node_size > 0 ? node_size : 0) * ((size_t)1 << n) * sizeof(float));
    size_t const need  = table * (input_binary ? 2 : 1);
    if (need > kNoAllocScratchBytes) {
        return fail("bbhip_fp32_StochasticLut_Forward_NoAlloc: node_size=%d at n=%d needs %zu bytes of scratch, the fixed block holds %zu "
                    "(use bbhip_fp32_StochasticLut_Forward)", node_size, n, need, (size_t)kNoAllocScratchBytes);
    }
    Scratch fixed;
    fixed.fixed = static_cast<char *>(base);
    fixed.fixed_cap = kNoAllocScratchBytes;
    ForwardCall c{};
    c.n = n; c.x = dev_x_buf; c.y = dev_y_buf; c.idx = dev_input_index; c.W = dev_W;
    c.node_size = node_size; c.frame_size = frame_size; c.x_stride = frame_stride; c.y_stride = frame_stride;
    c.xmode = input_binary ? kXBinary : kXClamp; c.ymode = kYClamp;
    c.lut_binarize = lut_binarize; c.bias = unbinarize_bias;
    return forward_entry(c, stream, &fixed);
}

int bbhip_bit_fp32_StochasticLut_Forward(int n, int const *dev_x_buf, float *dev_y_buf, int const *dev_input_index,
                                         float const *dev_W, int node_size, int frame_size, int frame_stride,
                                         int bin_frame_stride, int lut_binarize, float unbinarize_bias, void *stream)
{
    ForwardCall c{};
    c.n = n; c.x = dev_x_buf; c.y = dev_y_buf; c.idx = dev_input_index; c.W = dev_W;
    c.node_size = node_size; c.frame_size = frame_size; c.x_stride = bin_frame_stride; c.y_stride = frame_stride;
    c.xmode = kXBit; c.ymode = kYClamp;
    c.lut_binarize = lut_binarize; c.bias = unbinarize_bias;
    return forward_entry(c, stream);
}

int bbhip_bit_bit_fp32_StochasticLut_Forward(int n, int const *dev_x_buf, int *dev_y_buf, int const *dev_input_index,
                                             float const *dev_W, int node_size, int frame_size, int frame_stride,
                                             int lut_binarize, float unbinarize_bias, void *stream)
{
    ForwardCall c{};
    c.n = n; c.x = dev_x_buf; c.y = dev_y_buf; c.idx = dev_input_index; c.W = dev_W;
    c.node_size = node_size; c.frame_size = frame_size; c.x_stride = frame_stride; c.y_stride = frame_stride;
    c.xmode = kXBit; c.ymode = kYBit;
    c.lut_binarize = lut_binarize; c.bias = unbinarize_bias;
    return forward_entry(c, stream);
}

int bbhip_fp32_DifferentiableLutN_ForwardNoBn(int n, float const *dev_x_buf, float *dev_y_buf,
        int const *dev_input_index, float const *dev_W, float unbinarize_bias,
        int node_size, int frame_size, int frame_stride, int lut_binarize, int binary_mode, void *stream)
{
    ForwardCall c{};
    c.n = n; c.x = dev_x_buf; c.y = dev_y_buf; c.idx = dev_input_index; c.W = dev_W;
    c.node_size = node_size; c.frame_size = frame_size; c.x_stride = frame_stride; c.y_stride = frame_stride;
    c.xmode = binary_mode ? kXBinary : kXClamp; c.ymode = binary_mode ? kYBinarize : kYClamp;
    c.lut_binarize = lut_binarize; c.bias = unbinarize_bias;
    return forward_entry(c, stream);
}

int bbhip_fp32_StochasticLut_Backward(int n, float const *dev_x_buf, float const *dev_dy_buf, float *dev_dx_buf,
                                      float *dev_dx_tmp, int const *dev_input_index, int const *dev_reverse_index,
                                      float const *dev_W, float *dev_dW, int reverse_index_stride,
                                      int input_node_size, int output_node_size, int frame_size, int frame_stride,
                                      int tmp_frame_size, int tmp_frame_stride, int input_binary, int lut_binarize,
                                      float unbinarize_bias, void *stream)
{
    BackwardCall c{};
    c.n = n; c.x = dev_x_buf; c.dy = dev_dy_buf; c.dx = dev_dx_buf; c.dx_tmp = dev_dx_tmp;
    c.idx = dev_input_index; c.rev = dev_reverse_index; c.W = dev_W; c.dW = dev_dW;
    c.rev_stride = reverse_index_stride; c.input_node_size = input_node_size; c.output_node_size = output_node_size;
    c.frame_size = frame_size; c.x_stride = frame_stride; c.frame_stride = frame_stride;
    c.tmp_frame_size = tmp_frame_size; c.tmp_frame_stride = tmp_frame_stride;
    c.xmode = input_binary ? kXBinary : kXClamp; c.lut_binarize = lut_binarize; c.bias = unbinarize_bias;
    return backward_entry(c, stream);
}

int bbhip_bit_fp32_StochasticLut_Backward(int n, int const *dev_x_buf, float const *dev_dy_buf, float *dev_dx_buf,
                                          float *dev_dx_tmp, int const *dev_input_index, int const *dev_reverse_index,
                                          float const *dev_W, float *dev_dW, int reverse_index_stride,
                                          int input_node_size, int output_node_size, int frame_size, int frame_stride,
                                          int bin_frame_stride, int tmp_frame_size, int tmp_frame_stride,
                                          int lut_binarize, float unbinarize_bias, void *stream)
{
    BackwardCall c{};
    c.n = n; c.x = dev_x_buf; c.dy = dev_dy_buf; c.dx = dev_dx_buf; c.dx_tmp = dev_dx_tmp;
    c.idx = dev_input_index; c.rev = dev_reverse_index; c.W = dev_W; c.dW = dev_dW;
    c.rev_stride = reverse_index_stride; c.input_node_size = input_node_size; c.output_node_size = output_node_size;
    c.frame_size = frame_size; c.x_stride = bin_frame_stride; c.frame_stride = frame_stride;
    c.tmp_frame_size = tmp_frame_size; c.tmp_frame_stride = tmp_frame_stride;
    c.xmode = kXBit; c.lut_binarize = lut_binarize; c.bias = unbinarize_bias;
    return backward_entry(c, stream);
}

// ---- DifferentiableLut -----------------------------------------------------------------------------

int bbhip_fp32_DifferentiableLutN_ForwardTraining(int n, float const *dev_x_buf, float *dev_y_buf,
        int const *dev_input_index, float const *dev_W, float *dev_mean_buf, float *dev_rstd_buf,
        float *dev_running_mean_buf, float *dev_running_var_buf, float gamma, float beta, float momentum,
        float unbinarize_bias, int node_size, int frame_size, int frame_stride, int lut_binarize, int binary_mode,
        void *stream)
{
    ForwardCall c{};
    c.n = n; c.x = dev_x_buf; c.y = dev_y_buf; c.idx = dev_input_index; c.W = dev_W;
    c.node_size = node_size; c.frame_size = frame_size; c.x_stride = frame_stride; c.y_stride = frame_stride;
    c.xmode = binary_mode ? kXBinary : kXClamp; c.ymode = binary_mode ? kYBinarize : kYClamp;
    c.lut_binarize = lut_binarize; c.bias = unbinarize_bias;
    c.bn = 1; c.mean = dev_mean_buf; c.rstd = dev_rstd_buf; c.running_mean = dev_running_mean_buf; c.running_var = dev_running_var_buf;
    c.gamma = gamma; c.beta = beta; c.momentum = momentum;
    return forward_entry(c, stream);
}

int bbhip_bit_fp32_DifferentiableLutN_ForwardTraining(int n, int const *dev_x_buf, int *dev_y_buf,
        int const *dev_input_index, float const *dev_W, float *dev_mean_buf, float *dev_rstd_buf,
        float *dev_running_mean_buf, float *dev_running_var_buf, float gamma, float beta, float momentum,
        float unbinarize_bias, int node_size, int frame_size, int frame_stride, int lut_binarize, void *stream)
{
    ForwardCall c{};
    c.n = n; c.x = dev_x_buf; c.y = dev_y_buf; c.idx = dev_input_index; c.W = dev_W;
    c.node_size = node_size; c.frame_size = frame_size; c.x_stride = frame_stride; c.y_stride = frame_stride;
    c.xmode = kXBit; c.ymode = kYBit;
    c.lut_binarize = lut_binarize; c.bias = unbinarize_bias;
    c.bn = 1; c.mean = dev_mean_buf; c.rstd = dev_rstd_buf; c.running_mean = dev_running_mean_buf; c.running_var = dev_running_var_buf;
    c.gamma = gamma; c.beta = beta; c.momentum = momentum;
    return forward_entry(c, stream);
}

int bbhip_fp32_DifferentiableLutN_ForwardTrainingClampW(int n, float const *dev_x_buf, float *dev_y_buf,
        int const *dev_input_index, float *dev_W, float *dev_mean_buf, float *dev_rstd_buf,
        float *dev_running_mean_buf, float *dev_running_var_buf, float gamma, float beta, float momentum,
        float unbinarize_bias, int node_size, int frame_size, int frame_stride, int lut_binarize, int binary_mode,
        float w_lo, float w_hi, void *stream)
{
    BBHIP_REQUIRE(w_lo <= w_hi);
    ForwardCall c{};
    c.n = n; c.x = dev_x_buf; c.y = dev_y_buf; c.idx = dev_input_index; c.W = dev_W;
    c.node_size = node_size; c.frame_size = frame_size; c.x_stride = frame_stride; c.y_stride = frame_stride;
    c.xmode = binary_mode ? kXBinary : kXClamp; c.ymode = binary_mode ? kYBinarize : kYClamp;
    c.lut_binarize = lut_binarize; c.bias = unbinarize_bias;
    c.bn = 1; c.mean = dev_mean_buf; c.rstd = dev_rstd_buf; c.running_mean = dev_running_mean_buf; c.running_var = dev_running_var_buf;
    c.gamma = gamma; c.beta = beta; c.momentum = momentum;
    c.clamp_W = dev_W; c.clamp_lo = w_lo; c.clamp_hi = w_hi;
    return forward_entry(c, stream);
}

int bbhip_bit_fp32_DifferentiableLutN_ForwardTrainingClampW(int n, int const *dev_x_buf, int *dev_y_buf,
        int const *dev_input_index, float *dev_W, float *dev_mean_buf, float *dev_rstd_buf,
        float *dev_running_mean_buf, float *dev_running_var_buf, float gamma, float beta, float momentum,
        float unbinarize_bias, int node_size, int frame_size, int frame_stride, int lut_binarize,
        float w_lo, float w_hi, void *stream)
{
    BBHIP_REQUIRE(w_lo <= w_hi);
    ForwardCall c{};
    c.n = n; c.x = dev_x_buf; c.y = dev_y_buf; c.idx = dev_input_index; c.W = dev_W;
    c.node_size = node_size; c.frame_size = frame_size; c.x_stride = frame_stride; c.y_stride = frame_stride;
    c.xmode = kXBit; c.ymode = kYBit;
    c.lut_binarize = lut_binarize; c.bias = unbinarize_bias;
    c.bn = 1; c.mean = dev_mean_buf; c.rstd = dev_rstd_buf; c.running_mean = dev_running_mean_buf; c.running_var = dev_running_var_buf;
    c.gamma = gamma; c.beta = beta; c.momentum = momentum;
    c.clamp_W = dev_W; c.clamp_lo = w_lo; c.clamp_hi = w_hi;
    return forward_entry(c, stream);
}

int bbhip_fp32_DifferentiableLutN_ForwardInference(int n, float const *dev_x_buf, float *dev_y_buf,
        int const *dev_input_index, float const *dev_W, float const *dev_running_mean_buf,
        float const *dev_running_var_buf, float gamma, float beta, float unbinarize_bias,
        int node_size, int frame_size, int frame_stride, int lut_binarize, int binary_mode, void *stream)
{
    ForwardCall c{};
    c.n = n; c.x = dev_x_buf; c.y = dev_y_buf; c.idx = dev_input_index; c.W = dev_W;
    c.node_size = node_size; c.frame_size = frame_size; c.x_stride = frame_stride; c.y_stride = frame_stride;
    c.xmode = binary_mode ? kXBinary : kXClamp; c.ymode = binary_mode ? kYBinarize : kYClamp;
    c.lut_binarize = lut_binarize; c.bias = unbinarize_bias;
    c.bn = 2; c.running_mean = const_cast<float *>(dev_running_mean_buf); c.running_var = const_cast<float *>(dev_running_var_buf);
    c.gamma = gamma; c.beta = beta;
    return forward_entry(c, stream);
}

int bbhip_bit_fp32_DifferentiableLutN_ForwardInference(int n, int const *dev_x_buf, int *dev_y_buf,
        int const *dev_input_index, float const *dev_W, float const *dev_running_mean_buf,
        float const *dev_running_var_buf, float gamma, float beta, float unbinarize_bias,
        int node_size, int frame_size, int frame_stride, int lut_binarize, void *stream)
{
    ForwardCall c{};
    c.n = n; c.x = dev_x_buf; c.y = dev_y_buf; c.idx = dev_input_index; c.W = dev_W;
    c.node_size = node_size; c.frame_size = frame_size; c.x_stride = frame_stride; c.y_stride = frame_stride;
    c.xmode = kXBit; c.ymode = kYBit;
    c.lut_binarize = lut_binarize; c.bias = unbinarize_bias;
    c.bn = 2; c.running_mean = const_cast<float *>(dev_running_mean_buf); c.running_var = const_cast<float *>(dev_running_var_buf);
    c.gamma = gamma; c.beta = beta;
    return forward_entry(c, stream);
}

int bbhip_fp32_DifferentiableLutN_Backward(int n, float const *dev_x_buf, float const *dev_dy_buf, float *dev_dx_buf,
        float *dev_dx_tmp, int const *dev_input_index, int const *dev_reverse_index, float const *dev_W,
        float *dev_dW, float const *dev_mean_buf, float const *dev_rstd_buf, float *dev_dmean_tmp,
        float *dev_dvar_tmp, float gamma, float beta, float unbinarize_bias, int reverse_index_stride,
        int input_node_size, int output_node_size, int frame_size, int frame_stride, int tmp_frame_size,
        int tmp_frame_stride, int lut_binarize, int binary_mode, void *stream)
{
    BackwardCall c{};
    c.n = n; c.x = dev_x_buf; c.dy = dev_dy_buf; c.dx = dev_dx_buf; c.dx_tmp = dev_dx_tmp;
    c.idx = dev_input_index; c.rev = dev_reverse_index; c.W = dev_W; c.dW = dev_dW;
    c.rev_stride = reverse_index_stride; c.input_node_size = input_node_size; c.output_node_size = output_node_size;
    c.frame_size = frame_size; c.x_stride = frame_stride; c.frame_stride = frame_stride;
    c.tmp_frame_size = tmp_frame_size; c.tmp_frame_stride = tmp_frame_stride;
    c.xmode = binary_mode ? kXBinary : kXClamp; c.lut_binarize = lut_binarize; c.bias = unbinarize_bias;
    c.bn = 1; c.mean = dev_mean_buf; c.rstd = dev_rstd_buf; c.dmean_tmp = dev_dmean_tmp; c.dvar_tmp = dev_dvar_tmp;
    c.gamma = gamma; c.beta = beta;
    return backward_entry(c, stream);
}

int bbhip_bit_fp32_DifferentiableLutN_Backward(int n, int const *dev_x_buf, float const *dev_dy_buf, float *dev_dx_buf,
        float *dev_dx_tmp, int const *dev_input_index, int const *dev_reverse_index, float const *dev_W,
        float *dev_dW, float const *dev_mean_buf, float const *dev_rstd_buf, float *dev_dmean_tmp,
        float *dev_dvar_tmp, float gamma, float beta, float unbinarize_bias, int reverse_index_stride,
        int input_node_size, int output_node_size, int frame_size, int frame_stride, int x_frame_stride,
        int tmp_frame_size, int tmp_frame_stride, int lut_binarize, void *stream)
{
    BackwardCall c{};
    c.n = n; c.x = dev_x_buf; c.dy = dev_dy_buf; c.dx = dev_dx_buf; c.dx_tmp = dev_dx_tmp;
    c.idx = dev_input_index; c.rev = dev_reverse_index; c.W = dev_W; c.dW = dev_dW;
    c.rev_stride = reverse_index_stride; c.input_node_size = input_node_size; c.output_node_size = output_node_size;
    c.frame_size = frame_size; c.x_stride = x_frame_stride; c.frame_stride = frame_stride;
    c.tmp_frame_size = tmp_frame_size; c.tmp_frame_stride = tmp_frame_stride;
    c.xmode = kXBit; c.lut_binarize = lut_binarize; c.bias = unbinarize_bias;
    c.bn = 1; c.mean = dev_mean_buf; c.rstd = dev_rstd_buf; c.dmean_tmp = dev_dmean_tmp; c.dvar_tmp = dev_dvar_tmp;
    c.gamma = gamma; c.beta = beta;
    return backward_entry(c, stream);
}

// ---- BinaryLut6 ------------------------------------------------------------------------------------

int bbhip_bit_BinaryLut6_Forward(int const *dev_x_buf, int *dev_y_buf, int const *dev_input_index, int const *dev_table,
                                 int node_size, int frame_size, int frame_stride, void *stream)
{
    clear_hints();                                 // a hint is for the next LUT forward call only
    BBHIP_REQUIRE(dev_x_buf != nullptr && dev_y_buf != nullptr && dev_input_index != nullptr && dev_table != nullptr);
    BBHIP_REQUIRE(node_size > 0 && node_size <= (0x7fffffff >> 6) && frame_size > 0);
    BBHIP_REQUIRE(frame_stride >= (frame_size + 31) / 32);
    BBHIP_REQUIRE(frame_stride <= 0x07ffffff);          // row pitch in bytes, times the four nodes of a wavefront, stays a 32-bit extent
    hipStream_t st = static_cast<hipStream_t>(stream);
    BinArgs a{};
    a.x = reinterpret_cast<uint32_t const *>(dev_x_buf);
    a.y = reinterpret_cast<uint32_t *>(dev_y_buf);
    a.idx = dev_input_index; a.table = dev_table;
    a.node_size = node_size; a.frame_size = frame_size; a.stride = frame_stride;
    a.word_count = (frame_size + 31) / 32;
    a.chunk = bin_chunk_words();
    a.chunk_count = ceil_div(a.word_count, a.chunk);
    // nodes per wavefront: four share a unit's set-up where that still leaves the launch 2048 workgroups
    int npw = bin_nodes_per_wave();
    if (npw == 0) {
        npw = 4;
        while (npw > 1 && (long long)a.chunk_count * ceil_div(node_size, kWavesPerBlk * npw) < 2048) { npw /= 2; }
    }
    a.tiles = make_tile_divisor(ceil_div(node_size, kWavesPerBlk * npw));
    BBHIP_REQUIRE((long long)a.chunk_count * a.tiles.count <= 0x7fffffffLL);
    {
        ScopedTimer tm(kTimeBinary, st);
        dim3 const grid(a.chunk_count * a.tiles.count), block(kBlock);
        bool const exact = (node_size % npw) == 0;
        switch (npw) {
        case 1: hipLaunchKernelGGL((binary_lut6_kernel<1, true>), grid, block, 0, st, a); break;
        case 2: if (exact) { hipLaunchKernelGGL((binary_lut6_kernel<2, true>), grid, block, 0, st, a); }
                else       { hipLaunchKernelGGL((binary_lut6_kernel<2, false>), grid, block, 0, st, a); }
                break;
        default: if (exact) { hipLaunchKernelGGL((binary_lut6_kernel<4, true>), grid, block, 0, st, a); }
                 else       { hipLaunchKernelGGL((binary_lut6_kernel<4, false>), grid, block, 0, st, a); }
                 break;
        }
    }
    BBHIP_LAUNCH_CHECK();
    return 0;
}

int bbhip_bit_BinaryLutN_Forward(int n, int const *dev_x_buf, int *dev_y_buf, int const *dev_input_index, int const *dev_table,
                                 int node_size, int frame_size, int frame_stride, void *stream)
{
    if (n == 6) { return bbhip_bit_BinaryLut6_Forward(dev_x_buf, dev_y_buf, dev_input_index, dev_table, node_size, frame_size, frame_stride, stream); }
    clear_hints();
    if (n < 2 || n > 6) { return fail("%s: LUT width n=%d not in 2..6", __func__, n); }
    BBHIP_REQUIRE(dev_x_buf != nullptr && dev_y_buf != nullptr && dev_input_index != nullptr && dev_table != nullptr);
    BBHIP_REQUIRE(node_size > 0 && node_size <= (0x7fffffff >> 6) && frame_size > 0);
    BBHIP_REQUIRE(frame_stride >= (frame_size + 31) / 32);
    hipStream_t st = static_cast<hipStream_t>(stream);
    uint32_t const *x = reinterpret_cast<uint32_t const *>(dev_x_buf);
    uint32_t *y = reinterpret_cast<uint32_t *>(dev_y_buf);
    int const words = (frame_size + 31) / 32;
    ScopedTimer tm(kTimeBinary, st);
    for (int n0 = 0; n0 < node_size; n0 += 65535) {            // grid.y is limited to 65535 nodes per launch
        dim3 const grid(ceil_div(words, kBlock), (node_size - n0 < 65535) ? node_size - n0 : 65535), block(kBlock);
        switch (n) {
        case 2: hipLaunchKernelGGL(binary_lutn_kernel<2>, grid, block, 0, st, x, y, dev_input_index, dev_table, n0, frame_size, frame_stride); break;
        case 3: hipLaunchKernelGGL(binary_lutn_kernel<3>, grid, block, 0, st, x, y, dev_input_index, dev_table, n0, frame_size, frame_stride); break;
        case 4: hipLaunchKernelGGL(binary_lutn_kernel<4>, grid, block, 0, st, x, y, dev_input_index, dev_table, n0, frame_size, frame_stride); break;
        default: hipLaunchKernelGGL(binary_lutn_kernel<5>, grid, block, 0, st, x, y, dev_input_index, dev_table, n0, frame_size, frame_stride); break;
        }
        BBHIP_LAUNCH_CHECK();
    }
    return 0;
}

}  // extern "C"
