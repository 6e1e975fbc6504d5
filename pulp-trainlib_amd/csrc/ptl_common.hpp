// Shared declarations of the HIP side: separable index maps, the GEMM
// problem descriptor, library state and error plumbing.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace ptl {

typedef _Float16 half_t;

// Largest spatial extent the packed coordinate look-up entries can carry.
constexpr int HW_LIMIT = 8191;

// ---------------------------------------------------------------------------
// Separable three-digit index map.
//
// An index idx in [0, n) is split as idx = (q2*d1 + q1)*d0 + q0 and mapped to
//   off = q2*o2 + q1*o1 + q0*o0 + ob   (element offset into a tensor)
//   h   = q2*h2 + q1*h1 + q0*h0 + hb   (vertical coordinate contribution)
//   w   = q2*w2 + q1*w1 + q0*w0 + wb   (horizontal coordinate contribution)
// A GEMM operand element (row, k) lives at off(row) + off(k) and exists iff
// 0 <= h(row)+h(k) < HL and 0 <= w(row)+w(k) < WL; elements that do not exist
// read as zero.  Plain matrices, batched CHW/HWC tensors and the implicit
// im2col patch matrices of forward, weight-gradient and input-gradient
// convolution are all instances of this form.
// ---------------------------------------------------------------------------
struct AxisMap {
    int n;           // extent
    int d1, d0;      // digit radices
    int o2, o1, o0, ob;
    int h2, h1, h0, hb;
    int w2, w1, w0, wb;
};

// How an operand tile is fetched from global memory.
enum FillMode : int {
    FILL_ELEM_K = 0,  // element loads, consecutive threads along k
    FILL_ELEM_R = 1,  // element loads, consecutive threads along rows
    FILL_VEC_K = 2,   // 16-byte loads along k   (k is a plain contiguous axis)
    FILL_VEC_R = 3,   // 16-byte loads along rows (row is a contiguous axis)
};

struct OperandMap {
    AxisMap row;
    AxisMap k;
    int HL, WL;  // coordinate box
    int mode;    // FillMode
};

struct OutMap {
    AxisMap n;
    AxisMap m;
};

struct GemmArgs {
    const void *A;
    const void *B;
    void *C;       // output tensor (written through `c` when splits == 1)
    float *ws;     // split-K partial sums, [splits][N][M] fp32
    OperandMap a;  // rows = n index
    OperandMap b;  // rows = m index
    OutMap c;
    int N, M, K;
    int splits;
    int kchunk;    // K range per split (multiple of the k tile)
    int tiles_n, tiles_m;
    // Convolution as a sum over filter taps (look-up-free kernel only): k runs over (tap, channel); after the
    // `slabs_per_tap` slabs of a tap the A pointer jumps to the next tap of the padded, channel-blocked input:
    // by tap_jump_x bytes within a filter row, by tap_jump_y at the end of one.  taps <= 1: an ordinary product.
    // Lean kernel, k in runs: after every seg_slabs slabs the slab pointers of A / B jump by these bytes (k
    // made of an outer digit and a contiguous inner one, e.g. (sample, pixel)); 0 = k is one run.
    int seg_slabs;
    long long a_seg_jump, b_seg_jump;
    int taps, slabs_per_tap, tap_kw;
    long long tap_jump_x, tap_jump_y;
    // Weight gradient over taps: grid.y enumerates (tap, k split), tap_splits splits per tap; tap (ky, kx) reads
    // B shifted by ky*tap_jump_y + kx*tap_jump_x bytes and writes its own partial sums.  0: off.
    int tap_splits;
};

inline AxisMap axis_plain(int n, int stride, int base = 0) {
    AxisMap a = {};
    a.n = n;
    a.d1 = 1;
    a.d0 = n > 0 ? n : 1;
    a.o0 = stride;
    a.ob = base;
    return a;
}

// idx = q1*d0 + q0 with independent strides (e.g. (sample, pixel)).
inline AxisMap axis_two(int n, int d0, int s1, int s0, int base = 0) {
    AxisMap a = {};
    a.n = n;
    a.d1 = 1 << 30;
    a.d0 = d0;
    a.o1 = s1;
    a.o0 = s0;
    a.ob = base;
    return a;
}

__host__ __device__ inline void axis_decode(const AxisMap &a, int idx, int &off, int &h, int &w) {
    // One- and two-digit maps are the common case; skip the divisions they do not need
    // (the branches are uniform across a wave).
    int q0, q1, q2;
    if (a.d0 >= a.n) {
        q0 = idx;
        q1 = 0;
        q2 = 0;
    } else if (a.d1 >= (1 << 30)) {
        q1 = idx / a.d0;
        q0 = idx - q1 * a.d0;
        q2 = 0;
    } else {
        int t = idx / a.d0;
        q0 = idx - t * a.d0;
        q2 = t / a.d1;
        q1 = t - q2 * a.d1;
    }
    off = q2 * a.o2 + q1 * a.o1 + q0 * a.o0 + a.ob;
    h = q2 * a.h2 + q1 * a.h1 + q0 * a.h0 + a.hb;
    w = q2 * a.w2 + q1 * a.w1 + q0 * a.w0 + a.wb;
}

// ---------------------------------------------------------------------------
// Library state
// ---------------------------------------------------------------------------
struct State {
    bool ready = false;
    int device = -1;
    hipStream_t stream = nullptr;
    float *ws = nullptr;  // split-K / partial-sum workspace
    size_t ws_bytes = 0;
    void *scratch = nullptr;  // general scratch (dilated gradients, staging)
    size_t scratch_bytes = 0;
    hipEvent_t ev0 = nullptr, ev1 = nullptr;
    int num_cu = 256;
    void *zeros = nullptr;  // 256 zero bytes: source of elements that do not exist
    int gemm_path = 0;      // 0: fastest kernel that fits; 1: staged GEMM only; 2: direct convolution whenever it fits; 3: tap-sum route on the GEMM whenever it fits; 5: tap-sum route, LDS-resident input tile where it fits
    int last_gemm_streamed = 0;  // 1 if the last pipelined GEMM ran the streaming kernel
    int last_conv_resident = 0;  // 1 if the last Conv2D forward / input-gradient call kept its input tile in LDS for all taps
    int last_conv_direct = 0;  // 1 if the last Conv2D forward / input-gradient call ran the direct kernel
    int last_gemm_tile = 0;    // rows * 1000 + columns of the tile of the last look-up-free pipelined product
};

State &state();
bool ensure_init();
void set_error(const char *fmt, ...);
bool hip_ok(hipError_t e, const char *what);
float *workspace(size_t bytes);
void *scratch(size_t bytes);

template <typename T>
int gemm(const GemmArgs &g);  // returns 0 on success

// Pipelined LDS-DMA kernel: 0 = launched, -1 = problem does not fit, 2 = HIP failure.
template <typename T>
int gemm_async(GemmArgs &g);

// Two independent products; one launch where both fit the look-up-free kernel with the same
// tile shape, else one after the other.
template <typename T>
int gemm_pair(const GemmArgs &g0, const GemmArgs &g1);
template <typename T>
int gemm_async_pair(GemmArgs &g0, GemmArgs &g1);

// GEMV / outer-product kernels for products with a unit dimension.
template <typename T>
int mm_dispatch(const T *A, const T *B, T *C, int N, int M, int K, int trans_B);

}  // namespace ptl
