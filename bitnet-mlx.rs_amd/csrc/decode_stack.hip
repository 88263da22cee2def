// One launch for the BitLinear projections of a run of decoder blocks at one token (batch-1 decode).
//
// At one token a decoder block is four dependent steps (q,k,v | o | gate,up | down), each a few megabytes of
// weights: launched one by one, the time goes to launch hand-over and to waiting for the first weight bytes,
// not to HBM bandwidth.  This kernel keeps one workgroup per compute unit resident for the whole run of blocks
// and replaces the launch boundaries by a barrier across the grid.  What makes that pay:
//   * weights do not depend on activations, so a workgroup requests the weight tiles of its NEXT step (into
//     registers) before it waits at the barrier; HBM streams while the barrier and the quantiser run;
//   * a step's input row is read, normalised and quantised by every workgroup for itself, exactly as in the
//     fused decode GEMV (same code from rowquant.hpp, same summation order, same bits).
//
// Per step a workgroup of 16 wavefronts owns up to four 16-row blocks (blocks b, b+G, ... for workgroup b of G),
// at most 75 weight tiles; wavefronts 0..14 take tiles w, w+15, ... and leave one partial sum per tile and row
// in LDS; wavefront 15 holds no tiles: it polls the barrier flags, so that its polls do not queue behind weight
// loads (a wavefront's loads return in issue order).  The quantiser keeps the declared summation order of the sum of squares (256 virtual
// lanes): all 1024 threads load, square, normalise and round their own chunks, but the chains of additions run
// in threads 0..255 over the squares parked in LDS.
//
// Measured on MI355X (BitNet-2B shapes): a step costs about 7.3 us either way, about 3.3 us of it the barrier
// (store acknowledgement, flag propagation and a poll, each a trip through the fabric between XCDs), which is
// what a kernel boundary costs as well; over 30 blocks the single launch is about 5 % faster than 120 launches.
// The path is therefore optional (bitnet_hip_decoder_set_single_launch).
//
// Layer composition: bitnet-inference/src/engine/transformer_layers.rs:626-710 (projections only; the
// attention mixing between v and o is outside this path, v is broadcast to the query heads instead),
// feed-forward :603-623 with ReLU^2 gating :307-316.
//
// Grid barrier and visibility.  The compute units sit in eight XCDs whose L2 caches are not coherent with each
// other, and cache-wide write-back / invalidate fences cost tens of microseconds here.  Instead:
//   * a step's outputs are stored with device-scope (sc1, write-through) stores; each wavefront waits until its
//     stores are acknowledged (vmcnt 0), the workgroup meets at its own barrier, and only then does workgroup b
//     publish flags[b] = epoch, again with an sc1 store;
//   * every workgroup polls the G flags (one per thread, sc1 loads) until all have reached the epoch;
//   * activations live in a ring with one slice per block, so within a launch no address is written after it
//     has been read and none is read before the barrier that follows its writing: an L2 can hold no stale copy,
//     and plain cached loads are safe (the first reader of an XCD fills its L2, the other 31 workgroups hit);
//   * in the ring every 16-row block of an activation vector has a 128-byte line of its own (element n sits at
//     float 32*(n/16) + n%16), so no cache line of the ring is written by two workgroups.
// Epochs only grow, across launches too, so the flags never need clearing.  Every wait is bounded: after
// SPIN_LIMIT ticks of the 100 MHz clock, or when another workgroup has given up, the workgroup raises the
// abort word and leaves the kernel, so the grid always drains; the host reports the failure at the next call.
#include "kernels.hpp"
#include "rowquant.hpp"
#include "tiledot.hpp"

namespace bitnet {

namespace {

#ifndef STACK_NT
#define STACK_NT 1024
#endif
constexpr int NT = STACK_NT;    // threads per workgroup
constexpr int NW = NT / 64;     // wavefronts
constexpr int TW = NW - 1;      // wavefronts that hold weight tiles; the last one polls the grid barrier
constexpr int SLOTS = (40 + TW - 1) / TW;  // weight tiles (16 bytes per lane) such a wavefront holds for one step
constexpr int MAX_TILES = TW * SLOTS;
constexpr int MAX_RB = 4;       // row blocks per workgroup and step
constexpr int NCH = 2048 / NT;  // 16-byte f32 chunks of the input row per thread: K <= 8192
constexpr int MAX_LAYERS = 32;  // blocks per launch (the descriptions of their steps sit in LDS)
constexpr long long SPIN_LIMIT = 5000000;  // 50 ms

struct PhaseProj {
    const uint8_t *w;
    float ws;
    float *out;
    int n;
    int rb_end;      // cumulative row blocks
    int out_padded;  // out is a ring vector (one 128-byte line per 16 elements) rather than a dense one
};
struct Phase {  // one step of one block, the same for the whole grid; kept in LDS
    PhaseProj proj[3];
    int nproj;
    int nrb;  // row blocks per workgroup in this step
    const float *x, *x2, *gamma, *residual;
    int x_padded, res_padded;
    int k, kt_count;
};

// Float offset of element n of a ring vector.
__device__ __forceinline__ int padded(int n) { return ((n >> 4) << 5) + (n & 15); }

struct Shared {
    Phase phases[4 * MAX_LAYERS];     // every step of the launch, built once at its start
    int red[MAX_TILES][TILE_ROWS];    // per weight tile: sum over its 256 columns, per row
    float red_f[2][NW];
    int red_i[NW];
    float scale;
    int verdict;  // of the polling wavefront: 1 = everyone has arrived, 2 = give up
};

// The description of step ph; every step of the launch is built by a thread of its own at the start.
__device__ __forceinline__ void make_phase(const StackParams &p, int ph, Phase &P)
{
    const int li = ph >> 2, l = p.layer_begin + li, kind = ph & 3;
    const bool last = l + 1 == p.layer_end;
    const StackLayer &L = p.table[l];
    // ring slice of block l: q | k | v | x1 | gate | up | x_next, each padded (32 floats per 16 elements)
    auto pad = [](int n) { return ((n + 15) >> 4) << 5; };
    const int o_k = pad(p.hidden), o_v = o_k + pad(p.kv_dim), o_x1 = o_v + pad(p.kv_dim), o_gate = o_x1 + pad(p.hidden),
              o_up = o_gate + pad(p.ffn), o_xn = o_up + pad(p.ffn);
    float *slice = p.ring + (size_t)l * p.ring_stride;
    const bool first = l == p.layer_begin;
    const float *xin = first ? p.x_in : p.ring + (size_t)(l - 1) * p.ring_stride + o_xn;
    P.x2 = nullptr; P.gamma = nullptr; P.residual = nullptr; P.x_padded = 1; P.res_padded = 1;
    const PhaseProj none = {nullptr, 0.0f, nullptr, 0, 0, 0};
    P.proj[0] = P.proj[1] = P.proj[2] = none;
    int rb_total = 0;
    auto make = [&](int proj, float *ring_out, float *user_out, int n) {
        rb_total += (n + TILE_ROWS - 1) / TILE_ROWS;
        PhaseProj q = {L.w[proj], *L.w_scale[proj], user_out ? user_out : ring_out, n, rb_total, user_out ? 0 : 1};
        return q;
    };
    if (kind == 0) {
        P.x = xin; P.x_padded = !first; P.gamma = p.gamma + (size_t)(2 * l) * p.hidden; P.k = p.hidden; P.nproj = 3;
        P.proj[0] = make(BITNET_HIP_PROJ_Q, slice, last ? p.q_last : nullptr, p.hidden);
        P.proj[1] = make(BITNET_HIP_PROJ_K, slice + o_k, last ? p.k_last : nullptr, p.kv_dim);
        P.proj[2] = make(BITNET_HIP_PROJ_V, slice + o_v, nullptr, p.kv_dim);
    } else if (kind == 1) {
        P.x = slice + o_v; P.residual = xin; P.res_padded = !first; P.k = p.hidden; P.nproj = 1;
        P.proj[0] = make(BITNET_HIP_PROJ_O, slice + o_x1, nullptr, p.hidden);
    } else if (kind == 2) {
        P.x = slice + o_x1; P.gamma = p.gamma + (size_t)(2 * l + 1) * p.hidden; P.k = p.hidden; P.nproj = 2;
        P.proj[0] = make(BITNET_HIP_PROJ_GATE, slice + o_gate, nullptr, p.ffn);
        P.proj[1] = make(BITNET_HIP_PROJ_UP, slice + o_up, nullptr, p.ffn);
    } else {
        P.x = slice + o_gate; P.x2 = slice + o_up; P.residual = slice + o_x1; P.k = p.ffn; P.nproj = 1;
        P.proj[0] = make(BITNET_HIP_PROJ_DOWN, slice + o_xn, last ? p.x_out : nullptr, p.hidden);
    }
    P.kt_count = (P.k + TILE_K - 1) / TILE_K;
    P.nrb = (rb_total + (int)gridDim.x - 1) / (int)gridDim.x;
}

// Pointers of the step description come out of LDS as generic pointers; accesses through a generic pointer are
// flat instructions, which count against the LDS wait counter as well, so that every wait for an LDS read would
// also wait for the weight tiles in flight.  Routing the pointer through the global address space makes the
// compiler emit global loads and stores.
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
#define BITNET_GLOBAL __attribute__((address_space(1)))
__device__ __forceinline__ float4 load_global4(const float *ptr)
{
    const f32x4 v = *(const BITNET_GLOBAL f32x4 *)(uintptr_t)ptr;
    return make_float4(v[0], v[1], v[2], v[3]);
}
__device__ __forceinline__ uint4 load_global4(const uint4 *ptr)
{
    const u32x4 v = *(const BITNET_GLOBAL u32x4 *)(uintptr_t)ptr;
    return make_uint4(v[0], v[1], v[2], v[3]);
}
__device__ __forceinline__ float load_global(const float *ptr) { return *(const BITNET_GLOBAL float *)(uintptr_t)ptr; }

__device__ __forceinline__ int total_row_blocks(const Phase &P) { return P.proj[P.nproj - 1].rb_end; }

// Row block rb of the step -> projection index and the block's position inside that projection.
__device__ __forceinline__ void locate(const Phase &P, int rb, int &pj, int &local)
{
    pj = 0;
    if (P.nproj > 1 && rb >= P.proj[0].rb_end) pj = 1;
    if (P.nproj > 2 && rb >= P.proj[1].rb_end) pj = 2;
    local = rb - (pj == 0 ? 0 : P.proj[pj - 1].rb_end);
}

// The i-th row block of this workgroup.
__device__ __forceinline__ int row_block_of(int i) { return (int)blockIdx.x + i * (int)gridDim.x; }

// Tile T of the workgroup (T = i * kt_count + kt) -> row block index i (at most MAX_RB - 1) and k-tile kt.
__device__ __forceinline__ void tile_of(const Phase &P, int T, int &i, int &kt)
{
    i = (T >= P.kt_count) + (T >= 2 * P.kt_count) + (T >= 3 * P.kt_count);
    kt = T - i * P.kt_count;
}

// Request the step's weight tiles: the workgroup's tiles are numbered T = i * kt_count + kt (i-th row block,
// k-tile kt); slot u of wavefront w < TW holds tile w + TW * u.
__device__ __forceinline__ void prefetch(const Phase &P, uint4 (&wreg)[SLOTS])
{
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int total = total_row_blocks(P);
#pragma unroll
    for (int u = 0; u < SLOTS; ++u) {
        const int T = wave + TW * u;
        int i, kt;
        tile_of(P, T, i, kt);
        const int rb = row_block_of(i);
        wreg[u] = make_uint4(0, 0, 0, 0);
        if (wave < TW && T < P.nrb * P.kt_count && rb < total) {
            int pj, local;
            locate(P, rb, pj, local);
            wreg[u] = load_global4(reinterpret_cast<const uint4 *>(P.proj[pj].w) + ((size_t)local * P.kt_count + kt) * 64 + lane);
        }
    }
}

// Device-scope (write-through) store: visible to the other XCDs once acknowledged.
__device__ __forceinline__ void store_device_scope(float *ptr, float v)
{
    __hip_atomic_store((BITNET_GLOBAL unsigned *)(uintptr_t)ptr,
                       __builtin_bit_cast(unsigned, v), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Time stamps of the segments of a step (100 MHz clock), for a timing build with -DSTACK_TIMING only.
#ifdef STACK_TIMING
__device__ long long stack_stamps[64 * 8 * 2];
#define STACK_STAMP(i)                                                                                        \
    if (threadIdx.x == 0 && ph < 64 && (blockIdx.x == 0 || blockIdx.x == gridDim.x - 1))                       \
        stack_stamps[(ph * 8 + (i)) * 2 + (blockIdx.x != 0)] = wall_clock64();
#else
#define STACK_STAMP(i)
#endif

// Quantise the step's input row into LDS, multiply with the tiles held in registers, finish and store the
// workgroup's output rows.  lds_a: the int8 row (zero past K); lds_sq: the squares of the row (RMSNorm steps).
template <int MODE>
__device__ __forceinline__ void run_phase(const StackParams &p, const uint4 (&wreg)[SLOTS], uint4 *lds_a, float4 *lds_sq,
                                          Shared &sh, int ph)
{
    const Phase &P = sh.phases[ph];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int chunks = P.k >> 2, lds_words = P.kt_count * 64;
    uint32_t *lds_w = reinterpret_cast<uint32_t *>(lds_a);
    const bool norm = P.gamma != nullptr;

    // what the epilogue threads (16 per row block) will need from memory is requested first
    int e_n = -1, e_pj = 0;
    float e_res = 0.0f;
    if (tid < TILE_ROWS * MAX_RB) {
        const int i = tid >> 4, r = tid & 15, rb = row_block_of(i);
        if (i < P.nrb && rb < total_row_blocks(P)) {
            int local;
            locate(P, rb, e_pj, local);
            const int n = local * TILE_ROWS + r;
            if (n < P.proj[e_pj].n) {
                e_n = n;
                if (P.residual) e_res = load_global(P.residual + (P.res_padded ? padded(n) : n));  // single-projection steps only
            }
        }
    }

    // Chunk c is elements 4c .. 4c+3 after the step's input transform (as load_chunk of rowquant.hpp).  The row was
    // written before the last grid barrier (or by an earlier launch) at addresses nobody has read since.
    float4 v[NCH], gm[NCH];
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
        const int c = tid + NT * i;
        v[i] = gm[i] = make_float4(0.f, 0.f, 0.f, 0.f);
        if (c < chunks) {
            // float offset of (transformed) element 4c in its source vector; chunks never straddle a 16-element line
            int e = 4 * c;
            if constexpr (MODE == BITNET_HIP_INPUT_GQA_BROADCAST) {
                const int h = e / p.head_dim, d = e - h * p.head_dim;
                e = (h / p.gqa_group) * p.head_dim + d;
            }
            const int off = P.x_padded ? padded(e) : e;
            if constexpr (MODE == BITNET_HIP_INPUT_RELU2_MUL) {
                const float4 g = load_global4(P.x + off), u = load_global4(P.x2 + off);
                v[i] = make_float4(relu2_mul(g.x, u.x), relu2_mul(g.y, u.y), relu2_mul(g.z, u.z), relu2_mul(g.w, u.w));
            } else {
                v[i] = load_global4(P.x + off);
            }
            if (norm) gm[i] = load_global4(P.gamma + 4 * (size_t)c);
        }
    }
    RowDivisor rdiv = {1.0f, 1.0f, false};
    if (norm) {
        // sum of squares in the declared order: virtual lane t (thread t < 256) adds the squares of chunks
        // t, t + 256, ... element by element, then the butterflies and the four-way sum (rowquant.hpp)
#pragma unroll
        for (int i = 0; i < NCH; ++i) {
            const int c = tid + NT * i;
            if (c < chunks)
                lds_sq[c] = make_float4(f32_mul(v[i].x, v[i].x), f32_mul(v[i].y, v[i].y), f32_mul(v[i].z, v[i].z),
                                        f32_mul(v[i].w, v[i].w));
        }
        lds_barrier();
        if (tid < 256) {
            float part = 0.0f;
            for (int c = tid; c < chunks; c += 256) {
                const float4 q = lds_sq[c];
                part = f32_add(f32_add(f32_add(f32_add(part, q.x), q.y), q.z), q.w);
            }
            part = wave_sum_f32(part);
            if (lane == 0) sh.red_f[0][wave] = part;
        }
        lds_barrier();
        const float ss = f32_add(f32_add(f32_add(sh.red_f[0][0], sh.red_f[0][1]), sh.red_f[0][2]), sh.red_f[0][3]);
        rdiv = make_row_divisor(rms_from_ss(ss, P.k, p.eps));
    }
    float amax = 0.0f;
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
        const int c = tid + NT * i;
        if (norm && c < chunks) v[i] = normalize4(v[i], rdiv, gm[i]);
        amax = absmax4(amax, v[i]);
    }
    amax = wave_max_f32(amax);
    if (lane == 0) sh.red_f[1][wave] = amax;
    lds_barrier();
    STACK_STAMP(4);
    amax = 0.0f;
#pragma unroll
    for (int w = 0; w < NW; ++w) amax = fmaxf(amax, sh.red_f[1][w]);
    const float scale = scale_from_absmax(amax);
    int isum = 0;
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
        const int c = tid + NT * i;
        if (c < chunks) lds_w[c] = quant4_packed(v[i], scale, &isum);
        else if (c < lds_words) lds_w[c] = 0;
    }
    isum = wave_sum_i32(isum);
    if (lane == 0) sh.red_i[wave] = isum;
    if (tid == 0) sh.scale = scale;
    lds_barrier();
    STACK_STAMP(5);

    const int kq = lane >> 4;
    if (wave < TW) {
#pragma unroll
        for (int u = 0; u < SLOTS; ++u) {
            const int T = wave + TW * u;
            if (T < P.nrb * P.kt_count) {  // tiles of row blocks past the end were loaded as zero
                int i, kt;
                tile_of(P, T, i, kt);
                int acc = dot64(wreg[u], lds_a + kt * 16 + kq, 0);
                acc = sum_over_lane_groups(acc);
                if (lane < TILE_ROWS) sh.red[T][lane] = acc;
            }
        }
    }
    lds_barrier();
    STACK_STAMP(6);

    if (e_n >= 0) {
        const int i = tid >> 4, r = tid & 15;
        int total = 0;
        for (int kt = 0; kt < P.kt_count; ++kt) total += sh.red[i * P.kt_count + kt][r];
        int asum = 0;
#pragma unroll
        for (int w = 0; w < NW; ++w) asum += sh.red_i[w];
        total -= asum;
        float y = f32_mul((float)total, P.proj[e_pj].ws);
        y = f32_div(y, sh.scale);
        if (P.residual) y = f32_add(y, e_res);
        store_device_scope(P.proj[e_pj].out + (P.proj[e_pj].out_padded ? padded(e_n) : e_n), y);
    }
}

// Once every wavefront's stores have been acknowledged, the workgroup's flag takes the epoch.
__device__ __forceinline__ void grid_arrive(const StackParams &p, unsigned epoch)
{
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // nothing else of this wavefront is in flight at this point
    lds_barrier();
    if (threadIdx.x == 0) __hip_atomic_store(&p.flags[blockIdx.x], epoch, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Wait until every workgroup's flag has reached the epoch.  Only the last wavefront polls (it has no weight loads
// in flight); the others wait for it at the workgroup barrier.  Returns false (for the whole workgroup) when
// the wait was abandoned.
__device__ __forceinline__ bool grid_wait(const StackParams &p, unsigned epoch, Shared &sh)
{
    const int tid = threadIdx.x, lane = tid & 63;
    int verdict = 0;  // 1: everyone has arrived, 2: give up
    if (tid >= NT - 64) {
        const long long t0 = wall_clock64();
        for (;;) {
            bool ok = true;
            for (int b = lane; b < (int)gridDim.x; b += 64) {
                const unsigned f = __hip_atomic_load(&p.flags[b], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                ok = ok && (int)(f - epoch) >= 0;
            }
            if (__builtin_amdgcn_ballot_w64(!ok) == 0) { verdict = 1; break; }
            const unsigned ab = __hip_atomic_load(p.abort_word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if (ab != 0 || wall_clock64() - t0 > p.spin_limit) { verdict = 2; break; }  // uniform over the wavefront
        }
    }
    if (tid == NT - 64) sh.verdict = verdict;
    lds_barrier();
    if (sh.verdict == 2) {
        if (tid == 0) {
            __hip_atomic_store(p.abort_word, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_store(p.host_status, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
        }
        return false;
    }
    asm volatile("" ::: "memory");  // compiler only: no global load of the step may be hoisted above the wait
    return true;
}

__global__ __launch_bounds__(NT, 1) void decode_stack_kernel(StackParams p)
{
    extern __shared__ uint4 lds_dyn[];  // the int8 input row of the current step, then the f32 squares of a row
    __shared__ Shared sh;
    uint4 *lds_a = lds_dyn;
    float4 *lds_sq = reinterpret_cast<float4 *>(lds_dyn + p.lds_row_bytes / 16);
    uint4 wreg[SLOTS];

    // every step of the launch is described once, by a thread of its own
    const int nphase = p.step_end;  // steps are numbered from the first step of block layer_begin
    if ((int)threadIdx.x >= p.step_begin && (int)threadIdx.x < nphase) make_phase(p, threadIdx.x, sh.phases[threadIdx.x]);
    lds_barrier();

    prefetch(sh.phases[p.step_begin], wreg);
    for (int ph = p.step_begin; ph < nphase; ++ph) {
        STACK_STAMP(0);
        if (ph > p.step_begin && !grid_wait(p, p.epoch0 + (unsigned)(ph - p.step_begin), sh)) return;
        STACK_STAMP(1);
        const int kind = ph & 3;
        if (kind == 1) run_phase<BITNET_HIP_INPUT_GQA_BROADCAST>(p, wreg, lds_a, lds_sq, sh, ph);
        else if (kind == 3) run_phase<BITNET_HIP_INPUT_RELU2_MUL>(p, wreg, lds_a, lds_sq, sh, ph);
        else run_phase<BITNET_HIP_INPUT_PLAIN>(p, wreg, lds_a, lds_sq, sh, ph);
        STACK_STAMP(2);
        if (ph + 1 < nphase) {
            grid_arrive(p, p.epoch0 + (unsigned)(ph - p.step_begin) + 1u);
            STACK_STAMP(3);
            prefetch(sh.phases[ph + 1], wreg);
        }
    }
}

}  // namespace

bool decode_stack_supported(size_t hidden, size_t ffn, size_t kv_dim, size_t head_dim, int sum_order, int grid)
{
    if (sum_order != BITNET_HIP_SUM_BLOCK256 || grid <= 0) return false;
    if (hidden % 4 || ffn % 4 || head_dim % 4 || kv_dim % 4) return false;
    const size_t g = (size_t)grid;
    auto per_group = [&](size_t rbs) { return (rbs + g - 1) / g; };  // row blocks per workgroup
    const size_t nrb_qkv = per_group(row_blocks(hidden) + 2 * row_blocks(kv_dim)), nrb_o = per_group(row_blocks(hidden)),
                 nrb_gu = per_group(2 * row_blocks(ffn));
    if (nrb_qkv > (size_t)MAX_RB || nrb_gu > (size_t)MAX_RB) return false;
    // tiles a workgroup can hold
    if ((nrb_qkv > nrb_gu ? nrb_qkv : nrb_gu) * k_tiles(hidden) > (size_t)MAX_TILES || nrb_o * k_tiles(ffn) > (size_t)MAX_TILES)
        return false;
    if (hidden > (size_t)NCH * NT * 4 || ffn > (size_t)NCH * NT * 4) return false;  // chunks a thread can hold
    if (hidden % 16 || kv_dim % 16 || ffn % 16 || head_dim % 16) return false;      // whole 16-element lines
    return true;
}

size_t decode_stack_max_layers() { return MAX_LAYERS; }

size_t decode_stack_ring_stride(size_t hidden, size_t ffn, size_t kv_dim)
{
    auto pad = [](size_t n) { return (n + 15) / 16 * 32; };  // one 128-byte line per 16 elements
    return 3 * pad(hidden) + 2 * pad(kv_dim) + 2 * pad(ffn);
}

int launch_decode_stack(const StackParams &params, int grid, hipStream_t stream)
{
    StackParams p = params;
    p.spin_limit = SPIN_LIMIT;
    p.lds_row_bytes = (int)(k_tiles((size_t)(p.hidden > p.ffn ? p.hidden : p.ffn)) * TILE_K);
    const size_t lds = (size_t)p.lds_row_bytes + k_tiles((size_t)p.hidden) * TILE_K * sizeof(float);
    void *args[] = {&p};
    hipError_t e = hipLaunchCooperativeKernel(reinterpret_cast<const void *>(&decode_stack_kernel), dim3(grid), dim3(NT),
                                              args, lds, stream);
    if (e != hipSuccess) {
        (void)hipGetLastError();
        return fail(BITNET_HIP_KERNEL_ERROR, "decode_stack_kernel: cooperative launch failed: %s", hipGetErrorString(e));
    }
    return BITNET_HIP_OK;
}

}  // namespace bitnet
