// lm_head: the vocabulary projection whose consumer wants a token, not 262 144 logits.
//
//   greedy   the projection with the argmax as its epilogue: each wavefront keeps the best packed (score, row)
//            of its rows and a small second kernel folds those; no logit is ever stored.  Replaces
//            rocm_mlx_q4_projection_greedy (go/engine/hip/kernels/quant/affine_projection_fused.hipinc:190-248).
//   scores   every row's (score, row) packed into 64 bits, the input of top-k sampling:
//            rocm_mlx_q4_projection_scores (:411-446).
//   top-k    the k largest packed values, sorted descending: what rocm_packed_topk
//            (go/engine/hip/kernels/sampling/topk.hipinc:45-84) yields per chunk, here per wavefront segment
//            and repeated until one segment is left.
//
// The streaming part is the dot2 body; only the epilogue differs.  pack_scores_kernel applies the same two
// epilogues to fp32 scores already in memory (shapes the dot2 kernels do not take, several rows).
#include "aq_qmv_body.h"

namespace aq {

template <int BITS, int R, int FUSE>
__global__ __launch_bounds__(4 * kWave) void qmv_head_kernel(const QmvArgs a) {
    qmv_dot2_body<BITS, 1, R, 4, 2, false, FUSE>(a, blockIdx.x);
}

typedef void (*QmvHeadKernel)(const QmvArgs);
struct QmvHeadEntry {
    int bits, fuse, rows;
    QmvHeadKernel fn;
};
#define AQ_HEAD(BITS, FUSE, R) {BITS, FUSE, R, qmv_head_kernel<BITS, R, FUSE>}
#define AQ_HEAD_SET(BITS) \
    AQ_HEAD(BITS, 3, 1), AQ_HEAD(BITS, 3, 2), AQ_HEAD(BITS, 3, 4), AQ_HEAD(BITS, 4, 1), AQ_HEAD(BITS, 4, 2), AQ_HEAD(BITS, 4, 4)
static const QmvHeadEntry kHeadTable[] = {AQ_HEAD_SET(4), AQ_HEAD_SET(8)};

static const QmvHeadEntry* find_head(int bits, int fuse, int rows) {
    for (const QmvHeadEntry& e : kHeadTable)
        if (e.bits == bits && e.fuse == fuse && e.rows == rows) return &e;
    return nullptr;
}

bool qmv_head_supported(int bits, int fuse, int rows) { return find_head(bits, fuse, rows) != nullptr; }

size_t qmv_head_partials(int N, int rows) { return (size_t)((N + rows * 4 - 1) / (rows * 4)) * 4; }

// Folds the per-wavefront maxima into best[0]: kHeadFoldGroups workgroups each fold a slice into their own
// slot, take a ticket, and the one that draws the last ticket folds the slots and zeroes the ticket counter
// again.  Sixty-four tickets on one address are cheap; one ticket per wavefront of the projection is not.
__global__ __launch_bounds__(256) void fold_best_kernel(const unsigned long long* __restrict__ partial, int count,
                                                        unsigned long long* fold, unsigned long long* __restrict__ best) {
    unsigned int* tickets = reinterpret_cast<unsigned int*>(fold);
    unsigned long long* slots = fold + 16;
    const int per_group = (count + kHeadFoldGroups - 1) / kHeadFoldGroups;
    const int begin = blockIdx.x * per_group;
    const int end = min(begin + per_group, count);
    unsigned long long mine = 0;
    constexpr int U = 4;
    for (int base = begin; base < end; base += 256 * U) {
        unsigned long long t[U];
#pragma unroll
        for (int u = 0; u < U; u++) {
            const int i = base + u * 256 + (int)threadIdx.x;
            // clamped, not predicated: reading a value twice does not change a maximum, and the loads stay
            // unconditional so that all of them are issued before the first is waited for
            t[u] = partial[min(i, end - 1)];
        }
#pragma unroll
        for (int u = 0; u < U; u++) mine = t[u] > mine ? t[u] : mine;
    }
    if (begin >= end) mine = 0;
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        const unsigned long long other = __shfl_xor(mine, o, kWave);
        mine = other > mine ? other : mine;
    }
    __shared__ unsigned long long wave_best[4];
    __shared__ int last;
    if ((threadIdx.x & (kWave - 1)) == 0) wave_best[threadIdx.x >> 6] = mine;
    __syncthreads();
    if (threadIdx.x == 0) {
        unsigned long long b = wave_best[0];
        for (int i = 1; i < 4; i++) b = wave_best[i] > b ? wave_best[i] : b;
        __atomic_store_n(&slots[blockIdx.x], b, __ATOMIC_RELAXED);
        __threadfence();
        last = atomicAdd(tickets, 1u) == (unsigned int)kHeadFoldGroups - 1u;
    }
    __syncthreads();
    if (!last || threadIdx.x >= kWave) return;
    __threadfence();
    unsigned long long m = __atomic_load_n(&slots[threadIdx.x], __ATOMIC_RELAXED);  // kHeadFoldGroups == 64 lanes
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        const unsigned long long other = __shfl_xor(m, o, kWave);
        m = other > m ? other : m;
    }
    if (threadIdx.x == 0) {
        best[0] = m;
        atomicExch(tickets, 0u);
    }
}

hipError_t qmv_head_launch(int bits, int fuse, int rows, const QmvArgs& a, hipStream_t stream) {
    const QmvHeadEntry* e = find_head(bits, fuse, rows);
    if (!e || a.M != 1) return hipErrorInvalidValue;
    const int rows_per_wg = rows * 4;
    const size_t lds = (size_t)a.K * 2;
    if (hipError_t rc = ensure_dynamic_lds(reinterpret_cast<const void*>(e->fn), (size_t)lds)) return rc;
    if (fuse == 3 && (!a.partial || !a.fold)) return hipErrorInvalidValue;
    hipLaunchKernelGGL(e->fn, dim3((unsigned)((a.N + rows_per_wg - 1) / rows_per_wg)), dim3(4 * kWave), lds, stream, a);
    hipError_t rc = hipGetLastError();
    if (rc != hipSuccess || fuse != 3) return rc;
    static_assert(kHeadFoldGroups == kWave, "the last workgroup reads one slot per lane");
    hipLaunchKernelGGL(fold_best_kernel, dim3(kHeadFoldGroups), dim3(256), 0, stream, a.partial,
                       (int)qmv_head_partials(a.N, rows), a.fold, reinterpret_cast<unsigned long long*>(a.y));
    return hipGetLastError();
}

// Greedy over a list of candidate rows (rocm_mlx_q4_projection_selected_greedy,
// go/engine/hip/kernels/quant/affine_projection_fused.hipinc:485-546).  The scores come from the gathered matvec: every
// candidate r is scored as one row of the window of `width` rows that starts at min(r, N - width) (an "expert" of a
// slab whose experts are one row apart), so a candidate costs width rows of weights and no kernel of its own is needed.
// windows: start[z] = first row of candidate z's window, -1 for an id outside [0, N).
__global__ __launch_bounds__(256) void selected_windows_kernel(const int32_t* __restrict__ rows, int count, int N, int width,
                                                               int32_t* __restrict__ start) {
    const int z = blockIdx.x * 256 + threadIdx.x;
    if (z >= count) return;
    const int r = rows[z];
    start[z] = (r >= 0 && r < N) ? min(r, N - width) : -1;
}
// pick: best[0] = max over the valid candidates with a finite score of pack(score, row); 0 when there is none.
__global__ __launch_bounds__(256) void selected_pick_kernel(const float* __restrict__ scores, const int32_t* __restrict__ rows,
                                                            const int32_t* __restrict__ start, int count, int width,
                                                            unsigned long long* __restrict__ best) {
    unsigned long long mine = 0;
    for (int z = threadIdx.x; z < count; z += 256) {
        const int e = start[z];
        if (e < 0) continue;
        const int r = rows[z];
        const float v = scores[(int64_t)z * width + (r - e)];
        if (isfinite(v)) {
            const unsigned long long p = pack_score_index(v, (uint32_t)r);
            mine = p > mine ? p : mine;
        }
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        const unsigned long long other = __shfl_xor(mine, o, kWave);
        mine = other > mine ? other : mine;
    }
    __shared__ unsigned long long wave_best[4];
    if ((threadIdx.x & (kWave - 1)) == 0) wave_best[threadIdx.x >> 6] = mine;
    __syncthreads();
    if (threadIdx.x == 0) {
        unsigned long long b = wave_best[0];
        for (int i = 1; i < 4; i++) b = wave_best[i] > b ? wave_best[i] : b;
        best[0] = b;
    }
}
hipError_t selected_windows_launch(const int32_t* rows, int count, int N, int width, int32_t* start, hipStream_t stream) {
    hipLaunchKernelGGL(selected_windows_kernel, dim3((unsigned)((count + 255) / 256)), dim3(256), 0, stream, rows, count, N, width, start);
    return hipGetLastError();
}
hipError_t selected_pick_launch(const float* scores, const int32_t* rows, const int32_t* start, int count, int width,
                                unsigned long long* best, hipStream_t stream) {
    hipLaunchKernelGGL(selected_pick_kernel, dim3(1), dim3(256), 0, stream, scores, rows, start, count, width, best);
    return hipGetLastError();
}

hipError_t head_fold_launch(const unsigned long long* partial, int count, unsigned long long* fold, unsigned long long* best,
                            hipStream_t stream) {
    hipLaunchKernelGGL(fold_best_kernel, dim3(kHeadFoldGroups), dim3(256), 0, stream, partial, count, fold, best);
    return hipGetLastError();
}

// grid.y = activation row; a workgroup folds its share of a row before touching the shared maximum
__global__ __launch_bounds__(256) void pack_scores_kernel(const float* __restrict__ scores, int N, const int32_t* suppress,
                                                          int suppress_count, unsigned long long* best,
                                                          unsigned long long* packed_out) {
    const int m = blockIdx.y;
    const float* row_scores = scores + (int64_t)m * N;
    unsigned long long mine = 0;
    for (int n = blockIdx.x * 256 + threadIdx.x; n < N; n += gridDim.x * 256) {
        const float v = row_scores[n];
        unsigned long long p = 0;
        if (isfinite(v) && !token_suppressed((uint32_t)n, suppress, suppress_count)) p = pack_score_index(v, (uint32_t)n);
        if (packed_out) packed_out[(int64_t)m * N + n] = p;
        mine = p > mine ? p : mine;
    }
    if (!best) return;
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        const unsigned long long other = __shfl_xor(mine, o, kWave);
        mine = other > mine ? other : mine;
    }
    __shared__ unsigned long long wave_best[4];
    if ((threadIdx.x & (kWave - 1)) == 0) wave_best[threadIdx.x >> 6] = mine;
    __syncthreads();
    if (threadIdx.x == 0) {
        unsigned long long b = wave_best[0];
        for (int i = 1; i < 4; i++) b = wave_best[i] > b ? wave_best[i] : b;
        if (b != 0) atomicMax(best + m, b);
    }
}

hipError_t pack_scores_launch(const float* scores, int M, int N, const int32_t* suppress, int suppress_count,
                              unsigned long long* best_or_null, unsigned long long* packed_or_null, hipStream_t stream) {
    if (M <= 0 || N <= 0) return hipSuccess;
    int bx = (N + 255) / 256;
    if (bx > 1024) bx = 1024;
    hipLaunchKernelGGL(pack_scores_kernel, dim3((unsigned)bx, (unsigned)M), dim3(256), 0, stream, scores, N, suppress,
                       suppress_count, best_or_null, packed_or_null);
    return hipGetLastError();
}

// Maximum over the 64 lanes, unsigned: DPP folds inside each row of 16 lanes (a lane out of range reads 0,
// the identity), then the four row results meet through SGPRs.
__device__ __forceinline__ uint32_t wave_max_u32(uint32_t v) {
    v = max(v, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0xB1, 0xF, 0xF, true));
    v = max(v, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x4E, 0xF, 0xF, true));
    v = max(v, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x141, 0xF, 0xF, true));
    v = max(v, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x140, 0xF, 0xF, true));
    const uint32_t a = (uint32_t)__builtin_amdgcn_readlane((int)v, 0), b = (uint32_t)__builtin_amdgcn_readlane((int)v, 16);
    const uint32_t c = (uint32_t)__builtin_amdgcn_readlane((int)v, 32), d = (uint32_t)__builtin_amdgcn_readlane((int)v, 48);
    return max(max(a, b), max(c, d));
}

// One wavefront reduces kTopKSegment packed values to their top_k largest, sorted descending.  Every lane
// sorts its kTopKPerLane values in registers; then, top_k times, the wavefront takes the largest of the 64
// list heads (high words first, then the low words of the lanes that hold that high word) and the winning
// lane drops its head.  Entries past `count` read as 0, which is also the "no candidate" value.
__device__ __forceinline__ void topk_reduce_segment(const unsigned long long* __restrict__ in, int64_t count, int top_k,
                                                    unsigned long long* __restrict__ out, int64_t segment, int lane) {
    constexpr int V = kTopKPerLane;
    const int64_t begin = segment * kTopKSegment;
    if (begin >= count) return;  // whole wavefronts
    unsigned long long v[V];
#pragma unroll
    for (int j = 0; j < V; j++) {
        const int64_t i = begin + j * kWave + lane;
        v[j] = i < count ? in[i] : 0ull;
    }
    // bitonic network over the lane's own values, fully unrolled: descending order
#pragma unroll
    for (int width = 2; width <= V; width <<= 1) {
#pragma unroll
        for (int stride = width >> 1; stride > 0; stride >>= 1) {
#pragma unroll
            for (int i = 0; i < V; i++) {
                const int j = i ^ stride;
                if (j > i) {
                    const bool descending = (i & width) == 0;
                    const unsigned long long a = v[i], b = v[j];
                    const bool swap = descending ? a < b : a > b;
                    v[i] = swap ? b : a;
                    v[j] = swap ? a : b;
                }
            }
        }
    }
    unsigned long long mine = 0;
    for (int it = 0; it < top_k; it++) {
        const uint32_t hi = (uint32_t)(v[0] >> 32), lo = (uint32_t)v[0];
        const uint32_t best_hi = wave_max_u32(hi);
        const uint32_t best_lo = wave_max_u32(hi == best_hi ? lo : 0u);
        const unsigned long long best = ((unsigned long long)best_hi << 32) | best_lo;
        if (best == 0) break;  // nothing but "no candidate" left; uniform over the wavefront
        const unsigned long long holders = __ballot(v[0] == best);
        if (lane == __ffsll((long long)holders) - 1) {  // equal values: one lane at a time gives its copy
#pragma unroll
            for (int j = 0; j + 1 < V; j++) v[j] = v[j + 1];
            v[V - 1] = 0;
        }
        if (lane == it) mine = best;
    }
    if (lane < top_k) out[segment * top_k + lane] = mine;
}

// A round of the segment-by-segment reduction.  With `gate` set the round only runs when the candidate list of
// the threshold path below has overflowed (*gate > kTopKCandidates); otherwise it leaves at once.
__global__ __launch_bounds__(256) void packed_topk_kernel(const unsigned long long* __restrict__ in, int64_t count, int top_k,
                                                          unsigned long long* __restrict__ out, const uint32_t* gate) {
    if (gate && *gate <= (uint32_t)kTopKCandidates) return;
    topk_reduce_segment(in, count, top_k, out, (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6), threadIdx.x & (kWave - 1));
}

// Threshold path, for inputs of many segments.  The top_k-th largest of the segment maxima is a value T that
// at least top_k entries reach (the maxima themselves), so the top_k largest entries all lie among the entries
// >= T; for scores that are not arranged by rank that set is a little over top_k entries, and one workgroup
// orders it by counting.  Three launches: maxima, filter, finish.  When more than kTopKCandidates entries
// reach T (long runs of equal scores, an input sorted by score) the finish launch runs the first round of the
// segment-by-segment reduction instead and the gated rounds after it complete the answer.
// A wavefront of these two kernels takes a piece of 64 * V entries: V is the largest of 16, 4, 1 that leaves at
// least top_k pieces.
template <int V>
__global__ __launch_bounds__(256) void topk_segment_max_kernel(const unsigned long long* __restrict__ in, int64_t count,
                                                               unsigned long long* __restrict__ segmax, uint32_t* counter) {
    const int lane = threadIdx.x & (kWave - 1);
    const int64_t segment = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    const int64_t begin = segment * (kWave * V);
    if (blockIdx.x == 0 && threadIdx.x == 0) *counter = 0;
    if (begin >= count) return;
    unsigned long long m = 0;
#pragma unroll
    for (int j = 0; j < V; j++) {
        const int64_t i = begin + j * kWave + lane;
        const unsigned long long v = i < count ? in[i] : 0ull;
        m = v > m ? v : m;
    }
    const uint32_t hi = (uint32_t)(m >> 32), lo = (uint32_t)m;
    const uint32_t best_hi = wave_max_u32(hi);
    const uint32_t best_lo = wave_max_u32(hi == best_hi ? lo : 0u);
    if (lane == 0) segmax[segment] = ((unsigned long long)best_hi << 32) | best_lo;
}

// The largest t, a multiple of 2^kTopKThresholdShift, that at least top_k of the high words `key` (SV a lane, zero
// where there is none) reach: built bit by bit from the top, every count one ballot.
constexpr int kTopKThresholdShift = 8;

template <int SV>
__device__ __forceinline__ uint32_t topk_threshold_key(const uint32_t (&key)[SV], int top_k) {
    uint32_t t = 0;
    for (int bit = 31; bit >= kTopKThresholdShift; bit--) {
        const uint32_t trial = t | (1u << bit);
        int reach = 0;
#pragma unroll
        for (int j = 0; j < SV; j++) reach += __popcll(__ballot(key[j] >= trial));
        if (reach >= top_k) t = trial;
    }
    return t;
}

template <int SV>
__device__ __forceinline__ uint32_t topk_threshold(const unsigned long long* __restrict__ segmax, int segments, int top_k,
                                                   int lane) {
    uint32_t key[SV];
#pragma unroll
    for (int j = 0; j < SV; j++) key[j] = j * kWave + lane < segments ? (uint32_t)(segmax[j * kWave + lane] >> 32) : 0u;
    return topk_threshold_key<SV>(key, top_k);
}

template <int V>
__global__ __launch_bounds__(256) void topk_filter_kernel(const unsigned long long* __restrict__ in, int64_t count, int top_k,
                                                          const unsigned long long* __restrict__ segmax, int segments,
                                                          uint32_t* counter, unsigned long long* __restrict__ cand) {
    const int lane = threadIdx.x & (kWave - 1);
    const int64_t segment = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    const int64_t begin = segment * (kWave * V);
    if (begin >= count) return;
    unsigned long long v[V];
#pragma unroll
    for (int j = 0; j < V; j++) {
        const int64_t i = begin + j * kWave + lane;
        v[j] = i < count ? in[i] : 0ull;
    }
    // T: at least top_k segment maxima have a high word (the score) >= T's, so at least top_k entries reach T
    // and the top_k largest are among them; every wavefront works T out for itself from the same list
    const uint32_t t_key = segments <= 4 * kWave ? topk_threshold<4>(segmax, segments, top_k, lane)
                                                 : topk_threshold<kTopKThresholdSegments / kWave>(segmax, segments, top_k, lane);
    const unsigned long long t = (unsigned long long)t_key << 32;
    unsigned long long mask[V];
    int total = 0;
#pragma unroll
    for (int j = 0; j < V; j++) {
        mask[j] = __ballot(v[j] >= t && v[j] != 0);
        total += __popcll(mask[j]);
    }
    if (total == 0) return;  // uniform over the wavefront
    uint32_t base = 0;
    if (lane == 0) base = atomicAdd(counter, (uint32_t)total);
    base = (uint32_t)__builtin_amdgcn_readfirstlane((int)base);
    const unsigned long long below = (1ull << lane) - 1;
#pragma unroll
    for (int j = 0; j < V; j++) {
        const uint32_t pos = base + (uint32_t)__popcll(mask[j] & below);
        if (((mask[j] >> lane) & 1) && pos < (uint32_t)kTopKCandidates) cand[pos] = v[j];
        base += (uint32_t)__popcll(mask[j]);
    }
}

// The candidates are distinct unless the input repeats a value, so an entry's place in the output is the number
// of candidates above it (equal values take consecutive places in list order).
__global__ __launch_bounds__(256) void topk_finish_kernel(const unsigned long long* __restrict__ in, int64_t count, int top_k,
                                                          const uint32_t* counter, const unsigned long long* __restrict__ cand,
                                                          unsigned long long* __restrict__ out,
                                                          unsigned long long* __restrict__ round_out) {
    const uint32_t n = *counter;
    if (n > (uint32_t)kTopKCandidates) {
        topk_reduce_segment(in, count, top_k, round_out, (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6),
                            threadIdx.x & (kWave - 1));
        return;
    }
    if (blockIdx.x != 0) return;
    constexpr int PER = kTopKCandidates / 256;
    __shared__ unsigned long long c[kTopKCandidates];
    unsigned long long mine[PER];
    int rank[PER];
#pragma unroll
    for (int i = 0; i < PER; i++) {
        const uint32_t idx = threadIdx.x + 256u * i;
        mine[i] = idx < n ? cand[idx] : 0ull;
        c[idx] = mine[i];
        rank[i] = 0;
    }
    __syncthreads();
    for (uint32_t o = 0; o < n; o++) {
        const unsigned long long other = c[o];
#pragma unroll
        for (int i = 0; i < PER; i++) {
            const uint32_t idx = threadIdx.x + 256u * i;
            rank[i] += (other > mine[i] || (other == mine[i] && o < idx)) ? 1 : 0;
        }
    }
#pragma unroll
    for (int i = 0; i < PER; i++) {
        const uint32_t idx = threadIdx.x + 256u * i;
        if (idx < n && rank[i] < top_k) out[rank[i]] = mine[i];
    }
    if (threadIdx.x >= n && threadIdx.x < (uint32_t)top_k) out[threadIdx.x] = 0ull;  // fewer candidates than top_k
}

static int64_t topk_segments(int64_t count) { return (count + kTopKSegment - 1) / kTopKSegment; }

// Entries a lane takes on the threshold path, 0 when the input goes segment by segment: the path needs at least
// top_k maxima and a wavefront keeps the whole list of maxima in registers.
static int topk_threshold_per_lane(int64_t count, int top_k) {
    if (count <= kTopKSegment) return 0;
    for (int v : {16, 4, 1}) {
        const int64_t pieces = (count + kWave * v - 1) / (kWave * v);
        if (pieces >= top_k && pieces <= kTopKThresholdSegments) return v;
    }
    return 0;
}

constexpr int kTopKHeader = 2;  // scratch[0]: candidate counter (its low word)

size_t packed_topk_scratch_entries(int64_t count, int top_k) {
    if (count <= kTopKSegment) return 0;
    // first round's output, then the second round's beside it (every later round is smaller)
    const int64_t c1 = topk_segments(count) * top_k;
    const int64_t c2 = c1 > kTopKSegment ? topk_segments(c1) * top_k : 0;
    int64_t total = c1 + c2;
    if (topk_threshold_per_lane(count, top_k)) total += kTopKHeader + kTopKThresholdSegments + kTopKCandidates;
    return (size_t)total;
}

template <int V>
static void topk_threshold_launch(const unsigned long long* in, int64_t count, int top_k, unsigned long long* segmax,
                                  uint32_t* counter, unsigned long long* cand, hipStream_t stream) {
    const int64_t pieces = (count + kWave * V - 1) / (kWave * V);
    const dim3 grid((unsigned)((pieces + 3) / 4));
    hipLaunchKernelGGL(topk_segment_max_kernel<V>, grid, dim3(256), 0, stream, in, count, segmax, counter);
    hipLaunchKernelGGL(topk_filter_kernel<V>, grid, dim3(256), 0, stream, in, count, top_k, segmax, (int)pieces, counter, cand);
}

hipError_t packed_topk_launch(const unsigned long long* in, int64_t count, int top_k, unsigned long long* out,
                              unsigned long long* scratch, hipStream_t stream) {
    if (top_k <= 0 || top_k > kTopKMax || count <= 0) return hipErrorInvalidValue;
    const int64_t first = topk_segments(count);
    const int64_t c1 = first * top_k;
    unsigned long long* bufs[2] = {scratch, scratch + c1};
    const uint32_t* gate = nullptr;
    int which = 0;
    const unsigned long long* src = in;
    int64_t n = count;
    if (const int per_lane = topk_threshold_per_lane(count, top_k)) {
        const int64_t c2 = c1 > kTopKSegment ? topk_segments(c1) * top_k : 0;
        unsigned long long* extra = scratch + c1 + c2;
        uint32_t* counter = reinterpret_cast<uint32_t*>(extra);
        unsigned long long* segmax = extra + kTopKHeader;
        unsigned long long* cand = segmax + kTopKThresholdSegments;
        if (per_lane == 16) topk_threshold_launch<16>(in, count, top_k, segmax, counter, cand, stream);
        else if (per_lane == 4) topk_threshold_launch<4>(in, count, top_k, segmax, counter, cand, stream);
        else topk_threshold_launch<1>(in, count, top_k, segmax, counter, cand, stream);
        hipLaunchKernelGGL(topk_finish_kernel, dim3((unsigned)((first + 3) / 4)), dim3(256), 0, stream, in, count, top_k, counter,
                           cand, out, bufs[0]);
        hipError_t rc = hipGetLastError();
        if (rc != hipSuccess) return rc;
        gate = counter;
        src = bufs[0];
        n = c1;
        which = 1;
    }
    while (true) {
        const int64_t segments = topk_segments(n);
        unsigned long long* dst = segments == 1 ? out : bufs[which];
        hipLaunchKernelGGL(packed_topk_kernel, dim3((unsigned)((segments + 3) / 4)), dim3(256), 0, stream, src, n, top_k, dst,
                           gate);
        hipError_t rc = hipGetLastError();
        if (rc != hipSuccess || segments == 1) return rc;
        src = dst;
        n = segments * top_k;
        which ^= 1;
    }
}

// Temperature / top-p sampling over the packed top-k list (rocm_packed_topk_sample,
// go/engine/hip/kernels/sampling/topk.hipinc:86-191; score decode and softcap kernels/common/numeric.hipinc:95-110).
// The reference runs the whole thing on one thread and evaluates exp() of every candidate in each of its four
// passes; here each of up to 128 threads evaluates its candidate's weight once (tanh and exp in double are the
// cost), thread 0 adds them once in list order, as the reference does, so every sum rounds the same way, and the
// threads compare against that running sum side by side.  out[0] = 0 when nothing can be sampled.
constexpr int kSampleMax = 128;

__device__ __forceinline__ double sample_score(unsigned long long packed, double softcap) {
    const uint32_t key = (uint32_t)(packed >> 32);
    const double score = (double)__uint_as_float((key & 0x80000000u) ? key ^ 0x80000000u : ~key);
    return softcap > 0.0 ? tanh(score / softcap) * softcap : score;
}

__global__ __launch_bounds__(kSampleMax) void packed_topk_sample_kernel(const unsigned long long* __restrict__ in,
                                                                        int top_k, float raw_temperature, float raw_top_p,
                                                                        float softcap_f, double draw,
                                                                        unsigned long long* __restrict__ out) {
    __shared__ unsigned long long vals[kSampleMax];
    __shared__ double wts[kSampleMax];
    __shared__ double prefix[kSampleMax];
    __shared__ double total_s;
    __shared__ int bad, limit_s, kept_s, pick_s;
    const int t = threadIdx.x;
    vals[t] = t < top_k ? in[t] : 0ull;
    if (t == 0) {
        bad = 0;
        limit_s = top_k;
        kept_s = 0;
        pick_s = kSampleMax;
    }
    __syncthreads();
    int first_valid = top_k;  // the same scan on every thread: the branches below are uniform
    for (int i = 0; i < top_k; ++i)
        if (vals[i] != 0ull) {
            first_valid = i;
            break;
        }
    unsigned long long result = 0ull;
    bool sample = false;
    double temperature = 1.0, top_p = 1.0;
    if (first_valid < top_k) {
        if (raw_temperature <= 0.0f && raw_top_p <= 0.0f) {
            result = vals[first_valid];  // greedy
        } else {
            temperature = raw_temperature == 0.0f ? 1.0 : (double)raw_temperature;
            top_p = raw_top_p == 0.0f ? 1.0 : (double)raw_top_p;
            sample = temperature > 0.0 && top_p > 0.0 && top_p <= 1.0;
        }
    }
    if (!sample) {
        if (t == 0) out[0] = result;
        return;
    }
    const double softcap = (double)softcap_f;
    const double max_value = sample_score(vals[first_valid], softcap) / temperature;
    wts[t] = (t >= first_valid && t < top_k && vals[t] != 0ull)
                 ? exp(sample_score(vals[t], softcap) / temperature - max_value)
                 : 0.0;
    const bool valid = t >= first_valid && t < top_k && vals[t] != 0ull;
    if (valid && !isfinite(wts[t])) bad = 1;  // any non-finite weight: nothing is sampled
    __syncthreads();
    // The reference's four passes all add the same weights in the same order from 0.0: its total, its nucleus
    // cumulative, its selected total and its draw cumulative are entries of ONE running sum.  Thread 0 forms that
    // sum once; the comparisons against it are independent and every thread does its own.
    if (t == 0) {
        double run = 0.0;  // holes carry weight 0.0, and x + 0.0 is x: no branch in the chain of adds
#pragma unroll 8
        for (int i = 0; i < top_k; ++i) {
            run += wts[i];
            prefix[i] = run;
        }
        total_s = run;
    }
    __syncthreads();
    const double total = total_s;
    if (bad || !(total > 0.0) || !isfinite(total)) {
        if (t == 0) out[0] = 0ull;
        return;
    }
    if (top_p < 1.0 && valid && prefix[t] / total >= top_p) atomicMin(&limit_s, t + 1);
    __syncthreads();
    const int limit = limit_s;
    if (valid && t < limit) atomicMax(&kept_s, t);  // the last candidate inside the nucleus
    __syncthreads();
    const int kept = kept_s;
    const double selected_total = prefix[kept];
    if (!(selected_total > 0.0) || !isfinite(selected_total)) {
        if (t == 0) out[0] = 0ull;
        return;
    }
    if (draw < 0.0) draw = 0.0;
    if (draw >= 1.0) draw = 0x1.fffffffffffffp-1;  // the double below 1
    const double target = draw * selected_total;
    if (valid && t < limit && target <= prefix[t]) atomicMin(&pick_s, t);
    __syncthreads();
    if (t == 0) out[0] = vals[pick_s < kSampleMax ? pick_s : kept];
}

hipError_t packed_topk_sample_launch(const unsigned long long* in, int top_k, float temperature, float top_p, float softcap,
                                     double draw, unsigned long long* out, hipStream_t stream) {
    if (top_k <= 0 || top_k > kSampleMax) return hipErrorInvalidValue;
    hipLaunchKernelGGL(packed_topk_sample_kernel, dim3(1), dim3(kSampleMax), 0, stream, in, top_k, temperature, top_p, softcap,
                       draw, out);
    return hipGetLastError();
}

}  // namespace aq
