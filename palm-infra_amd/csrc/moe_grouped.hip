// Routed experts for many rows (a prompt), planned on the device: the (token, choice) pairs are grouped by expert, and two
// grouped products on the matrix cores run all experts' rows in one launch each.
//
//   plan      count the pairs of every expert; pad every expert's run of pairs to whole tiles of GT_TOKENS rows and lay the
//             runs one after the other; place every pair in its run in the order of the pairs (token, then choice), so that
//             nothing depends on the order in which threads arrive; the slots that pad a run hold -1
//   grouped   for every tile (its expert comes from the plan): mid = silu(G_e x) * (U_e x) for the tile's rows x, then
//             y = D_e mid.  The weights are the first operand of the matrix instruction, so that a lane ends with four
//             neighbouring features of one row; a wave owns 32 features x 64 rows and reads its fragments from memory itself
//             (a weight fragment feeds four products, a row fragment two or four)
//   combine   out[t] = sum_c weight[t, c] * y[place of pair (t, c)], in the order of c, 32-bit
#include "mfma.h"

constexpr int GT_TOKENS = 64;                     // rows of a tile
constexpr int GT_RUNS = GT_TOKENS / 16;           // runs of 16 rows: what one matrix instruction takes
constexpr int GT_WAVES = 4;
constexpr int GT_FEATURES = 32 * GT_WAVES;        // features of a block's tile
constexpr int PLAN_THREADS = 256;

__device__ inline bf16x8 grouped_row8(const bf16_t* row, int col, int dim) {
    // eight values of a row from column `col`; columns beyond `dim` are zero (dim is a multiple of eight); the read itself
    // is unconditional
    const bf16x8 v = load_bf16x8(row + min(col, dim - 8));
    return col < dim ? v : zero_bf16x8();
}

// One block per expert: counts[e] = pairs that chose e.
__global__ __launch_bounds__(PLAN_THREADS) void moe_count_kernel(const int* __restrict__ chosen, int n_pairs, int* __restrict__ counts) {
    __shared__ int part[PLAN_THREADS / WAVE];
    const int e = blockIdx.x;
    int mine = 0;
    for (int p = threadIdx.x; p < n_pairs; p += PLAN_THREADS) mine += chosen[p] == e;
#pragma unroll
    for (int off = WAVE / 2; off > 0; off >>= 1) mine += __shfl_xor(mine, off, WAVE);
    if (threadIdx.x % WAVE == 0) part[threadIdx.x / WAVE] = mine;
    __syncthreads();
    if (threadIdx.x == 0) {
        int total = 0;
        for (int w = 0; w < PLAN_THREADS / WAVE; ++w) total += part[w];
        counts[e] = total;
    }
}

// One block: starts[e] = first slot of expert e's run (runs padded to whole tiles), starts[experts] = slots in all;
// tile_expert[i] = the expert of tile i, -1 beyond the last tile.
__global__ __launch_bounds__(PLAN_THREADS) void moe_runs_kernel(const int* __restrict__ counts, int experts, int max_tiles,
                                                                int* __restrict__ starts, int* __restrict__ tile_expert) {
    if (threadIdx.x == 0) {
        int at = 0;
        for (int e = 0; e < experts; ++e) {
            starts[e] = at;
            at += (counts[e] + GT_TOKENS - 1) / GT_TOKENS * GT_TOKENS;
        }
        starts[experts] = at;
    }
    __syncthreads();
    for (int i = threadIdx.x; i < max_tiles; i += PLAN_THREADS) tile_expert[i] = -1;
    __syncthreads();
    for (int e = threadIdx.x; e < experts; e += PLAN_THREADS)
        for (int i = starts[e] / GT_TOKENS; i < starts[e + 1] / GT_TOKENS; ++i) tile_expert[i] = e;
}

// One block per expert: its pairs into its run, in the order of the pairs.  slot_pair[slot] = pair (or -1), pair_slot[pair] = slot.
__global__ __launch_bounds__(PLAN_THREADS) void moe_place_kernel(const int* __restrict__ chosen, int n_pairs, const int* __restrict__ starts,
                                                                 int* __restrict__ slot_pair, int* __restrict__ pair_slot) {
    __shared__ int wave_count[PLAN_THREADS / WAVE];
    __shared__ int base_s;
    const int e = blockIdx.x, lane = threadIdx.x % WAVE, wave = threadIdx.x / WAVE;
    if (threadIdx.x == 0) base_s = starts[e];
    __syncthreads();
    for (int p0 = 0; p0 < n_pairs; p0 += PLAN_THREADS) {
        const int p = p0 + threadIdx.x;
        const bool mine = p < n_pairs && chosen[p] == e;
        const unsigned long long votes = __ballot(mine);
        const int before = __popcll(votes & ((1ull << lane) - 1ull));
        if (lane == 0) wave_count[wave] = __popcll(votes);
        __syncthreads();
        int base = base_s;
        for (int w = 0; w < wave; ++w) base += wave_count[w];
        if (mine) {
            slot_pair[base + before] = p;
            pair_slot[p] = base + before;
        }
        __syncthreads();
        if (threadIdx.x == 0) {
            int total = 0;
            for (int w = 0; w < PLAN_THREADS / WAVE; ++w) total += wave_count[w];
            base_s += total;
        }
        __syncthreads();
    }
    for (int s = base_s + threadIdx.x; s < starts[e + 1]; s += PLAN_THREADS) slot_pair[s] = -1;
}

// grid (tiles, blocks of GT_FEATURES features).  a: the rows [*, k_dim]; row_of_slot: null (the rows lie in slot order) or
// slot -> pair, the pair's row being pair / top.  w: [experts, n_w_rows, k_dim]; FORM 1 (gated): n_w_rows = 2 n_features, an
// expert's gate rows first, and the result is silu(gate) * up; FORM 2: the product through the exact gelu; FORM 0: the product
// as it is.  out: bfloat16 [slots, n_features].
template <int FORM>
__global__ __launch_bounds__(GT_WAVES * WAVE) void moe_grouped_kernel(const bf16_t* __restrict__ a, const int* __restrict__ slot_pair, int top,
                                                                      const bf16_t* __restrict__ w, const int* __restrict__ tile_expert,
                                                                      int n_features, int k_dim, bf16_t* __restrict__ out) {
    constexpr bool GATED = FORM == 1;
    const int tile = blockIdx.x;
    const int e = tile_expert[tile];
    if (e < 0) return;
    const int lane = threadIdx.x % WAVE, wave = threadIdx.x / WAVE;
    const int r = lane % 16, g = lane / 16;
    const int f0 = blockIdx.y * GT_FEATURES + wave * 32;
    if (f0 >= n_features) return;
    const int slot0 = tile * GT_TOKENS;
    // the rows of the tile's runs of 16 slots, as the second operand: column r is a row of activations
    const bf16_t* ar[GT_RUNS];
#pragma unroll
    for (int tt = 0; tt < GT_RUNS; ++tt) {
        const int slot = slot0 + 16 * tt + r;
        const int pair = slot_pair ? slot_pair[slot] : slot;
        const int row = slot_pair ? max(pair, 0) / top : slot;          // a slot that pads the run reads row 0; nobody reads its result
        ar[tt] = a + (size_t)row * k_dim;
    }
    const size_t w_rows = GATED ? 2 * (size_t)n_features : (size_t)n_features;
    const bf16_t* wr[GATED ? 4 : 2];
#pragma unroll
    for (int ft = 0; ft < 2; ++ft) {
        const int f = min(f0 + 16 * ft + r, n_features - 1);
        wr[ft] = w + ((size_t)e * w_rows + f) * k_dim;
        if (GATED) wr[2 + ft] = w + ((size_t)e * w_rows + n_features + f) * k_dim;
    }
    f32x4 acc[GATED ? 4 : 2][GT_RUNS];
#pragma unroll
    for (int i = 0; i < (GATED ? 4 : 2); ++i)
#pragma unroll
        for (int tt = 0; tt < GT_RUNS; ++tt) acc[i][tt] = f32x4{0.f, 0.f, 0.f, 0.f};
    for (int k0 = 0; k0 < k_dim; k0 += 32) {
        const int col = k0 + 8 * g;
        bf16x8 af[GT_RUNS], wf[GATED ? 4 : 2];
#pragma unroll
        for (int tt = 0; tt < GT_RUNS; ++tt) af[tt] = grouped_row8(ar[tt], col, k_dim);
#pragma unroll
        for (int i = 0; i < (GATED ? 4 : 2); ++i) wf[i] = grouped_row8(wr[i], col, k_dim);
#pragma unroll
        for (int i = 0; i < (GATED ? 4 : 2); ++i)
#pragma unroll
            for (int tt = 0; tt < GT_RUNS; ++tt) acc[i][tt] = mfma_16x16x32(wf[i], af[tt], acc[i][tt]);
    }
    // lane (r, g) holds features f0 + 16 ft + 4 g + i of the row in slot slot0 + 16 tt + r
#pragma unroll
    for (int ft = 0; ft < 2; ++ft)
#pragma unroll
        for (int tt = 0; tt < GT_RUNS; ++tt) {
            const int f = f0 + 16 * ft + 4 * g;
            if (f >= n_features) continue;                              // n_features is a multiple of four
            float v[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                if (GATED) {
                    const float gt = acc[ft][tt][i];
                    v[i] = gt / (1.0f + expf(-gt)) * acc[2 + ft][tt][i];
                } else if (FORM == 2) {
                    const float z = acc[ft][tt][i];
                    v[i] = 0.5f * z * (1.0f + erff(z * 0.70710678118654752f));
                } else {
                    v[i] = acc[ft][tt][i];
                }
            }
            uint2 pk;
            pk.x = (uint32_t)f32_to_bf16(v[0]).bits | ((uint32_t)f32_to_bf16(v[1]).bits << 16);
            pk.y = (uint32_t)f32_to_bf16(v[2]).bits | ((uint32_t)f32_to_bf16(v[3]).bits << 16);
            *reinterpret_cast<uint2*>(out + (size_t)(slot0 + 16 * tt + r) * n_features + f) = pk;
        }
}

// One block per token.
__global__ void moe_combine_kernel(const bf16_t* __restrict__ y, const int* __restrict__ pair_slot, const float* __restrict__ weight, int top,
                                   int width, float* __restrict__ out) {
    const size_t t = blockIdx.x;
    for (int d = threadIdx.x; d < width; d += blockDim.x) {
        float total = 0.f;
        for (int c = 0; c < top; ++c) total = fmaf(weight[t * top + c], to_float(y[(size_t)pair_slot[t * top + c] * width + d]), total);
        out[t * width + d] = total;
    }
}

PALM_API int palm_moe_tile_tokens() { return GT_TOKENS; }

// chosen, weight [n, top]; h bfloat16 [n, width]; gate_up bfloat16 [experts, 2 ff, width] (form 1: [experts, ff, width], up rows
// alone, through the exact gelu); down bfloat16 [experts, width, ff].
// Room, with max_tiles = ceil(n top / tile) + experts and slots = max_tiles * tile: plan: (2 experts + 1 + max_tiles + slots
// + n top) ints; mid: slots * ff bfloat16; y: slots * width bfloat16.  out float32 [n, width].
PALM_API int palm_moe_grouped(hipStream_t stream, const void* h, const void* gate_up, const void* down, const int* chosen,
                              const float* weight, int n_tokens, int top, int experts, int width, int ff, int* plan, void* mid, void* y,
                              float* out, int form) {
    PALM_CHECK(form == 0 || form == 1, "moe_grouped: form %d is neither gated silu (0) nor plain gelu (1)", form);
    PALM_CHECK(n_tokens >= 0 && top > 0 && experts > 0 && width > 0 && ff > 0, "moe_grouped: n=%d top=%d experts=%d width=%d ff=%d", n_tokens,
               top, experts, width, ff);
    PALM_CHECK(width % 8 == 0 && ff % 8 == 0, "moe_grouped: width %d and inner size %d must be multiples of eight", width, ff);
    if (n_tokens == 0) return 0;
    const long long n_pairs = (long long)n_tokens * top;
    PALM_CHECK(n_pairs < (1ll << 30), "moe_grouped: %lld pairs are more than one launch takes", n_pairs);
    const int max_tiles = (int)((n_pairs + GT_TOKENS - 1) / GT_TOKENS) + experts;
    int* counts = plan;
    int* starts = counts + experts;
    int* tile_expert = starts + experts + 1;
    int* slot_pair = tile_expert + max_tiles;
    int* pair_slot = slot_pair + (size_t)max_tiles * GT_TOKENS;
    moe_count_kernel<<<experts, PLAN_THREADS, 0, stream>>>(chosen, (int)n_pairs, counts);
    moe_runs_kernel<<<1, PLAN_THREADS, 0, stream>>>(counts, experts, max_tiles, starts, tile_expert);
    moe_place_kernel<<<experts, PLAN_THREADS, 0, stream>>>(chosen, (int)n_pairs, starts, slot_pair, pair_slot);
    if (form == 0)
        moe_grouped_kernel<1><<<dim3(max_tiles, (ff + GT_FEATURES - 1) / GT_FEATURES), GT_WAVES * WAVE, 0, stream>>>(
            (const bf16_t*)h, slot_pair, top, (const bf16_t*)gate_up, tile_expert, ff, width, (bf16_t*)mid);
    else
        moe_grouped_kernel<2><<<dim3(max_tiles, (ff + GT_FEATURES - 1) / GT_FEATURES), GT_WAVES * WAVE, 0, stream>>>(
            (const bf16_t*)h, slot_pair, top, (const bf16_t*)gate_up, tile_expert, ff, width, (bf16_t*)mid);
    moe_grouped_kernel<0><<<dim3(max_tiles, (width + GT_FEATURES - 1) / GT_FEATURES), GT_WAVES * WAVE, 0, stream>>>(
        (const bf16_t*)mid, nullptr, top, (const bf16_t*)down, tile_expert, width, ff, (bf16_t*)y);
    moe_combine_kernel<<<n_tokens, 256, 0, stream>>>((const bf16_t*)y, pair_slot, weight, top, width, out);
    PALM_LAUNCHED();
    return 0;
}
