// Attention over latent cache rows on the matrix cores (bfloat16).  A row is [c ; kr] of r + dr numbers, shared by all
// heads; the queries arrive with the keys' projection folded in (csrc/latent.hip), so head h of token n scores
// q'[n, h] . row_j and sums the rows' c-parts.  All heads of a token meet the same rows: the (token, head) pairs of a
// request are the columns of one product.
//
// A workgroup of 8 waves takes 128 consecutive (token, head) pairs of one request, a wave 16 of them, and walks the keys
// in tiles of 32 that all waves share through LDS: the tile's rows as they lie, for S^T = K Q'^T
// (v_mfma_f32_16x16x32_bf16: lane l holds K[key l%16][8 numbers from 8*(l/16)] and Q'[the same numbers][pair l%16]; the
// result holds S^T[key 4*(l/16) + i][pair l%16], i = 0..3), and their c-parts transposed, for O^T = C^T P^T
// (the same instruction, a tile being one step of 32 keys: lane l holds C^T[number l%16][keys 4*(l/16) ..+3 of both
// halves of the tile], two 8-byte reads of the transposed tile, and P^T[those keys][pair l%16], which is what the first
// product left in the lane).  A lane therefore keeps one pair's
// column throughout: its maximum, its sum and its window are the lane's own.  Softmax in base 2, 32-bit.
// The next tile's rows are fetched into registers while the present one is multiplied.
//
// `splits` > 1: the tiles of a workgroup's keys are dealt to that many workgroups, whose shares (sums, maximum, sum of
// weights, 32-bit) a second kernel adds up in the order of the shares.
//
// Sizes: r a multiple of 16 up to 512, r + dr a multiple of 8; the class RT (r <= 16 RT) also bounds r + dr (rounded up
// to 32) by 32 (RT / 2 + 2).
#include "common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 lm_bf16x8;
typedef __attribute__((ext_vector_type(4))) float lm_f32x4;
typedef __attribute__((ext_vector_type(4))) uint32_t lm_u32x4;
typedef __attribute__((ext_vector_type(2))) uint32_t lm_u32x2;

#define LM_THREADS 512
#define LM_PAIRS 128  // (token, head) pairs of a workgroup
#define LM_KEYS 32    // keys of a tile
#define LM_CLD 40     // row stride of the transposed tile in elements: 32 keys + 8 of padding

struct LatentArgs {
    bf16* out;            // [N, H, r]
    const bf16* q;        // [N, H, dk]
    const bf16* pool;     // rows of dk numbers
    const int* tables;
    const int* table_rows;
    const int* cu_seqlens;
    const int* context_lens;
    float* ws;            // shares: [N * H, splits, r + 2]
    int table_width, heads, r, dk, dkp, block_size, window, splits;
    uint32_t page_magic;  // ceil(2^32 / block_size): key / block_size is the high word of key * page_magic (0: block_size is 1)
    float scale_log2;
};

template <int RT>
__global__ __launch_bounds__(LM_THREADS) void attend_latent_mfma_kernel(LatentArgs a) {
    constexpr int QT = RT / 2 + 2;          // steps of 32 numbers of a query
    constexpr int NIT = (LM_KEYS / 2 * QT * 4 + LM_THREADS - 1) / LM_THREADS;  // pairs of 16-byte pieces of a tile per thread
    extern __shared__ __attribute__((aligned(16))) uint16_t lm_lds[];
    const int seq = blockIdx.y, split = blockIdx.z;
    const int first = a.cu_seqlens[seq], count = a.cu_seqlens[seq + 1] - first, ctx = a.context_lens[seq];
    const int pairs = count * a.heads, p0 = blockIdx.x * LM_PAIRS;
    if (p0 >= pairs) return;
    const int tid = threadIdx.x, wave = tid / LLMS_WAVE, lane = tid % LLMS_WAVE;
    const int l16 = lane % 16, quad = lane / 16;
    const int kld = a.dkp + 8;
    uint16_t* ks = lm_lds;                       // [32][kld]
    uint16_t* ct = lm_lds + LM_KEYS * kld;       // [r][LM_CLD]
    const int* table = a.tables + (size_t)(a.table_rows ? a.table_rows[seq] : seq) * a.table_width;
    const int start = ctx - count;  // position of the request's first token of this step (< 0: a request without keys)

    // the workgroup's keys: from the first pair's window to the last pair's position
    const int tl_last = (min(pairs, p0 + LM_PAIRS) - 1) / a.heads;
    const int lo_block = a.window > 0 ? max(0, start + p0 / a.heads - a.window + 1) : 0;
    const int hi_block = start + tl_last;
    int t_begin = lo_block / LM_KEYS, t_end = hi_block >= 0 ? hi_block / LM_KEYS + 1 : 0;
    if (hi_block < 0) t_begin = 0;
    if (a.splits > 1) {
        const int per = (max(t_end - t_begin, 0) + a.splits - 1) / a.splits;
        t_begin = t_begin + split * per;
        t_end = min(t_end, t_begin + per);
    }

    // this lane's pair
    const int pair = p0 + wave * 16 + l16;
    const bool valid = pair < pairs;
    const int tl = valid ? pair / a.heads : 0, head = valid ? pair - tl * a.heads : 0;
    const int pos = valid ? start + tl : -1;
    const int lo = a.window > 0 ? max(0, pos - a.window + 1) : 0;
    // the wave's keys (uniform over the wave): a tile outside them is not multiplied
    const int w_first = min(pairs - 1, p0 + wave * 16), w_last = min(pairs - 1, p0 + wave * 16 + 15);
    const bool w_any = p0 + wave * 16 < pairs;
    const int w_lo = a.window > 0 ? max(0, start + w_first / a.heads - a.window + 1) : 0;
    const int w_hi = start + w_last / a.heads;
    // keys [w_from, w_seen] are seen by every pair of the wave (none when some of its 16 columns hold no pair)
    const bool w_full = p0 + wave * 16 + 15 < pairs;
    const int w_seen = w_full ? start + w_first / a.heads : -1;
    const int w_from = a.window > 0 ? max(0, w_hi - a.window + 1) : 0;

    const lm_u32x4 zero4 = {0, 0, 0, 0};
    lm_u32x4 qf[QT];
    {
        const bf16* qrow = a.q + ((size_t)(first + tl) * a.heads + head) * a.dk;
#pragma unroll
        for (int c = 0; c < QT; ++c) {
            const int k = 32 * c + 8 * quad;
            qf[c] = (valid && k < a.dk) ? *reinterpret_cast<const lm_u32x4*>(qrow + k) : zero4;
        }
    }
    lm_f32x4 o[RT];
#pragma unroll
    for (int t = 0; t < RT; ++t) o[t] = (lm_f32x4){0.f, 0.f, 0.f, 0.f};
    float m = -INFINITY, l = 0.f;
    const int rt = a.r / 16, qt = a.dkp / 32, cpk = a.dkp / 8;  // (pieces of 8 numbers per key, padding included)

    // A thread's items of a tile: two neighbouring keys' 16-byte pieces at the same place of their rows, so that the
    // transposed tile is written in whole words (a number of both keys).  Item id = (piece / 2, pair of keys, piece % 2):
    // the lanes of a wave hold all 16 pairs of keys for four pieces, and their stores into the transposed tile fall
    // into different banks.  Page ids are looked up a tile ahead of the rows they lead to, so that no tile waits for
    // two loads in a row.
    lm_u32x4 pf[NIT][2];
    int pg[NIT][2];
    auto page_of = [&](int key) { return a.page_magic ? (int)__umulhi((uint32_t)key, a.page_magic) : key; };
    auto lookup = [&](int tile) {
#pragma unroll
        for (int i = 0; i < NIT; ++i) {
            const int id = tid + i * LM_THREADS;
            const int key = tile * LM_KEYS + 2 * ((id >> 1) & 15);
#pragma unroll
            for (int k = 0; k < 2; ++k)
                pg[i][k] = (key + k >= lo_block && key + k <= hi_block) ? table[page_of(key + k)] : 0;
        }
    };
    auto fetch = [&](int tile) {
#pragma unroll
        for (int i = 0; i < NIT; ++i) {
            const int id = tid + i * LM_THREADS;
            const int piece = ((id >> 5) << 1) | (id & 1);  // (32 pieces per round of the workgroup's 512 threads)
            const int key = tile * LM_KEYS + 2 * ((id >> 1) & 15);
#pragma unroll
            for (int k = 0; k < 2; ++k) {
                const bool there = piece < cpk && key + k >= lo_block && key + k <= hi_block && piece * 8 < a.dk;
                lm_u32x4 v = zero4;
                if (there)  // (page * block_size + key % block_size, without a division)
                    v = *reinterpret_cast<const lm_u32x4*>(
                        a.pool + (size_t)((pg[i][k] - page_of(key + k)) * a.block_size + key + k) * a.dk + piece * 8);
                pf[i][k] = v;
            }
        }
    };
    auto stage = [&]() {
#pragma unroll
        for (int i = 0; i < NIT; ++i) {
            const int id = tid + i * LM_THREADS;
            const int piece = ((id >> 5) << 1) | (id & 1), key_in = 2 * ((id >> 1) & 15);
            if (piece >= cpk) continue;
            *reinterpret_cast<lm_u32x4*>(&ks[key_in * kld + piece * 8]) = pf[i][0];
            *reinterpret_cast<lm_u32x4*>(&ks[(key_in + 1) * kld + piece * 8]) = pf[i][1];
            if (piece * 8 < a.r) {
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const uint32_t k0 = pf[i][0][e], k1 = pf[i][1][e];
                    uint32_t* word = reinterpret_cast<uint32_t*>(&ct[(piece * 8 + 2 * e) * LM_CLD + key_in]);
                    word[0] = (k0 & 0xffffu) | (k1 << 16);
                    word[LM_CLD / 2] = (k0 >> 16) | (k1 & 0xffff0000u);
                }
            }
        }
    };

    if (t_begin < t_end) {
        lookup(t_begin);
        fetch(t_begin);
        if (t_begin + 1 < t_end) lookup(t_begin + 1);
        stage();
    }
    __syncthreads();
    for (int tile = t_begin; tile < t_end; ++tile) {
        if (tile + 1 < t_end) {
            fetch(tile + 1);
            if (tile + 2 < t_end) lookup(tile + 2);
        }
        const int key0 = tile * LM_KEYS;
        if (w_any && key0 <= w_hi && key0 + LM_KEYS > w_lo) {
            lm_f32x4 s[2];
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                s[h] = (lm_f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int c = 0; c < QT; ++c) {
                    if (c < qt) {
                        const lm_u32x4 kf = *reinterpret_cast<const lm_u32x4*>(&ks[(16 * h + l16) * kld + 32 * c + 8 * quad]);
                        s[h] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(lm_bf16x8, kf),
                                                                       __builtin_bit_cast(lm_bf16x8, qf[c]), s[h], 0, 0, 0);
                    }
                }
            }
            // A tile that every pair of the wave sees whole is not compared key by key (uniform over the wave).
            const bool whole = key0 + LM_KEYS - 1 <= w_seen && key0 >= w_from;
            float top = -INFINITY;
#pragma unroll
            for (int h = 0; h < 2; ++h)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int key = key0 + 16 * h + 4 * quad + i;
                    float v = s[h][i] * a.scale_log2;
                    if (!whole) v = (key <= pos && key >= lo) ? v : -INFINITY;
                    s[h][i] = v;
                    top = fmaxf(top, v);
                }
            top = fmaxf(top, __shfl_xor(top, 16, LLMS_WAVE));
            top = fmaxf(top, __shfl_xor(top, 32, LLMS_WAVE));
            // The weights are taken against a reference that follows the maximum only when some pair's maximum has
            // passed it by more than 2^8 (the quotient at the end does not depend on the reference): the sums are
            // rescaled in few tiles.
            const bool moved = __any(top > m + 8.f);
            const float m_new = moved ? fmaxf(m, top) : m;
            const bool some = m_new > -INFINITY;
            const float fix = (moved && some) ? __builtin_amdgcn_exp2f(m - m_new) : 1.f;
            // the tile's 32 keys as one step of the 32-deep instruction: a lane's 8 keys are the 4 it holds of each
            // half of the tile (the order of keys within a step is free as long as both operands agree)
            lm_u32x4 pw;
            float add = 0.f;
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                float p[4];
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    p[i] = some ? __builtin_amdgcn_exp2f(s[h][i] - m_new) : 0.f;
                    add += p[i];
                }
                pw[2 * h] = pack_bf16x2(p[0], p[1]);
                pw[2 * h + 1] = pack_bf16x2(p[2], p[3]);
            }
            l = l * fix + add;
            m = m_new;
            if (moved) {
#pragma unroll
                for (int t = 0; t < RT; ++t)
                    if (t < rt) o[t] = o[t] * fix;
            }
#pragma unroll
            for (int t = 0; t < RT; ++t) {
                if (t < rt) {
                    const uint16_t* crow = &ct[(16 * t + l16) * LM_CLD + 4 * quad];
                    const lm_u32x2 c0 = *reinterpret_cast<const lm_u32x2*>(crow), c1 = *reinterpret_cast<const lm_u32x2*>(crow + 16);
                    const lm_u32x4 cf = {c0[0], c0[1], c1[0], c1[1]};
                    o[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(lm_bf16x8, cf),
                                                                   __builtin_bit_cast(lm_bf16x8, pw), o[t], 0, 0, 0);
                }
            }
        }
        __syncthreads();
        if (tile + 1 < t_end) stage();
        __syncthreads();
    }
    l += __shfl_xor(l, 16, LLMS_WAVE);
    l += __shfl_xor(l, 32, LLMS_WAVE);
    if (!valid) return;
    const size_t row = (size_t)(first + tl) * a.heads + head;
    if (a.splits > 1) {
        float* share = a.ws + (row * a.splits + split) * (a.r + 2);
#pragma unroll
        for (int t = 0; t < RT; ++t)
            if (t < rt) *reinterpret_cast<lm_f32x4*>(share + 16 * t + 4 * quad) = o[t];
        if (quad == 0) {
            share[a.r] = m;
            share[a.r + 1] = l;
        }
        return;
    }
    const float inv = l > 0.f ? 1.f / l : 0.f;
    bf16* orow = a.out + row * a.r;
#pragma unroll
    for (int t = 0; t < RT; ++t)
        if (t < rt)
            *reinterpret_cast<lm_u32x2*>(orow + 16 * t + 4 * quad) =
                (lm_u32x2){pack_bf16x2(o[t][0] * inv, o[t][1] * inv), pack_bf16x2(o[t][2] * inv, o[t][3] * inv)};
}

// grid: (token, head) pairs; adds the shares up in their order.  Every thread reads the shares' maxima and sums at
// once (all loads asked for before the first is used), then its numbers of every share.
#define LM_MAX_SPLITS 16
__global__ __launch_bounds__(256) void latent_merge_kernel(bf16* __restrict__ out, const float* __restrict__ ws, int r, int splits) {
    const size_t row = blockIdx.x;
    const float* shares = ws + row * splits * (r + 2);
    float mz[LM_MAX_SPLITS], lz[LM_MAX_SPLITS];
#pragma unroll
    for (int z = 0; z < LM_MAX_SPLITS; ++z) {
        mz[z] = z < splits ? shares[(size_t)z * (r + 2) + r] : -INFINITY;
        lz[z] = z < splits ? shares[(size_t)z * (r + 2) + r + 1] : 0.f;
    }
    float top = -INFINITY;
#pragma unroll
    for (int z = 0; z < LM_MAX_SPLITS; ++z) top = fmaxf(top, mz[z]);
    float total = 0.f;
#pragma unroll
    for (int z = 0; z < LM_MAX_SPLITS; ++z) {
        mz[z] = mz[z] > -INFINITY ? __builtin_amdgcn_exp2f(mz[z] - top) : 0.f;  // (from here on: the share's factor)
        total += lz[z] * mz[z];
    }
    const float inv = total > 0.f ? 1.f / total : 0.f;
    for (int c = threadIdx.x; c < r; c += 256) {
        float part[LM_MAX_SPLITS];
#pragma unroll
        for (int z = 0; z < LM_MAX_SPLITS; ++z) part[z] = z < splits ? shares[(size_t)z * (r + 2) + c] : 0.f;
        float v = 0.f;
#pragma unroll
        for (int z = 0; z < LM_MAX_SPLITS; ++z) v += mz[z] > 0.f ? part[z] * mz[z] : 0.f;
        out[row * r + c] = from_f32<bf16>(v * inv);
    }
}

template <int RT>
static int launch_latent(const LatentArgs& a, dim3 grid, size_t lds, hipStream_t stream) {
    auto kernel = attend_latent_mfma_kernel<RT>;
    if (lds > 48 * 1024)
        LLMS_HIP_CHECK(hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    kernel<<<grid, LM_THREADS, lds, stream>>>(a);
    return LLMS_OK;
}

extern "C" {

// The size class (8, 16 or 32) that takes r and r + dr, or 0.
int llms_attend_latent_mfma_class(int r, int dk) {
    if (r <= 0 || r % 16 != 0 || dk < r || dk % 8 != 0) return 0;
    const int dkp = (dk + 31) / 32 * 32;
    for (int rt = 8; rt <= 32; rt *= 2)
        if (r <= 16 * rt && dkp <= 32 * (rt / 2 + 2)) return rt;
    return 0;
}

// requests [0, n_seqs) of a step; `max_pairs`: most (token, head) pairs of one request; ws: float [n_rows * heads * splits * (r + 2)]
int llms_attend_latent_mfma(void* out, const void* q, const void* pool, const int* tables, int table_width,
                            const int* table_rows, const int* cu_seqlens, const int* context_lens, float* ws, int n_seqs,
                            int n_rows, int max_count, int heads, int r, int dr, int block_size, int window, float scale,
                            int splits, hipStream_t stream) {
    LLMS_REQUIRE(n_seqs > 0 && n_rows > 0 && max_count > 0 && heads > 0 && block_size > 0 && table_width > 0,
                 "attend_latent_mfma: sizes must be positive");
    const int dk = r + dr, rt = llms_attend_latent_mfma_class(r, dk);
    LLMS_REQUIRE(rt != 0, "attend_latent_mfma: r a multiple of 16 up to 512, r + dr a multiple of 8 within the class");
    LLMS_REQUIRE(((uintptr_t)q % 16) == 0 && ((uintptr_t)pool % 16) == 0 && ((uintptr_t)out % 8) == 0,
                 "attend_latent_mfma: operands must be 16-byte aligned");
    LLMS_REQUIRE(splits >= 1 && splits <= LM_MAX_SPLITS && (splits == 1 || ws), "attend_latent_mfma: 1 to 16 shares, with their workspace");
    LatentArgs a;
    a.out = (bf16*)out, a.q = (const bf16*)q, a.pool = (const bf16*)pool, a.tables = tables, a.table_rows = table_rows;
    a.cu_seqlens = cu_seqlens, a.context_lens = context_lens, a.ws = ws;
    a.table_width = table_width, a.heads = heads, a.r = r, a.dk = dk, a.dkp = (dk + 31) / 32 * 32;
    a.block_size = block_size, a.window = window, a.splits = splits;
    a.scale_log2 = scale * 1.4426950408889634f;
    a.page_magic = block_size == 1 ? 0u : (uint32_t)(((1ull << 32) + block_size - 1) / block_size);
    const long long blocks = ((long long)max_count * heads + LM_PAIRS - 1) / LM_PAIRS;
    LLMS_REQUIRE(blocks < (1ll << 31) && n_seqs <= 65535, "attend_latent_mfma: too many workgroups for one launch");
    dim3 grid((unsigned)blocks, n_seqs, splits);
    const size_t lds = ((size_t)LM_KEYS * (a.dkp + 8) + (size_t)r * LM_CLD) * sizeof(uint16_t);
    int status = rt == 8 ? launch_latent<8>(a, grid, lds, stream)
                 : rt == 16 ? launch_latent<16>(a, grid, lds, stream)
                            : launch_latent<32>(a, grid, lds, stream);
    if (status != LLMS_OK) return status;
    if (splits > 1) latent_merge_kernel<<<(unsigned)((size_t)n_rows * heads), 256, 0, stream>>>((bf16*)out, ws, r, splits);
    LLMS_LAUNCH_CHECK();
}

}  // extern "C"
