// A decode step's norm, QKV projection and attention over the cache as one kernel, for steps
// in which every request brings one token (at most 16 of them) and heads of up to 64.
//
// A decode step of few tokens is a chain of small kernels, each of which costs its boundary and a
// first trip to memory whatever its work. The folded norm + QKV product and the split attention
// were two links of that chain, with the queries written and read back between them. Here a
// workgroup does both for (head, role, group of tokens): it normalises its tokens' rows of the
// residual stream itself (the reference's layernorm, src/core/transformer.cpp:77-106), projects
// what its role needs of its head from the fused QKV matrix (:2657-2673, bias :1263-1273) and goes
// straight on to its share of the attention (:2162-2453):
//
//   role z < S   the head's query of each token, then keys [k_z, k_{z+1}) of the token's cached
//                keys (its own position left out), as attention_decode does: a running maximum,
//                sum and weighted values a lane group, merged over groups and waves in a fixed
//                order, left as split z of the (token, head) pair;
//   role S       query and key: the key goes to the token's slot of the pages (:2875-2890), and the
//                score of the token's own key, with a sum of 1, is the maximum and sum of split S;
//   role S + 1   the value: to the token's slot, and as the weighted values of split S.
//
// So the token's own key and value never travel through memory inside the step, and the S + 1
// splits are merged by whoever reads them (the output projection cut over its inner dimension,
// liyab_gemm_att_parts). The keys' loads are asked for before the query's products, which they do
// not depend on. Queries, keys and values are rounded to bfloat16 where the unfused kernels
// round them (what the pages hold is what every later step reads). Statistics, scores,
// exponentials and sums are 32-bit.
#include "common.h"

namespace liyab {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float floatx4;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;

namespace decode_qkv {

constexpr int FW = 8;        // waves a workgroup
constexpr int MAX_TG = 8;    // tokens a workgroup (a wave normalises one row)
constexpr int AU = 4;        // keys a lane group asks for together

union Frag {
    u32x4 u;
    bf16x8 v;
};

struct Args {
    const float* planes;  // the residual stream's rows [M][K], a sum of n_planes planes
    int n_planes;
    int64_t plane_stride;
    const float* ln_weight;  // [K] or null
    const float* ln_bias;    // [K] or null
    float eps;
    const bf16_t* w;    // [3 * n_head * hd][K]: queries, keys, values
    const float* bias;  // [3 * n_head * hd] or null
    bf16_t* kc;         // [pages][n_head][page_size][hd]
    bf16_t* vc;
    int num_pages, page_size, page_shift;
    const int* block_tables;  // [M][max_blocks]: row m is token m's request
    int max_blocks;
    const int* tok_pos;  // [M]
    const int* slots;    // [M]: page * page_size + offset of each token's own position
    int M, K, n_head, hd;
    float scale;
    int window;
    int S;          // splits of the cached keys
    int TG;         // tokens a workgroup
    int wpt_shift;  // log2 of the waves that share a token's keys
    float* partials;  // [M][n_head][S + 1][hd + 4]
};

struct Partial {
    float m, l;
    float acc[8];
};

__device__ __forceinline__ void unpack8(const u32x4& v, float* f) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        f[2 * i] = __uint_as_float(v[i] << 16);
        f[2 * i + 1] = __uint_as_float(v[i] & 0xffff0000u);
    }
}

// a <- merge(a, other): both rescaled to the larger maximum; a comes first
__device__ __forceinline__ void merge_partial(Partial& a, float mo, float lo, const float* acco) {
    const float M = fmaxf(a.m, mo);
    const float wa = a.m == -INFINITY ? 0.0f : __expf(a.m - M);
    const float wb = mo == -INFINITY ? 0.0f : __expf(mo - M);
    a.l = wa * a.l + wb * lo;
#pragma unroll
    for (int e = 0; e < 8; ++e) a.acc[e] = wa * a.acc[e] + wb * acco[e];
    a.m = M;
}

template <int MAXV, int NT>  // a row of K in MAXV pieces of 4 floats a lane; heads of 16 * NT
__global__ void __launch_bounds__(64 * FW)
attention_decode_qkv_kernel(Args a) {
    constexpr int LPK = NT == 1 ? 2 : (NT == 2 ? 4 : 8);  // lanes that share a key (8 dimensions each)
    constexpr int KPP = 64 / LPK;                          // keys a wave takes a pass
    constexpr int HDP = 16 * NT;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    const int K = a.K, hd = a.hd, ldx = K + 8;
    const int TG = a.TG;
    bf16_t* xs = reinterpret_cast<bf16_t*>(smem);  // [TG][K + 8]: the normalised rows
    size_t at = ((static_cast<size_t>(TG) * ldx * 2 + 15) / 16) * 16;
    float* red = reinterpret_cast<float*>(smem + at);  // [waves][NT][256]: the waves' sums of a projection
    at += static_cast<size_t>(FW) * NT * 256 * sizeof(float);
    float* qs = reinterpret_cast<float*>(smem + at);  // [MAX_TG][HDP]: the first projection (query, or value)
    at += MAX_TG * HDP * sizeof(float);
    float* ks = reinterpret_cast<float*>(smem + at);  // [MAX_TG][HDP]: the second (key)
    at += MAX_TG * HDP * sizeof(float);
    float* wsum = reinterpret_cast<float*>(smem + at);  // [waves][LPK][10]: the waves' attention sums
    at += FW * LPK * 10 * sizeof(float);
    int* sbt = reinterpret_cast<int*>(smem + at);  // [TG][max_blocks]: the tokens' page ids

    const int tid = threadIdx.x, lane = tid % 64, wave = tid / 64;
    const int i = lane % 16, g = lane / 16;
    const int h = blockIdx.x, role = blockIdx.y;
    const int m0 = blockIdx.z * TG, nt = min(TG, a.M - m0);
    const int S = a.S, q_dim = a.n_head * hd;
    const u32x4 zero = {0, 0, 0, 0};

    // 8 consecutive k of a row; past the end it is the last piece, read and dropped
    auto piece = [&](const bf16_t* row, int k) {
        const u32x4 v = *reinterpret_cast<const u32x4*>(row + min(k, K - 8));
        return k < K ? v : zero;
    };
    // a trip of a wave is two units of 64 k; this lane's 8 start at 8 g
    auto load_w = [&](int row0, int u0, Frag (&f)[2][NT][2]) {
#pragma unroll
        for (int p = 0; p < 2; ++p) {
            const int k = (u0 + p) * 64 + g * 8;
#pragma unroll
            for (int t = 0; t < NT; ++t) {
                const bf16_t* wrow = a.w + static_cast<int64_t>(row0 + 16 * t + i) * K;
                f[p][t][0].u = piece(wrow, k);
                f[p][t][1].u = piece(wrow, k + 32);
            }
        }
    };
    // rows of the fused matrix this role projects first: its head's query, or (role S + 1) value
    const int row_first = (role == S + 1 ? 2 * q_dim : 0) + h * hd;
    Frag wc[2][NT][2];

    // -- the tokens' page ids (key splits only), brought into the caches' pages ----------------
    if (role < S) {
        const int n_ids = TG * a.max_blocks;
        for (int idx = tid; idx < n_ids; idx += 64 * FW) {
            const int m = idx / a.max_blocks, b = idx - m * a.max_blocks;
            const int id = a.block_tables[static_cast<int64_t>(m0 + min(m, nt - 1)) * a.max_blocks + b];
            sbt[idx] = min(max(id, 0), a.num_pages - 1);
        }
    }

    // -- the norm: a wave a row, the row in registers (gemm_skinny_ln's, the same bits) ---------
    {
        const int nv = K / 4;
        const floatx4 fzero = {0.0f, 0.0f, 0.0f, 0.0f}, fone = {1.0f, 1.0f, 1.0f, 1.0f};
        const int m = min(wave, nt - 1);  // a wave past the last row works on the last row and keeps nothing
        const bool keep = wave < nt;
        const float* row0 = a.planes + static_cast<int64_t>(m0 + m) * K;
        floatx4 v[MAXV], gw[MAXV], gb[MAXV];
#pragma unroll
        for (int j = 0; j < MAXV; ++j) {
            const int p = min(lane + kWave * j, nv - 1);  // past the row: its last piece again, unused
            v[j] = reinterpret_cast<const floatx4*>(row0)[p];
            gw[j] = a.ln_weight != nullptr ? reinterpret_cast<const floatx4*>(a.ln_weight)[p] : fone;
            gb[j] = a.ln_bias != nullptr ? reinterpret_cast<const floatx4*>(a.ln_bias)[p] : fzero;
        }
        bool first = true;
        for (int q0 = 1; q0 < a.n_planes || first; ++q0) {
            floatx4 plane[MAXV];
            const float* row = row0 + min(q0, a.n_planes - 1) * a.plane_stride;  // a plane past the last: the last again, dropped
#pragma unroll
            for (int j = 0; j < MAXV; ++j) plane[j] = reinterpret_cast<const floatx4*>(row)[min(lane + kWave * j, nv - 1)];
            if (first) {
                // the wave's share of the weights right behind the row's first loads: counted in order,
                // a wait for the row does not wait for the weights, which come from further away
                load_w(row_first, wave * 2, wc);
                __builtin_amdgcn_sched_barrier(0);  // keep the loads in this order
                first = false;
            }
#pragma unroll
            for (int j = 0; j < MAXV; ++j)
                if (q0 < a.n_planes) v[j] += plane[j];
        }
        float s = 0.0f;
#pragma unroll
        for (int j = 0; j < MAXV; ++j)
            if (lane + kWave * j < nv) s += (v[j][0] + v[j][1]) + (v[j][2] + v[j][3]);
        const float mean = wave_sum(s) / static_cast<float>(K);
        float ss = 0.0f;
#pragma unroll
        for (int j = 0; j < MAXV; ++j)
            if (lane + kWave * j < nv) {
                const floatx4 dev = v[j] - mean;
                ss += (dev[0] * dev[0] + dev[1] * dev[1]) + (dev[2] * dev[2] + dev[3] * dev[3]);
            }
        const float scale = 1.0f / sqrtf(wave_sum(ss) / static_cast<float>(K) + a.eps);
#pragma unroll
        for (int j = 0; j < MAXV; ++j)
            if (keep && lane + kWave * j < nv) {
                const floatx4 y = (v[j] - mean) * scale * gw[j] + gb[j];
                uint2 packed;
                packed.x = static_cast<uint32_t>(float_to_bf16(y[0])) | (static_cast<uint32_t>(float_to_bf16(y[1])) << 16);
                packed.y = static_cast<uint32_t>(float_to_bf16(y[2])) | (static_cast<uint32_t>(float_to_bf16(y[3])) << 16);
                *reinterpret_cast<uint2*>(xs + m * ldx + 4 * (lane + kWave * j)) = packed;
            }
    }
    lds_barrier();  // rows and page ids are in LDS; the weights may still be on their way

    // -- this wave's token and its share of the token's keys (key splits) -----------------------
    const int WPT = 1 << a.wpt_shift;
    const int mt = wave >> a.wpt_shift, sw = wave & (WPT - 1);
    const bool tok_valid = role < S && mt < nt;
    const int mc = min(mt, nt - 1), tok = m0 + mc;
    const int c = lane % LPK, kg = lane / LPK;
    const bool active = c * 8 < hd;
    const int col = active ? c * 8 : 0;  // lanes past the head dimension read column 0 against a zero query
    // (a position past the block table's reach would index the staged ids out of range)
    const int pos = static_cast<int>(min(static_cast<int64_t>(max(a.tok_pos[tok], 0)), static_cast<int64_t>(a.max_blocks) * a.page_size - 1));
    const int first_key = a.window > 0 ? max(0, pos - a.window + 1) : 0;
    const int n_keys = pos - first_key;  // the cached keys: the token's own is role S's
    const int zc = min(role, S - 1);
    const int k_begin = first_key + static_cast<int>(static_cast<int64_t>(n_keys) * zc / S);
    const int k_end = tok_valid ? first_key + static_cast<int>(static_cast<int64_t>(n_keys) * (zc + 1) / S) : k_begin;
    const int64_t head_off = static_cast<int64_t>(h) * a.page_size * hd + col;
    const int64_t page_stride = static_cast<int64_t>(a.n_head) * a.page_size * hd;
    const int* my_bt = sbt + mc * a.max_blocks;
    const int last_pos = max(pos - 1, 0);
    auto fetch_keys = [&](int j0, u32x4 (&kv)[AU], u32x4 (&vv)[AU], bool (&valid)[AU]) {
#pragma unroll
        for (int u = 0; u < AU; ++u) {
            const int j = j0 + u * WPT * KPP + kg;
            valid[u] = j < k_end;
            const int jc = valid[u] ? j : last_pos;  // a mapped position; its values are not used
            // no branch around the loads: a load under a branch is waited for where the branch ends
            const int lp = a.page_shift >= 0 ? jc >> a.page_shift : jc / a.page_size;
            const int off = a.page_shift >= 0 ? jc & (a.page_size - 1) : jc % a.page_size;
            const int64_t src = static_cast<int64_t>(my_bt[lp]) * page_stride + head_off + static_cast<int64_t>(off) * hd;
            kv[u] = *reinterpret_cast<const u32x4*>(a.kc + src);
            vv[u] = *reinterpret_cast<const u32x4*>(a.vc + src);
        }
    };
    // the first trip's keys and values are asked for now, behind the weights: they do not depend on
    // the query and arrive while it is projected
    u32x4 kv0[AU], vv0[AU];
    bool valid0[AU];
    const int j_first = k_begin + sw * KPP;
    if (role < S) {
        fetch_keys(j_first, kv0, vv0, valid0);
    } else {
#pragma unroll
        for (int u = 0; u < AU; ++u) {
            kv0[u] = zero;
            vv0[u] = zero;
            valid0[u] = false;
        }
    }

    // -- a projection: dst[m][d] = bf16(x[m] . w[row0 + d] + bias[row0 + d]) -------------------
    const bf16_t* arow = xs + min(i, nt - 1) * ldx;  // rows past the last token repeat it; their sums are dropped
    const int units = (K + 63) / 64;
    auto project = [&](int row0, float* dst) {
        floatx4 acc[NT];
#pragma unroll
        for (int t = 0; t < NT; ++t) acc[t] = floatx4{0.0f, 0.0f, 0.0f, 0.0f};
        auto multiply = [&](int u0) {
#pragma unroll
            for (int p = 0; p < 2; ++p) {
                const int k = (u0 + p) * 64 + g * 8;
                Frag x0, x1;
                x0.u = piece(arow, k);
                x1.u = piece(arow, k + 32);
#pragma unroll
                for (int t = 0; t < NT; ++t) {
                    acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wc[p][t][0].v, x0.v, acc[t], 0, 0, 0);
                    acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wc[p][t][1].v, x1.v, acc[t], 0, 0, 0);
                }
            }
        };
        int u0 = wave * 2;
        for (; u0 + 2 * FW < units; u0 += 2 * FW) {
            Frag wn[2][NT][2];
            load_w(row0, u0 + 2 * FW, wn);
            multiply(u0);
#pragma unroll
            for (int p = 0; p < 2; ++p)
#pragma unroll
                for (int t = 0; t < NT; ++t) {
                    wc[p][t][0] = wn[p][t][0];
                    wc[p][t][1] = wn[p][t][1];
                }
        }
        multiply(u0);  // a wave past the end of K holds zeros
        // acc[t][c] = partial C^T[d = 16 t + 4 g + c][m = i]; kept [tile][m][d] per wave, added up in wave order
#pragma unroll
        for (int t = 0; t < NT; ++t)
#pragma unroll
            for (int cc = 0; cc < 4; ++cc) red[(wave * NT + t) * 256 + i * 16 + 4 * g + cc] = acc[t][cc];
        lds_barrier();
        for (int e = tid; e < NT * 256; e += 64 * FW) {
            const int t = e / 256, m = (e % 256) / 16, d = 16 * t + e % 16;
            float v = 0.0f;
#pragma unroll
            for (int q = 0; q < FW; ++q) v += red[q * NT * 256 + e];
            if (a.bias != nullptr) v += a.bias[row0 + d];
            if (m < MAX_TG) dst[m * HDP + d] = bf16_to_float(float_to_bf16(v));
        }
        lds_barrier();
    };
    project(row_first, qs);

    const int split_count = S + 1;
    if (role >= S) {
        // -- the token's own position: key and score (role S), value (role S + 1) ---------------
        if (role == S) {
            load_w(q_dim + h * hd, wave * 2, wc);
            project(q_dim + h * hd, ks);
        }
        if (wave < nt) {
            const int t = m0 + wave, d = lane;
            const float first_v = d < hd ? qs[wave * HDP + d] : 0.0f;
            const float second_v = (role == S && d < hd) ? ks[wave * HDP + d] : 0.0f;
            const int64_t slot = a.slots[t];
            const bool mapped = static_cast<uint64_t>(slot) < static_cast<uint64_t>(a.num_pages) * static_cast<uint64_t>(a.page_size);
            const int64_t page = slot / a.page_size, off = slot - page * a.page_size;
            const int64_t dst = ((page * a.n_head + h) * a.page_size + off) * hd + d;
            float* p = a.partials + ((static_cast<int64_t>(t) * a.n_head + h) * split_count + S) * (hd + 4);
            if (role == S) {
                const float score = wave_sum(first_v * second_v) * a.scale;
                if (d < hd && mapped) a.kc[dst] = float_to_bf16(second_v);
                if (d == 0) {
                    p[hd] = score;
                    p[hd + 1] = 1.0f;
                }
            } else if (d < hd) {
                if (mapped) a.vc[dst] = float_to_bf16(first_v);
                p[d] = first_v;
            }
        }
        return;
    }

    // -- attention over this wave's share of its token's cached keys -----------------------------
    float qf[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) qf[e] = active ? qs[mc * HDP + col + e] : 0.0f;
    Partial st;
    st.m = -INFINITY;
    st.l = 0.0f;
#pragma unroll
    for (int e = 0; e < 8; ++e) st.acc[e] = 0.0f;
    auto absorb = [&](const u32x4 (&kv)[AU], const u32x4 (&vv)[AU], const bool (&valid)[AU]) {
        float s[AU];
        float m_new = st.m;
#pragma unroll
        for (int u = 0; u < AU; ++u) {
            float kf[8];
            unpack8(kv[u], kf);
            float d = 0.0f;
#pragma unroll
            for (int e = 0; e < 8; ++e) d = fmaf(kf[e], qf[e], d);
            d = group_sum<LPK>(d);  // over the lanes that share the key
            s[u] = valid[u] ? d * a.scale : -INFINITY;
            m_new = fmaxf(m_new, s[u]);
        }
        if (m_new == -INFINITY) return;  // this lane group had no key in this trip (and none before)
        const float corr = st.m == -INFINITY ? 0.0f : __expf(st.m - m_new);
        st.l *= corr;
#pragma unroll
        for (int e = 0; e < 8; ++e) st.acc[e] *= corr;
#pragma unroll
        for (int u = 0; u < AU; ++u) {
            if (!valid[u]) continue;
            const float p = __expf(s[u] - m_new);
            st.l += p;
            float vf[8];
            unpack8(vv[u], vf);
#pragma unroll
            for (int e = 0; e < 8; ++e) st.acc[e] = fmaf(p, vf[e], st.acc[e]);
        }
        st.m = m_new;
    };
    absorb(kv0, vv0, valid0);
    for (int j0 = j_first + WPT * KPP * AU; j0 < k_end; j0 += WPT * KPP * AU) {
        u32x4 kv[AU], vv[AU];
        bool valid[AU];
        fetch_keys(j0, kv, vv, valid);
        absorb(kv, vv, valid);
    }
    // lane groups of the wave, in a fixed tree
#pragma unroll
    for (int off = LPK; off < 64; off <<= 1) {
        const float mo = __shfl_xor(st.m, off, 64), lo = __shfl_xor(st.l, off, 64);
        float ao[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) ao[e] = __shfl_xor(st.acc[e], off, 64);
        merge_partial(st, mo, lo, ao);
    }
    if (kg == 0) {
        float* mine = wsum + (wave * LPK + c) * 10;
        mine[0] = st.m;
        mine[1] = st.l;
#pragma unroll
        for (int e = 0; e < 8; ++e) mine[2 + e] = st.acc[e];
    }
    __syncthreads();
    if (sw == 0 && kg == 0 && active && tok_valid) {
        for (int w = 1; w < WPT; ++w) {
            const float* other = wsum + ((wave + w) * LPK + c) * 10;
            merge_partial(st, other[0], other[1], other + 2);
        }
        // partials [token][head][split][hd + 4]: values, then maximum and sum
        float* p = a.partials + ((static_cast<int64_t>(tok) * a.n_head + h) * split_count + role) * (hd + 4);
#pragma unroll
        for (int e = 0; e < 8; ++e) p[c * 8 + e] = st.acc[e];
        if (c == 0) {
            p[hd] = st.m;
            p[hd + 1] = st.l;
        }
    }
}

inline size_t lds_bytes(int TG, int K, int NT, int max_blocks) {
    const int LPK = NT == 1 ? 2 : (NT == 2 ? 4 : 8);
    size_t at = ((static_cast<size_t>(TG) * (K + 8) * 2 + 15) / 16) * 16;
    at += static_cast<size_t>(FW) * NT * 256 * sizeof(float);
    at += 2 * static_cast<size_t>(MAX_TG) * 16 * NT * sizeof(float);
    at += static_cast<size_t>(FW) * LPK * 10 * sizeof(float);
    at += static_cast<size_t>(TG) * max_blocks * sizeof(int);
    return at;
}

template <int MAXV, int NT>
int launch(const Args& a, dim3 grid, size_t smem, hipStream_t stream) {
    auto kern = attention_decode_qkv_kernel<MAXV, NT>;
    static bool ready = false;
    if (!ready) {
        hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        ready = true;
    }
    kern<<<grid, 64 * FW, smem, stream>>>(a);
    return check_launch("attention_decode_qkv");
}

template <int MAXV>
int launch_heads(const Args& a, dim3 grid, size_t smem, hipStream_t stream) {
    switch (a.hd / 16) {
        case 1: return launch<MAXV, 1>(a, grid, smem, stream);
        case 2: return launch<MAXV, 2>(a, grid, smem, stream);
        case 3: return launch<MAXV, 3>(a, grid, smem, stream);
        default: return launch<MAXV, 4>(a, grid, smem, stream);
    }
}

}  // namespace decode_qkv
}  // namespace liyab

using namespace liyab;

// partials[m][h][z] for z < key_splits: split z of token m's cached keys (its own position left
// out); partials[m][h][key_splits]: the token's own key and value (maximum = its score, sum = 1),
// which also go to slot slots[m] of the pages. planes: float32 [n_planes][M][K], plane_stride
// floats apart; w_qkv [3 * n_head * hd][K] bfloat16 (queries, keys, values; as many key/value heads
// as query heads); caches bfloat16 [num_pages][n_head][page_size][hd]; block_tables [M][max_blocks]
// (row m is token m's request), tok_pos [M] the tokens' own positions. M <= 16; hd a multiple of 16
// up to 64; K a multiple of 8 up to 2048; key_splits 1..7; tokens_per_group 1, 2, 4 or 8.
extern "C" int liyab_attention_decode_qkv(const float* planes, int n_planes, int64_t plane_stride, const float* ln_weight,
                                          const float* ln_bias, float eps, const void* w_qkv, const float* b_qkv, void* kc,
                                          void* vc, int num_pages, int page_size, const int* block_tables, int max_blocks,
                                          const int* tok_pos, const int* slots, int M, int K, int n_head, int hd, float scale,
                                          int window, int key_splits, int tokens_per_group, float* partials,
                                          hipStream_t stream) {
    using namespace liyab::decode_qkv;
    LIYAB_REQUIRE(planes && w_qkv && kc && vc && block_tables && tok_pos && slots && partials, "attention_decode_qkv: null operand");
    LIYAB_REQUIRE(M >= 0 && M <= 16, "attention_decode_qkv: %d tokens (at most 16)", M);
    LIYAB_REQUIRE(K > 0 && K % 8 == 0 && K <= 2048, "attention_decode_qkv: K %d must be a multiple of 8, at most 2048", K);
    LIYAB_REQUIRE(hd >= 16 && hd <= 64 && hd % 16 == 0, "attention_decode_qkv: head size %d is not a multiple of 16 in 16..64", hd);
    LIYAB_REQUIRE(n_head > 0 && n_head <= 65535, "attention_decode_qkv: bad head count %d", n_head);
    LIYAB_REQUIRE(n_planes >= 1 && n_planes <= 16, "attention_decode_qkv: %d planes (1 to 16)", n_planes);
    LIYAB_REQUIRE(n_planes == 1 || plane_stride >= static_cast<int64_t>(M) * K, "attention_decode_qkv: planes of %lld floats overlap",
                  static_cast<long long>(plane_stride));
    auto al16 = [](const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; };
    LIYAB_REQUIRE(al16(planes) && al16(w_qkv) && al16(ln_weight) && al16(ln_bias) && al16(kc) && al16(vc) && al16(partials) && plane_stride % 4 == 0,
                  "attention_decode_qkv: operands must be 16-byte aligned");
    LIYAB_REQUIRE(eps >= 0.0f, "attention_decode_qkv: negative eps");
    LIYAB_REQUIRE(num_pages > 0 && page_size > 0 && max_blocks > 0 && static_cast<int64_t>(num_pages) * page_size < (int64_t{1} << 31),
                  "attention_decode_qkv: bad cache sizes (%d pages of %d, tables of %d)", num_pages, page_size, max_blocks);
    LIYAB_REQUIRE(window >= 0, "attention_decode_qkv: negative window");
    LIYAB_REQUIRE(key_splits >= 1 && key_splits <= 7, "attention_decode_qkv: %d splits of the cached keys (1 to 7)", key_splits);
    LIYAB_REQUIRE(tokens_per_group == 1 || tokens_per_group == 2 || tokens_per_group == 4 || tokens_per_group == 8,
                  "attention_decode_qkv: %d tokens a workgroup (1, 2, 4 or 8)", tokens_per_group);
    if (M == 0) return 0;
    const size_t smem = lds_bytes(tokens_per_group, K, hd / 16, max_blocks);
    LIYAB_REQUIRE(smem <= 160 * 1024, "attention_decode_qkv: %d tokens of %d with tables of %d pages need %zu bytes of LDS", tokens_per_group, K,
                  max_blocks, smem);
    int page_shift = -1, wpt_shift = 0;
    for (int b = 0; b < 31; ++b)
        if ((1 << b) == page_size) page_shift = b;
    while ((tokens_per_group << (wpt_shift + 1)) <= FW) ++wpt_shift;
    const Args a{planes, n_planes, plane_stride, ln_weight, ln_bias, eps, static_cast<const bf16_t*>(w_qkv), b_qkv,
                 static_cast<bf16_t*>(kc), static_cast<bf16_t*>(vc), num_pages, page_size, page_shift, block_tables, max_blocks,
                 tok_pos, slots, M, K, n_head, hd, scale, window, key_splits, tokens_per_group, wpt_shift, partials};
    const dim3 grid(n_head, key_splits + 2, (M + tokens_per_group - 1) / tokens_per_group);
    if (K <= 512) return launch_heads<2>(a, grid, smem, stream);
    if (K <= 768) return launch_heads<3>(a, grid, smem, stream);
    if (K <= 1024) return launch_heads<4>(a, grid, smem, stream);
    return launch_heads<8>(a, grid, smem, stream);
}
