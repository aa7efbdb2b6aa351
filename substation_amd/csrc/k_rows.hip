// Row operators: softmax(+scale+dropout), softmax backward, bias+dropout+
// residual+LayerNorm, LayerNorm backward(+dropout backward).
// One wave64 per row, the whole row in registers (single global read), fp32 math,
// 128-bit accesses where the row dimension is contiguous.  Short rows are
// processed several per wave at once so that enough loads are in flight.
// Counterparts: pytorch_module/block_softmax.cuh:12-188, block_bs.cuh:13-156,
// block_bdrln.cuh:17-352, block_blnrd.cuh:14-259.
#include "sub_ops.hpp"

namespace sub {

namespace {

constexpr int BLOCK = 256;
constexpr int WPB = BLOCK / WAVE;
constexpr float LOG2E = 1.4426950408889634f;

__device__ __forceinline__ int nvalid_at(int R, int e0) {
    int n = R - e0;
    return n < 0 ? 0 : (n > 8 ? 8 : n);
}

// VPL: 8-packs per lane (row length <= 8*GRP*VPL).  RPW: rows per lane group per
// step.  FAST: all views vectorisable (see ld8).  GRP: lanes per row; rows of up
// to 256 (128) elements take half (a quarter) of a wave, so that two (four) of
// them are processed side by side and no lane idles.
// amask (optional, p == nullptr when absent): additive attention mask indexed by
// (query position, key position) only, x = beta * scale + amask * mscale
// (substation/attention.py:65-68 adds it before the scaling, hence mscale).
template <int VPL, int RPW, bool FAST, bool FLAT = false, int GRP = WAVE, bool MASKED = false>
__global__ __launch_bounds__(BLOCK) void k_softmax(RowSpace rs, View beta, View alpha, View mask,
                                                   View drop, View amask, float scale, float mscale,
                                                   PhiloxKey key_, unsigned nrows) {
    const PhiloxKey key = resolved(key_);
    constexpr int SPW = WAVE / GRP;                    // rows side by side in a wave
    const int lane = threadIdx.x & 63, gl = lane % GRP, sub = lane / GRP;
    const unsigned step = gridDim.x * WPB * RPW * SPW;
    for (unsigned row0 = (blockIdx.x * WPB + (threadIdx.x >> 6)) * RPW * SPW; row0 < nrows; row0 += step) {
        float x[RPW][VPL][8];
        RowIdx ix[RPW];
        float m[RPW], s[RPW];
#pragma unroll
        for (int r = 0; r < RPW; ++r) {
            const unsigned row = row0 + r * SPW + sub;
            const bool live = row < nrows;
            ix[r] = row_index_of<FLAT>(rs, live ? row : row0);
            const long ob = view_offset_of<FLAT>(beta, ix[r]);
            const long oam = MASKED ? view_offset_of<FLAT>(amask, ix[r]) : 0;
            m[r] = -INFINITY;
#pragma unroll
            for (int c = 0; c < VPL; ++c) {
                int e0 = (c * GRP + gl) * 8;
                int nv = live ? nvalid_at(rs.R, e0) : 0;
                F8 f = ld8<FAST, true>(beta, ob, e0, nv, -INFINITY);
                if (MASKED) {
                    // every (head, sample) re-reads the mask: plain loads, it stays in cache
                    F8 am = load8(amask, oam, e0, nv, 0.f);
#pragma unroll
                    for (int i = 0; i < 8; ++i) f.v[i] = f.v[i] * scale + am.v[i] * mscale;
                } else {
#pragma unroll
                    for (int i = 0; i < 8; ++i) f.v[i] = f.v[i] * scale;
                }
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    x[r][c][i] = f.v[i];
                    m[r] = fmaxf(m[r], x[r][c][i]);
                }
            }
        }
#pragma unroll
        for (int r = 0; r < RPW; ++r) m[r] = group_max<GRP>(m[r]);
#pragma unroll
        for (int r = 0; r < RPW; ++r) {
            s[r] = 0.f;
#pragma unroll
            for (int c = 0; c < VPL; ++c)
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    x[r][c][i] = __builtin_amdgcn_exp2f((x[r][c][i] - m[r]) * LOG2E);
                    s[r] += x[r][c][i];
                }
        }
#pragma unroll
        for (int r = 0; r < RPW; ++r) s[r] = group_sum<GRP>(s[r]);
#pragma unroll
        for (int r = 0; r < RPW; ++r) {
            const unsigned row = row0 + r * SPW + sub;
            if (row >= nrows) continue;
            const float inv = 1.0f / s[r];
            const long oa = view_offset_of<FLAT>(alpha, ix[r]), om = view_offset_of<FLAT>(mask, ix[r]), od = view_offset_of<FLAT>(drop, ix[r]);
#pragma unroll
            for (int c = 0; c < VPL; ++c) {
                int e0 = (c * GRP + gl) * 8;
                int nv = nvalid_at(rs.R, e0);
                if (nv > 0) {
                    h8 a, d;
                    uint32_t bits = keep_pack<FAST>(key, (uint64_t)row * (uint64_t)rs.R + (uint64_t)e0);
#pragma unroll
                    for (int i = 0; i < 8; ++i) a[i] = (half_t)(x[r][c][i] * inv);
                    a = pin(a);
#pragma unroll
                    for (int i = 0; i < 8; ++i) d[i] = ((bits >> i) & 1u) ? a[i] : (half_t)0.0f;
                    st8h<FAST, true>(alpha, oa, e0, nv, a);
                    st8h<FAST, true>(mask, om, e0, nv, mask_h8(bits));
                    st8h<FAST>(drop, od, e0, nv, d);
                }
            }
        }
    }
}

template <int VPL, int RPW, bool FAST, bool FLAT = false, int GRP = WAVE>
__global__ __launch_bounds__(BLOCK) void k_bs(RowSpace rs, View alpha, View mask, View ddrop,
                                              View dbeta, float scale, unsigned nrows) {
    constexpr int SPW = WAVE / GRP;
    const int lane = threadIdx.x & 63, gl = lane % GRP, sub = lane / GRP;
    const unsigned step = gridDim.x * WPB * RPW * SPW;
    for (unsigned row0 = (blockIdx.x * WPB + (threadIdx.x >> 6)) * RPW * SPW; row0 < nrows; row0 += step) {
        float a[RPW][VPL][8], g[RPW][VPL][8];
        RowIdx ix[RPW];
        float s[RPW];
#pragma unroll
        for (int r = 0; r < RPW; ++r) {
            const unsigned row = row0 + r * SPW + sub;
            const bool live = row < nrows;
            ix[r] = row_index_of<FLAT>(rs, live ? row : row0);
            const long oa = view_offset_of<FLAT>(alpha, ix[r]), om = view_offset_of<FLAT>(mask, ix[r]), od = view_offset_of<FLAT>(ddrop, ix[r]);
            s[r] = 0.f;
#pragma unroll
            for (int c = 0; c < VPL; ++c) {
                int e0 = (c * GRP + gl) * 8;
                int nv = live ? nvalid_at(rs.R, e0) : 0;
                F8 fa = ld8<FAST, true>(alpha, oa, e0, nv), fm = ld8<FAST, true>(mask, om, e0, nv), fd = ld8<FAST, true>(ddrop, od, e0, nv);
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    a[r][c][i] = fa.v[i];
                    g[r][c][i] = fm.v[i] * fd.v[i];
                    s[r] += a[r][c][i] * g[r][c][i];
                }
            }
        }
#pragma unroll
        for (int r = 0; r < RPW; ++r) s[r] = group_sum<GRP>(s[r]);
#pragma unroll
        for (int r = 0; r < RPW; ++r) {
            if (row0 + r * SPW + sub >= nrows) continue;
            const long oo = view_offset_of<FLAT>(dbeta, ix[r]);
#pragma unroll
            for (int c = 0; c < VPL; ++c) {
                int e0 = (c * GRP + gl) * 8;
                int nv = nvalid_at(rs.R, e0);
                if (nv > 0) {
                    h8 o;
#pragma unroll
                    for (int i = 0; i < 8; ++i) o[i] = (half_t)(scale * a[r][c][i] * (g[r][c][i] - s[r]));
                    st8h<FAST>(dbeta, oo, e0, nv, o);
                }
            }
        }
    }
}

template <int VPL, int RPW, bool FAST>
__global__ __launch_bounds__(BLOCK) void k_bdrln(RowSpace rs, View in, View resid, View lin_bias,
                                                 View scale, View bias, View lin, View mask,
                                                 View diff, View normed, View out, View istd,
                                                 PhiloxKey key_, float eps, unsigned nrows, uint8_t* mask_bits,
                                                 bool write_lin, KeepWordsJob side) {
    // side.blocks workgroups behind those of the rows only draw keep words: the rows wait for memory
    // with the vector units idle
    const unsigned row_blocks = gridDim.x - side.blocks;
    if (blockIdx.x >= row_blocks) {
        const PhiloxKey skey = resolved(side.key);
        const uint32_t tiles_n = side.N / 256, items = (side.M / 256) * tiles_n * 512;
        for (uint32_t id = (blockIdx.x - row_blocks) * BLOCK + threadIdx.x; id < items; id += side.blocks * BLOCK) {
            const uint32_t tile = id >> 9, tm = tile / tiles_n;
            const KeepWords k = relu_dropout_keep_words(skey, side.N, tm, tile - tm * tiles_n, (id >> 6) & 7, id & 63);
            reinterpret_cast<uint4*>(side.out)[id] = make_uint4(k.w[0], k.w[1], k.w[2], k.w[3]);
        }
        return;
    }
    const PhiloxKey key = resolved(key_);
    const int lane = threadIdx.x & 63;
    const unsigned step = row_blocks * WPB * RPW;
    const float invn = 1.0f / (float)rs.R;
    // the lane's columns of the LayerNorm scale and bias: the same for every row, fetched once
    // and together with the first row (in the store phase they were a round trip of their own)
    h8 sc8[VPL], bi8[VPL];
    if (FAST) {
#pragma unroll
        for (int c = 0; c < VPL; ++c) {
            const int e0 = (c * WAVE + lane) * 8, e0s = nvalid_at(rs.R, e0) ? e0 : 0;
            sc8[c] = ldg8<false>(scale.p + e0s);
            bi8[c] = ldg8<false>(bias.p + e0s);
        }
    }
    for (unsigned row0 = (blockIdx.x * WPB + (threadIdx.x >> 6)) * RPW; row0 < nrows; row0 += step) {
        float x[RPW][VPL][8];
        uint32_t bits[RPW][VPL];
        RowIdx ix[RPW];
        float s[RPW], q[RPW];
        // pass 1: loads of every row first, then bias/dropout/residual
#pragma unroll
        for (int r = 0; r < RPW; ++r) {
            const bool live = row0 + r < nrows;
            ix[r] = row_index(rs, live ? row0 + r : row0);
            const long oi = view_offset(in, ix[r]), orr = view_offset(resid, ix[r]);
            const long ol = view_offset(lin, ix[r]), om = view_offset(mask, ix[r]);
            s[r] = 0.f;
            // every load of the row before the first store: the compiler keeps a load behind a
            // store that might write what it reads, and the packs of a row would make one round
            // trip to memory each
            F8 fis[VPL], frs[VPL], fbs[VPL];
#pragma unroll
            for (int c = 0; c < VPL; ++c) {
                int e0 = (c * WAVE + lane) * 8;
                int nv = live ? nvalid_at(rs.R, e0) : 0;
                fis[c] = ld8<FAST, true>(in, oi, e0, nv);
                frs[c] = ld8<FAST>(resid, orr, e0, nv);
                fbs[c] = ld8<FAST>(lin_bias, 0, e0, nv);
            }
#pragma unroll
            for (int c = 0; c < VPL; ++c) {
                int e0 = (c * WAVE + lane) * 8;
                int nv = live ? nvalid_at(rs.R, e0) : 0;
                const F8 &fi = fis[c], &fr = frs[c], &fb = fbs[c];
                // (FAST: drawn for every lane, no branch between the loads and their first use)
                bits[r][c] = FAST ? keep_pack<true>(key, (uint64_t)(row0 + r) * (uint64_t)rs.R + (uint64_t)e0)
                             : nv > 0 ? keep_bits8(key, (uint64_t)(row0 + r) * (uint64_t)rs.R + (uint64_t)e0) : 0u;
                h8 lh;
#pragma unroll
                for (int i = 0; i < 8; ++i) lh[i] = (half_t)(fi.v[i] + fb.v[i]);
                lh = pin(lh);                                      // LIN is stored; use its rounded value
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    float kept = ((bits[r][c] >> i) & 1u) ? (float)lh[i] : 0.f;
                    // (FAST: a chunk outside the row was loaded as zeros and sums to zero)
                    x[r][c][i] = (FAST || i < nv) ? kept + fr.v[i] : 0.f;
                    s[r] += x[r][c][i];
                }
                if (nv > 0) {
                    if (write_lin) st8h<FAST, true>(lin, ol, e0, nv, lh);
                    if (mask_bits) mask_bits[(size_t)(row0 + r) * (rs.R >> 3) + (c * WAVE + lane)] = (uint8_t)bits[r][c];
                    else st8h<FAST, true>(mask, om, e0, nv, mask_h8(bits[r][c]));
                }
            }
        }
#pragma unroll
        for (int r = 0; r < RPW; ++r) s[r] = wave_sum(s[r]) * invn;      // mean
#pragma unroll
        for (int r = 0; r < RPW; ++r) {
            q[r] = 0.f;
#pragma unroll
            for (int c = 0; c < VPL; ++c) {
                int e0 = (c * WAVE + lane) * 8;
                int nv = nvalid_at(rs.R, e0);
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    x[r][c][i] = i < nv ? x[r][c][i] - s[r] : 0.f;
                    q[r] += x[r][c][i] * x[r][c][i];
                }
            }
        }
#pragma unroll
        for (int r = 0; r < RPW; ++r) q[r] = rsqrtf(wave_sum(q[r]) * invn + eps);   // 1/std
#pragma unroll
        for (int r = 0; r < RPW; ++r) {
            if (row0 + r >= nrows) continue;
            const float is = q[r];
            if (lane == 0) istd.p[view_offset(istd, ix[r])] = (half_t)is;
            const long od = view_offset(diff, ix[r]), on = view_offset(normed, ix[r]), oo = view_offset(out, ix[r]);
#pragma unroll
            for (int c = 0; c < VPL; ++c) {
                int e0 = (c * WAVE + lane) * 8;
                int nv = nvalid_at(rs.R, e0);
                if (nv > 0) {
                    F8 fs, fb;
                    if (FAST) {
                        // (opaque here: converted ahead of the loop, they would be waited for there,
                        // before the row's own loads are issued)
                        const h8 s8 = pin(sc8[c]), b8 = pin(bi8[c]);
#pragma unroll
                        for (int i = 0; i < 8; ++i) { fs.v[i] = (float)s8[i]; fb.v[i] = (float)b8[i]; }
                    } else {
                        fs = ld8<FAST>(scale, 0, e0, nv); fb = ld8<FAST>(bias, 0, e0, nv);
                    }
                    h8 d, n, o;
#pragma unroll
                    for (int i = 0; i < 8; ++i) {
                        float nn = x[r][c][i] * is;
                        d[i] = (half_t)x[r][c][i];
                        n[i] = (half_t)nn;
                        o[i] = (half_t)(nn * fs.v[i] + fb.v[i]);
                    }
                    st8h<FAST, true>(diff, od, e0, nv, d);
                    st8h<FAST, true>(normed, on, e0, nv, n);
                    st8h<FAST>(out, oo, e0, nv, o);
                }
            }
        }
    }
}

// k_bdrln for the layouts the encoder layer runs with: every view vectorisable and the row
// space flat (row r of a view starts r * s3 elements in), one row per wave and pass.  Same
// arithmetic in the same order, bit for bit; what goes is the generic kernel's bookkeeping
// (four outer indices and strides per view, a validity count per element: over 1000 vector
// instructions per row, half of them before the row's loads are issued, with four waves per
// SIMD taking turns on them; the launch was bound by that, not by memory).  Here a chunk is
// inside the row or outside it, the row's loads are issued first, together with the lane's
// columns of the three per-feature vectors, and the keep bits are drawn while they travel.
template <int VPL>
__global__ __launch_bounds__(BLOCK) void k_bdrln_flat(int R, unsigned nrows, View in, View resid, View lin_bias,
                                                      View scale, View bias, View lin, View mask, View diff,
                                                      View normed, View out, View istd, PhiloxKey key_, float eps,
                                                      uint8_t* mask_bits, bool write_lin, KeepWordsJob side) {
    fetch_args_now(R, nrows, in.p, in.s3, resid.p, resid.s3, lin_bias.p, scale.p, bias.p, lin.p, lin.s3, mask.p, mask.s3,
                   diff.p, diff.s3, normed.p, normed.s3, out.p, out.s3, istd.p, istd.s3, key_.k0, key_.k1, key_.site,
                   key_.step, key_.thr, key_.step_dev, eps, mask_bits, write_lin, side.blocks);
    const unsigned row_blocks = gridDim.x - side.blocks;
    if (blockIdx.x >= row_blocks) {
        const PhiloxKey skey = resolved(side.key);
        const uint32_t tiles_n = side.N / 256, items = (side.M / 256) * tiles_n * 512;
        for (uint32_t id = (blockIdx.x - row_blocks) * BLOCK + threadIdx.x; id < items; id += side.blocks * BLOCK) {
            const uint32_t tile = id >> 9, tm = tile / tiles_n;
            const KeepWords k = relu_dropout_keep_words(skey, side.N, tm, tile - tm * tiles_n, (id >> 6) & 7, id & 63);
            reinterpret_cast<uint4*>(side.out)[id] = make_uint4(k.w[0], k.w[1], k.w[2], k.w[3]);
        }
        return;
    }
    const int lane = threadIdx.x & 63;
    const float invn = 1.0f / (float)R;
    // (the step counter of a captured graph: fetched first and added where the keep bits are drawn, so
    // that the wait for it stands behind the issue of every other load)
    uint32_t step_extra = 0;
    if (key_.step_dev) step_extra = *key_.step_dev;
    // A chunk outside the row (rows shorter than the lanes cover) reads the row's first pack and has it
    // and-ed away: no branch around a load or around the first use of one, where the wait for it would go.
    typedef int i4v __attribute__((ext_vector_type(4)));
    bool inside[VPL];
    int e0[VPL], keep_all[VPL];
    h8 sc8[VPL], bi8[VPL], lb8[VPL];
#pragma unroll
    for (int c = 0; c < VPL; ++c) {
        e0[c] = (c * WAVE + lane) * 8;
        inside[c] = e0[c] < R;
        keep_all[c] = inside[c] ? -1 : 0;
        if (!inside[c]) e0[c] = 0;
        lb8[c] = ldg8<false>(lin_bias.p + e0[c]);
        sc8[c] = ldg8<false>(scale.p + e0[c]);
        bi8[c] = ldg8<false>(bias.p + e0[c]);
    }
    auto masked = [&](h8 v, int c) { return __builtin_bit_cast(h8, __builtin_bit_cast(i4v, v) & keep_all[c]); };
    for (unsigned row = blockIdx.x * WPB + (threadIdx.x >> 6); row < nrows; row += row_blocks * WPB) {
        h8 vi[VPL], vr[VPL];
#pragma unroll
        for (int c = 0; c < VPL; ++c) {
            vi[c] = ldg8<true>(in.p + (long)row * in.s3 + e0[c]);
            vr[c] = ldg8<false>(resid.p + (long)row * resid.s3 + e0[c]);
        }
        // the keep bits are drawn while the loads travel: nothing that waits for one may move up here
        __builtin_amdgcn_sched_barrier(0);
        PhiloxKey key = key_;
        {
            uint32_t se = step_extra;
            asm volatile("" : "+v"(se));                         // (not hoisted out of the loop, with its wait)
            key.step += (uint32_t)__builtin_amdgcn_readfirstlane((int)se);
            key.step_dev = nullptr;
        }
        uint32_t bits[VPL];
#pragma unroll
        for (int c = 0; c < VPL; ++c)
            bits[c] = keep_pack<true>(key, (uint64_t)row * (uint64_t)R + (uint64_t)((c * WAVE + lane) * 8));
        __builtin_amdgcn_sched_barrier(0);
        float x[VPL][8];
        float s = 0.f;
#pragma unroll
        for (int c = 0; c < VPL; ++c) {
            // (opaque here: converted ahead of the loop, the per-feature vectors would be waited for
            // there, before the row's own loads are issued)
            const h8 in8 = masked(vi[c], c), re8 = masked(vr[c], c), lbm = masked(pin(lb8[c]), c);
            h8 lh;
#pragma unroll
            for (int i = 0; i < 8; ++i) lh[i] = (half_t)((float)in8[i] + (float)lbm[i]);
            lh = pin(lh);                                          // LIN is stored; use its rounded value
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const float kept = __int_as_float(__float_as_int((float)lh[i]) & __builtin_amdgcn_sbfe((int)bits[c], i, 1));
                x[c][i] = kept + (float)re8[i];
                s += x[c][i];
            }
            if (inside[c]) {
                if (write_lin) stg8<true>(lin.p + (long)row * lin.s3 + e0[c], lh);
                if (mask_bits) mask_bits[(size_t)row * (R >> 3) + (c * WAVE + lane)] = (uint8_t)bits[c];
                else stg8<true>(mask.p + (long)row * mask.s3 + e0[c], mask_h8(bits[c]));
            }
        }
        const float mean = wave_sum(s) * invn;
        float q = 0.f;
#pragma unroll
        for (int c = 0; c < VPL; ++c)
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                x[c][i] = __int_as_float(__float_as_int(x[c][i] - mean) & keep_all[c]);
                q += x[c][i] * x[c][i];
            }
        const float is = rsqrtf(wave_sum(q) * invn + eps);       // 1/std
        if (lane == 0) istd.p[(long)row * istd.s3] = (half_t)is;
#pragma unroll
        for (int c = 0; c < VPL; ++c) {
            if (!inside[c]) continue;
            const h8 s8 = pin(sc8[c]), b8 = pin(bi8[c]);
            h8 d, n, o;
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const float nn = x[c][i] * is;
                d[i] = (half_t)x[c][i];
                n[i] = (half_t)nn;
                o[i] = (half_t)(nn * (float)s8[i] + (float)b8[i]);
            }
            stg8<true>(diff.p + (long)row * diff.s3 + e0[c], d);
            stg8<true>(normed.p + (long)row * normed.s3 + e0[c], n);
            stg8<false>(out.p + (long)row * out.s3 + e0[c], o);
        }
    }
}

template <int VPL, int RPW, bool FAST, bool FLAT = false>
__global__ __launch_bounds__(BLOCK) void k_blnrd(RowSpace rs, View dout, View istd, View diff,
                                                 View mask, View d_ln_in, View d_drop_in, unsigned nrows,
                                                 const uint8_t* mask_bits) {
    const int lane = threadIdx.x & 63;
    const unsigned step = gridDim.x * WPB * RPW;
    const float invn = 1.0f / (float)rs.R;
    for (unsigned row0 = (blockIdx.x * WPB + (threadIdx.x >> 6)) * RPW; row0 < nrows; row0 += step) {
        float g[RPW][VPL][8], df[RPW][VPL][8];
        h8 mk[RPW][VPL];
        RowIdx ix[RPW];
        float s1[RPW], s2[RPW], is[RPW];
#pragma unroll
        for (int r = 0; r < RPW; ++r) {
            const bool live = row0 + r < nrows;
            ix[r] = row_index_of<FLAT>(rs, live ? row0 + r : row0);
            const long oo = view_offset_of<FLAT>(dout, ix[r]), od = view_offset_of<FLAT>(diff, ix[r]), om = view_offset_of<FLAT>(mask, ix[r]);
            is[r] = (float)istd.p[view_offset_of<FLAT>(istd, ix[r])];
            s1[r] = 0.f; s2[r] = 0.f;
#pragma unroll
            for (int c = 0; c < VPL; ++c) {
                int e0 = (c * WAVE + lane) * 8;
                int nv = live ? nvalid_at(rs.R, e0) : 0;
                F8 fg = ld8<FAST, true>(dout, oo, e0, nv), fd = ld8<FAST, true>(diff, od, e0, nv);
                F8 fm;
                if (mask_bits) {
                    const uint32_t b = nv > 0 ? mask_bits[(size_t)(row0 + r) * (rs.R >> 3) + (c * WAVE + lane)] : 0u;
#pragma unroll
                    for (int i = 0; i < 8; ++i) fm.v[i] = (float)((b >> i) & 1u);
                } else {
                    fm = ld8<FAST, true>(mask, om, e0, nv);
                }
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    g[r][c][i] = fg.v[i];
                    df[r][c][i] = fd.v[i];
                    mk[r][c][i] = (half_t)fm.v[i];
                    s1[r] += g[r][c][i];
                    s2[r] = __fmaf_rn(g[r][c][i], df[r][c][i], s2[r]);
                }
            }
        }
#pragma unroll
        for (int r = 0; r < RPW; ++r) { s1[r] = wave_sum(s1[r]); s2[r] = wave_sum(s2[r]); }
#pragma unroll
        for (int r = 0; r < RPW; ++r) {
            if (row0 + r >= nrows) continue;
            const float c1 = s1[r] * is[r] * invn;
            const float c2 = s2[r] * is[r] * is[r] * is[r] * invn;
            const long o1 = view_offset_of<FLAT>(d_ln_in, ix[r]), o2 = view_offset_of<FLAT>(d_drop_in, ix[r]);
#pragma unroll
            for (int c = 0; c < VPL; ++c) {
                int e0 = (c * WAVE + lane) * 8;
                int nv = nvalid_at(rs.R, e0);
                if (nv > 0) {
                    h8 a, b;
#pragma unroll
                    for (int i = 0; i < 8; ++i) a[i] = (half_t)ln_bwd_value(g[r][c][i], df[r][c][i], is[r], c1, c2);
                    a = pin(a);
#pragma unroll
                    for (int i = 0; i < 8; ++i) b[i] = mk[r][c][i] != (half_t)0.0f ? a[i] : (half_t)0.0f;
                    st8h<FAST>(d_ln_in, o1, e0, nv, a);
                    st8h<FAST>(d_drop_in, o2, e0, nv, b);
                }
            }
        }
    }
}

inline int pick_vpl(int R, const char* what) {
    if (R <= 0) fail(std::string(what) + ": empty row");
    if (R <= 512) return 1;
    if (R <= 1024) return 2;
    if (R <= 2048) return 4;
    if (R <= 4096) return 8;
    fail(std::string(what) + ": rows longer than 4096 elements are not supported");
}

inline int row_grid(long nrows, int rpw) {
    long blocks = (nrows + (long)WPB * rpw - 1) / ((long)WPB * rpw);
    const long cap = 256L * 64;          // 256 CUs; waves beyond this loop
    return (int)(blocks < cap ? (blocks > 0 ? blocks : 1) : cap);
}

inline unsigned check_rows(const RowSpace& rs, const char* what) {
    long n = rs.rows();
    if (n >= (1L << 31)) fail(std::string(what) + ": too many rows");
    return (unsigned)n;
}

}  // namespace

// Dispatch on (VPL, rows per wave, FAST).  Rows per wave: 4 for rows of up to 512
// elements, 2 up to 1024, else 1; the generic (strided) path always takes 1.
// (extra_blocks: workgroups behind those of the rows, for a kernel that has a side job; a
// variable of the calling function.)
#define SUB_ROW_LAUNCH(KERNEL, V, RP, F, ...) \
    hipLaunchKernelGGL((KERNEL<V, RP, F>), dim3(row_grid(nrows, RP) + extra_blocks), dim3(BLOCK), 0, st, __VA_ARGS__)
#define SUB_ROW_LAUNCH_FLAT(KERNEL, V, RP, ...) \
    hipLaunchKernelGGL((KERNEL<V, RP, true, true>), dim3(row_grid(nrows, RP) + extra_blocks), dim3(BLOCK), 0, st, __VA_ARGS__)
// (flat: the fast kernels instantiated for a flat row space, see row_index_of)
#define SUB_ROW_DISPATCH_FLAT(KERNEL, vpl, ...)                                    \
    do {                                                                           \
        const bool many = nrows >= 256u * 16u * 4u;                                \
        switch (vpl) {                                                             \
            case 1: if (many) SUB_ROW_LAUNCH_FLAT(KERNEL, 1, 4, __VA_ARGS__);      \
                    else SUB_ROW_LAUNCH_FLAT(KERNEL, 1, 1, __VA_ARGS__); break;    \
            case 2: if (many) SUB_ROW_LAUNCH_FLAT(KERNEL, 2, 2, __VA_ARGS__);      \
                    else SUB_ROW_LAUNCH_FLAT(KERNEL, 2, 1, __VA_ARGS__); break;    \
            case 4: SUB_ROW_LAUNCH_FLAT(KERNEL, 4, 1, __VA_ARGS__); break;         \
            default: SUB_ROW_LAUNCH_FLAT(KERNEL, 8, 1, __VA_ARGS__); break;        \
        }                                                                          \
    } while (0)
#define SUB_ROW_DISPATCH(KERNEL, vpl, fast, ...)                                   \
    do {                                                                           \
        if (fast) {                                                                \
            /* several rows per wave only while that still leaves >= 16 waves per CU */ \
            const bool many = nrows >= 256u * 16u * 4u;                            \
            switch (vpl) {                                                         \
                case 1: if (many) SUB_ROW_LAUNCH(KERNEL, 1, 4, true, __VA_ARGS__);  \
                        else SUB_ROW_LAUNCH(KERNEL, 1, 1, true, __VA_ARGS__); break; \
                case 2: if (many) SUB_ROW_LAUNCH(KERNEL, 2, 2, true, __VA_ARGS__);  \
                        else SUB_ROW_LAUNCH(KERNEL, 2, 1, true, __VA_ARGS__); break; \
                case 4: SUB_ROW_LAUNCH(KERNEL, 4, 1, true, __VA_ARGS__); break;    \
                default: SUB_ROW_LAUNCH(KERNEL, 8, 1, true, __VA_ARGS__); break;   \
            }                                                                      \
        } else {                                                                   \
            switch (vpl) {                                                         \
                case 1: SUB_ROW_LAUNCH(KERNEL, 1, 1, false, __VA_ARGS__); break;   \
                case 2: SUB_ROW_LAUNCH(KERNEL, 2, 1, false, __VA_ARGS__); break;   \
                case 4: SUB_ROW_LAUNCH(KERNEL, 4, 1, false, __VA_ARGS__); break;   \
                default: SUB_ROW_LAUNCH(KERNEL, 8, 1, false, __VA_ARGS__); break;  \
            }                                                                      \
        }                                                                          \
    } while (0)

void launch_softmax(const RowSpace& rs, View beta, View alpha, View mask, View drop, View amask,
                    float scale, float mscale, PhiloxKey key, hipStream_t st) {
    const unsigned extra_blocks = 0;
    unsigned nrows = check_rows(rs, "softmax");
    if (nrows == 0) return;
    int vpl = pick_vpl(rs.R, "softmax");
    bool fast = beta.vec && alpha.vec && mask.vec && drop.vec;
    const bool masked = amask.p != nullptr;
    if (fast && rs.R <= 256 && nrows >= 256u * 16u * 4u) {
        // short rows: two or four side by side in every wave
#define SUB_SM_SHORT(G, RPS, M)                                                                        \
        hipLaunchKernelGGL((k_softmax<1, 4, true, false, G, M>), dim3(row_grid(nrows, RPS)), dim3(BLOCK), 0, st, rs, \
                           beta, alpha, mask, drop, amask, scale, mscale, key, nrows)
        if (rs.R <= 128) { if (masked) SUB_SM_SHORT(16, 16, true); else SUB_SM_SHORT(16, 16, false); }
        else { if (masked) SUB_SM_SHORT(32, 8, true); else SUB_SM_SHORT(32, 8, false); }
#undef SUB_SM_SHORT
        check_launch("softmax");
        return;
    }
    if (masked) {
        // one row per wave; the mask rows are re-read by every head and sample from cache
#define SUB_SM_MASKED(V, F)                                                                            \
        hipLaunchKernelGGL((k_softmax<V, 1, F, false, WAVE, true>), dim3(row_grid(nrows, 1)), dim3(BLOCK), 0, st, rs, \
                           beta, alpha, mask, drop, amask, scale, mscale, key, nrows)
        switch (vpl) {
            case 1: if (fast) SUB_SM_MASKED(1, true); else SUB_SM_MASKED(1, false); break;
            case 2: if (fast) SUB_SM_MASKED(2, true); else SUB_SM_MASKED(2, false); break;
            case 4: if (fast) SUB_SM_MASKED(4, true); else SUB_SM_MASKED(4, false); break;
            default: if (fast) SUB_SM_MASKED(8, true); else SUB_SM_MASKED(8, false); break;
        }
#undef SUB_SM_MASKED
        check_launch("softmax");
        return;
    }
    if (fast && rs.flat) SUB_ROW_DISPATCH_FLAT(k_softmax, vpl, rs, beta, alpha, mask, drop, amask, scale, mscale, key, nrows);
    else SUB_ROW_DISPATCH(k_softmax, vpl, fast, rs, beta, alpha, mask, drop, amask, scale, mscale, key, nrows);
    check_launch("softmax");
}

void launch_bs(const RowSpace& rs, View alpha, View mask, View ddrop, View dbeta, float scale,
               hipStream_t st) {
    const unsigned extra_blocks = 0;
    unsigned nrows = check_rows(rs, "softmax backward");
    if (nrows == 0) return;
    int vpl = pick_vpl(rs.R, "softmax backward");
    bool fast = alpha.vec && mask.vec && ddrop.vec && dbeta.vec;
    if (fast && rs.R <= 256 && nrows >= 256u * 16u * 4u) {
        if (rs.R <= 128)
            hipLaunchKernelGGL((k_bs<1, 4, true, false, 16>), dim3(row_grid(nrows, 16)), dim3(BLOCK), 0, st, rs, alpha,
                               mask, ddrop, dbeta, scale, nrows);
        else
            hipLaunchKernelGGL((k_bs<1, 4, true, false, 32>), dim3(row_grid(nrows, 8)), dim3(BLOCK), 0, st, rs, alpha,
                               mask, ddrop, dbeta, scale, nrows);
        check_launch("softmax backward");
        return;
    }
    if (fast && rs.flat) SUB_ROW_DISPATCH_FLAT(k_bs, vpl, rs, alpha, mask, ddrop, dbeta, scale, nrows);
    else SUB_ROW_DISPATCH(k_bs, vpl, fast, rs, alpha, mask, ddrop, dbeta, scale, nrows);
    check_launch("softmax backward");
}

void launch_bdrln(const RowSpace& rs, View in, View resid, View lin_bias, View scale, View bias,
                  View lin, View mask, View diff, View normed, View out, View istd, PhiloxKey key,
                  float eps, hipStream_t st, uint8_t* mask_bits, bool write_lin, KeepWordsJob* side) {
    if (mask_bits && rs.R % 8) fail("bias-dropout-residual-layernorm: a bit mask needs rows of whole 8-packs");
    unsigned nrows = check_rows(rs, "bias-dropout-residual-layernorm");
    if (nrows == 0) return;
    int vpl = pick_vpl(rs.R, "bias-dropout-residual-layernorm");
    bool fast = in.vec && resid.vec && lin_bias.vec && scale.vec && bias.vec && lin.vec && (mask.vec || mask_bits) &&
                diff.vec && normed.vec && out.vec;
    // the side job: as many workgroups as draw one lane's words per thread, at most four per CU
    KeepWordsJob job;
    if (side && side->out && side->key.thr && side->M % 256 == 0 && side->N % 256 == 0 && side->M > 0 && side->N > 0 &&
        (uint64_t)side->M * side->N / 8 / 16 <= 0x7fffffffu) {
        job = *side;
        const uint64_t items = (uint64_t)side->M / 256 * (side->N / 256) * 512;
        job.blocks = (uint32_t)((items + BLOCK - 1) / BLOCK < 1024 ? (items + BLOCK - 1) / BLOCK : 1024);
        side->blocks = job.blocks;
    } else if (side) {
        side->blocks = 0;
    }
    const unsigned extra_blocks = job.blocks;
    if (fast && rs.flat && (mask.p || mask_bits) && (lin.p || !write_lin)) {
        const dim3 grid(row_grid(nrows, 1) + extra_blocks);
#define SUB_BDRLN_FLAT(V) hipLaunchKernelGGL((k_bdrln_flat<V>), grid, dim3(BLOCK), 0, st, rs.R, nrows, in, resid, lin_bias, \
                                             scale, bias, lin, mask, diff, normed, out, istd, key, eps, mask_bits, write_lin, job)
        switch (vpl) {
            case 1: SUB_BDRLN_FLAT(1); break;
            case 2: SUB_BDRLN_FLAT(2); break;
            case 4: SUB_BDRLN_FLAT(4); break;
            default: SUB_BDRLN_FLAT(8); break;
        }
#undef SUB_BDRLN_FLAT
        check_launch("bias-dropout-residual-layernorm");
        return;
    }
    SUB_ROW_DISPATCH(k_bdrln, vpl, fast, rs, in, resid, lin_bias, scale, bias, lin, mask, diff, normed,
                     out, istd, key, eps, nrows, mask_bits, write_lin, job);
    check_launch("bias-dropout-residual-layernorm");
}

void launch_blnrd(const RowSpace& rs, View dout, View istd, View diff, View mask, View d_ln_in,
                  View d_drop_in, hipStream_t st, const uint8_t* mask_bits) {
    const unsigned extra_blocks = 0;
    if (mask_bits && rs.R % 8) fail("layernorm backward: a bit mask needs rows of whole 8-packs");
    unsigned nrows = check_rows(rs, "layernorm backward");
    if (nrows == 0) return;
    int vpl = pick_vpl(rs.R, "layernorm backward");
    bool fast = dout.vec && diff.vec && (mask.vec || mask_bits) && d_ln_in.vec && d_drop_in.vec;
    if (fast && rs.flat) SUB_ROW_DISPATCH_FLAT(k_blnrd, vpl, rs, dout, istd, diff, mask, d_ln_in, d_drop_in, nrows, mask_bits);
    else SUB_ROW_DISPATCH(k_blnrd, vpl, fast, rs, dout, istd, diff, mask, d_ln_in, d_drop_in, nrows, mask_bits);
    check_launch("layernorm backward");
}

}  // namespace sub
