// Shared host-side definitions: dimension ids, error reporting, layout algebra.
#pragma once

#include <cstdint>
#include <cstdio>
#include <cstring>
#include <stdexcept>
#include <string>
#include <vector>

namespace sub {

// Logical dimensions of the encoder layer (pytorch_module/encoder.py:43-53):
// B batch, J query position, K key position, H heads, P head size,
// I embedding, U feed-forward width, Q stack index (0=K, 1=Q, 2=V).
enum Dim { dB = 0, dJ, dK, dH, dP, dI, dU, dQ, NDIM };

inline int dim_of(char c) {
    switch (c) {
        case 'B': return dB; case 'J': return dJ; case 'K': return dK; case 'H': return dH;
        case 'P': return dP; case 'I': return dI; case 'U': return dU; case 'Q': return dQ;
        case 'S': return dJ;   // the reference's sizes map also names the sequence length 'S'
        default: return -1;
    }
}
inline char dim_char(int d) { return "BJKHPIUQ"[d]; }

struct Error : std::runtime_error {
    using std::runtime_error::runtime_error;
};

[[noreturn]] inline void fail(const std::string& msg) { throw Error(msg); }

struct Sizes {
    int64_t n[NDIM] = {0, 0, 0, 0, 0, 0, 0, 3};
};

// A dense row-major tensor whose dimension order is a permutation string.
// stride(d) = product of the sizes after d (pytorch_module/metahelpers.h:61-78);
// dims that do not occur have stride 0 and has[d] == false.
struct Layout {
    int rank = 0;
    int dims[NDIM] = {0};
    int64_t size[NDIM] = {0};     // per logical dim; 1 for absent dims
    int64_t stride[NDIM] = {0};   // per logical dim; 0 for absent dims
    bool has[NDIM] = {false};
    int64_t numel = 1;

    int pos(int d) const {
        for (int i = 0; i < rank; ++i) if (dims[i] == d) return i;
        return -1;
    }
    std::string str() const {
        std::string s;
        for (int i = 0; i < rank; ++i) s.push_back(dim_char(dims[i]));
        return s;
    }
};

inline Layout make_layout(const char* s, const Sizes& sz) {
    Layout l;
    if (!s) fail("layout string is null");
    size_t n = std::strlen(s);
    if (n > NDIM) fail(std::string("layout too long: ") + s);
    for (int d = 0; d < NDIM; ++d) l.size[d] = 1;
    for (size_t i = 0; i < n; ++i) {
        int d = dim_of(s[i]);
        if (d < 0) fail(std::string("unknown dimension letter in layout: ") + s);
        if (l.has[d]) fail(std::string("repeated dimension in layout: ") + s);
        if (sz.n[d] <= 0) fail(std::string("size of a dimension is not set for layout: ") + s);
        l.has[d] = true;
        l.dims[l.rank++] = d;
        l.size[d] = sz.n[d];
    }
    int64_t st = 1;
    for (int i = l.rank - 1; i >= 0; --i) {
        l.stride[l.dims[i]] = st;
        st *= l.size[l.dims[i]];
    }
    l.numel = st;
    return l;
}

// Rename a dimension (the reference's K/V views of J-indexed tensors,
// pytorch_module/encoder.py:339-347).
inline Layout rename_dim(const Layout& in, int from, int to) {
    if (!in.has[from]) return in;
    if (in.has[to]) fail("rename_dim: target dimension already present");
    Layout l = in;
    for (int i = 0; i < l.rank; ++i) if (l.dims[i] == from) l.dims[i] = to;
    l.has[to] = true; l.has[from] = false;
    l.size[to] = in.size[from]; l.size[from] = 1;
    l.stride[to] = in.stride[from]; l.stride[from] = 0;
    return l;
}

// Drop the outermost dimension (sub-tensor of a Q-stacked tensor).
inline Layout drop_front(const Layout& in, int d) {
    if (in.rank == 0 || in.dims[0] != d)
        fail(std::string("layout must start with ") + dim_char(d) + ": " + in.str());
    Layout l = in;
    for (int i = 1; i < in.rank; ++i) l.dims[i - 1] = in.dims[i];
    l.rank = in.rank - 1;
    l.numel = in.numel / in.size[d];
    l.has[d] = false; l.size[d] = 1; l.stride[d] = 0;
    return l;
}

// ---------------------------------------------------------------------------
// Einsum -> batched GEMM parameters (pytorch_module/einsumparser.h:9-55,
// gemm.cuh:52-61).  Generalised: up to three batch dimensions with their own
// strides (0 where an operand lacks the dimension) and a contraction that may
// be split into an outer and an inner merged group.
// ---------------------------------------------------------------------------
struct GemmShape {
    int64_t M = 1, N = 1, K0 = 1, K1 = 1;          // K = K0 * K1
    int64_t sAM = 0, sAK1 = 0, sAK0 = 0;
    int64_t sBN = 0, sBK1 = 0, sBK0 = 0;
    int64_t sCM = 0, sCN = 0;
    int nbatch = 0;
    int64_t nb[3] = {1, 1, 1};
    int64_t sAb[3] = {0, 0, 0}, sBb[3] = {0, 0, 0}, sCb[3] = {0, 0, 0};
    // logical dims of the M group, the N group (outer to inner) and the batch dims
    int nmd = 0, nnd = 0;
    int mdims[NDIM] = {0}, ndims[NDIM] = {0}, bdims[3] = {0, 0, 0};
    int64_t batch() const { return nb[0] * nb[1] * nb[2]; }
    int64_t K() const { return K0 * K1; }
};

namespace detail {
// True if the dims in g (given in the order of tensor t) are adjacent in t.
inline bool adjacent_in(const std::vector<int>& g, const Layout& t) {
    if (g.empty()) return true;
    int p0 = t.pos(g[0]);
    for (size_t i = 0; i < g.size(); ++i) if (t.pos(g[i]) != p0 + (int)i) return false;
    return true;
}
inline std::vector<int> ordered_by(const std::vector<int>& g, const Layout& t) {
    std::vector<int> r;
    for (int i = 0; i < t.rank; ++i)
        for (int d : g) if (d == t.dims[i]) r.push_back(d);
    return r;
}
// A group is mergeable over tensors t1,t2 when it is adjacent and identically
// ordered in both: then one stride (that of its last member) addresses it.
inline bool mergeable(const std::vector<int>& g, const Layout& t1, const Layout& t2) {
    auto o1 = ordered_by(g, t1), o2 = ordered_by(g, t2);
    return o1 == o2 && adjacent_in(o1, t1) && adjacent_in(o2, t2);
}
inline int64_t prod(const std::vector<int>& g, const Layout& t) {
    int64_t p = 1;
    for (int d : g) p *= t.size[d];
    return p;
}
inline int64_t group_stride(const std::vector<int>& g, const Layout& t) {
    if (g.empty()) return 1;          // einsumparser.h / metahelpers.h: empty group -> 1
    return t.stride[ordered_by(g, t).back()];
}
}  // namespace detail

inline GemmShape classify_einsum(const Layout& A, const Layout& B, const Layout& C) {
    using namespace detail;
    std::vector<int> batch, mg, ng, kg;
    for (int d = 0; d < NDIM; ++d) {
        bool a = A.has[d], b = B.has[d], c = C.has[d];
        if (a && b && c) batch.push_back(d);
        else if (a && b) kg.push_back(d);
        else if (a && c) mg.push_back(d);
        else if (b && c) ng.push_back(d);
        else if (a || b || c)
            fail(std::string("einsum: dimension ") + dim_char(d) + " occurs in only one operand");
    }
    for (int d : batch)
        if (A.size[d] != B.size[d] || A.size[d] != C.size[d]) fail("einsum: size mismatch");
    GemmShape g;
    // Peel outer dims of M / N (in the order of C) into batch dims until the
    // rest is mergeable.
    auto peel = [&](std::vector<int>& grp, const Layout& T) {
        grp = ordered_by(grp, C);
        while (!grp.empty() && !mergeable(grp, T, C)) {
            batch.push_back(grp.front());
            grp.erase(grp.begin());
        }
    };
    peel(mg, A);
    peel(ng, B);
    if (batch.size() > 3) fail("einsum: more than three batch dimensions after splitting");
    // batch dims ordered by their position in C (outermost first)
    batch = ordered_by(batch, C);
    g.nbatch = (int)batch.size();
    for (int i = 0; i < g.nbatch; ++i) {
        int d = batch[i];
        g.nb[i] = C.size[d];
        g.sAb[i] = A.has[d] ? A.stride[d] : 0;
        g.sBb[i] = B.has[d] ? B.stride[d] : 0;
        g.sCb[i] = C.stride[d];
    }
    for (int i = 0; i < g.nbatch; ++i) g.bdims[i] = batch[i];
    mg = ordered_by(mg, C); ng = ordered_by(ng, C);
    g.nmd = (int)mg.size(); g.nnd = (int)ng.size();
    for (int i = 0; i < g.nmd; ++i) g.mdims[i] = mg[i];
    for (int i = 0; i < g.nnd; ++i) g.ndims[i] = ng[i];
    g.M = prod(mg, A); g.sAM = group_stride(mg, A); g.sCM = group_stride(mg, C);
    g.N = prod(ng, B); g.sBN = group_stride(ng, B); g.sCN = group_stride(ng, C);
    // contraction: one merged group, or an outer + inner split
    kg = ordered_by(kg, A);
    if (kg.empty()) fail("einsum: no contraction dimension");
    if (mergeable(kg, A, B)) {
        g.K1 = prod(kg, A); g.sAK1 = group_stride(kg, A); g.sBK1 = group_stride(kg, B);
    } else {
        bool ok = false;
        for (size_t cut = 1; cut < kg.size() && !ok; ++cut) {
            std::vector<int> g0(kg.begin(), kg.begin() + cut), g1(kg.begin() + cut, kg.end());
            if (mergeable(g0, A, B) && mergeable(g1, A, B)) {
                g.K0 = prod(g0, A); g.sAK0 = group_stride(g0, A); g.sBK0 = group_stride(g0, B);
                g.K1 = prod(g1, A); g.sAK1 = group_stride(g1, A); g.sBK1 = group_stride(g1, B);
                ok = true;
            }
        }
        if (!ok) fail("einsum: contraction dimensions are not contiguous in " + A.str() + " / " + B.str());
    }
    return g;
}

// Strides of a tensor T (its dims a subset of C's) along the M, N and batch
// indices of a classified contraction, so that T can be added to C in the GEMM
// epilogue.  False when a merged group does not map to a single stride of T.
inline bool addend_strides(const GemmShape& g, const Layout& T, const Layout& C, int64_t& sM, int64_t& sN,
                           int64_t (&sb)[3]) {
    auto group = [&](const int* dims, int n, int64_t& out) {
        // dims outer -> inner; present dims must chain like a dense sub-block,
        // absent ones must all be absent (broadcast)
        int present = 0;
        for (int i = 0; i < n; ++i) present += T.has[dims[i]] ? 1 : 0;
        if (present == 0) { out = 0; return true; }
        if (present != n) return false;
        for (int i = 0; i + 1 < n; ++i)
            if (T.stride[dims[i]] != C.size[dims[i + 1]] * T.stride[dims[i + 1]]) return false;
        out = n ? T.stride[dims[n - 1]] : 0;
        return true;
    };
    if (!group(g.mdims, g.nmd, sM) || !group(g.ndims, g.nnd, sN)) return false;
    int covered = 0;
    for (int i = 0; i < 3; ++i) sb[i] = 0;
    for (int i = 0; i < g.nbatch; ++i) {
        sb[i] = T.has[g.bdims[i]] ? T.stride[g.bdims[i]] : 0;
        covered += T.has[g.bdims[i]] ? 1 : 0;
    }
    for (int i = 0; i < g.nmd; ++i) covered += T.has[g.mdims[i]] ? 1 : 0;
    for (int i = 0; i < g.nnd; ++i) covered += T.has[g.ndims[i]] ? 1 : 0;
    return covered == T.rank;     // every dim of T is one of C's free or batch dims
}

}  // namespace sub
