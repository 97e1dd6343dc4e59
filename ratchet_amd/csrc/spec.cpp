// Host-side rules of the Matmul operator (see spec.h).  Citations are to the
// reference checkout.
#include "spec.h"

#include <algorithm>

namespace rt {

static void set_why(std::string *why, const std::string &msg) {
    if (why) *why = msg;
}

static std::string shape_str(const Shape &s) {
    std::string r = "[";
    for (size_t i = 0; i < s.size(); i++) r += (i ? "," : "") + std::to_string(s[i]);
    return r + "]";
}

bool is_vector(const Shape &s) {
    // squeeze() drops every dim equal to 1; a vector has at most one left.
    return std::count_if(s.begin(), s.end(), [](int64_t d) { return d != 1; }) <= 1;
}

bool multi_broadcast(const Shape &a, const Shape &b, Shape &out) {
    size_t rank = std::max(a.size(), b.size());
    out.assign(rank, 1);
    for (size_t i = 0; i < rank; i++) {
        int64_t cur = 1;
        for (const Shape *s : {&a, &b}) {
            int64_t d = i < s->size() ? (*s)[s->size() - i - 1] : 1;
            if (d != 1) {
                if (cur != 1 && d != cur) return false;
                cur = d;
            }
        }
        out[rank - i - 1] = cur;
    }
    return true;
}

rt_status compute_c_shape(const Shape &a_in, const Shape &b_in, bool trans_lhs, bool trans_rhs,
                          bool trans_out, Shape &out, std::string *why) {
    Shape a = a_in, b = b_in;
    if (a.empty() || b.empty()) {
        set_why(why, "Matmul: rank-0 operand");
        return RT_ERR_INVALID_SHAPE;
    }
    const bool implicit_m = a.size() < 2, implicit_n = b.size() < 2;
    if (implicit_m) a.insert(a.begin() + (trans_lhs ? 1 : 0), 1);
    if (implicit_n) b.insert(b.begin() + (trans_rhs ? 0 : 1), 1);
    while (a.size() < b.size()) a.insert(a.begin(), 1);
    while (b.size() < a.size()) b.insert(b.begin(), 1);
    const size_t r = a.size();
    Shape prefix;
    if (!multi_broadcast(Shape(a.begin(), a.end() - 2), Shape(b.begin(), b.end() - 2), prefix)) {
        set_why(why, "Matmul broadcasting: a: " + shape_str(a) + " b: " + shape_str(b));
        return RT_ERR_INVALID_SHAPE;
    }
    int64_t m = a[r - 2], ka = a[r - 1], kb = b[r - 2], n = b[r - 1];
    if (trans_lhs) std::swap(m, ka);
    if (trans_rhs) std::swap(kb, n);
    if (ka != kb) {
        set_why(why, "Matmul broadcasting: ka != kb: " + std::to_string(ka) + " != " + std::to_string(kb));
        return RT_ERR_INVALID_SHAPE;
    }
    out = prefix;
    if (trans_out) {
        if (!implicit_n) out.push_back(n);
        if (!implicit_m) out.push_back(m);
    } else {
        if (!implicit_m) out.push_back(m);
        if (!implicit_n) out.push_back(n);
    }
    return RT_OK;
}

// The product of the extents stays below 2^56 (no intermediate overflows: every extent is at most 2^40).
static bool numel_fits(const Shape &s) {
    int64_t n = 1;
    for (int64_t v : s) {
        if (v == 0) return true;
        if (n > (int64_t(1) << 56) / v) return false;
        n *= v;
    }
    return true;
}

static rt_status read_desc(const rt_matmul_desc &d, Shape &a, Shape &b, Shape &bias, std::string *why) {
    if (!valid_dtype(d.lhs_dt) || !valid_dtype(d.rhs_dt) || (d.has_bias && !valid_dtype(d.bias_dt))) {
        set_why(why, "unknown dtype id");
        return RT_ERR_INVALID_ARG;
    }
    if (d.lhs_rank < 0 || d.lhs_rank > RT_MAX_RANK || d.rhs_rank < 0 || d.rhs_rank > RT_MAX_RANK ||
        (d.has_bias && (d.bias_rank < 0 || d.bias_rank > RT_MAX_RANK))) {
        set_why(why, "rank out of range");
        return RT_ERR_INVALID_ARG;
    }
    a.assign(d.lhs_shape, d.lhs_shape + d.lhs_rank);
    b.assign(d.rhs_shape, d.rhs_shape + d.rhs_rank);
    bias.clear();
    if (d.has_bias) bias.assign(d.bias_shape, d.bias_shape + d.bias_rank);
    for (const Shape *s : {&a, &b, &bias})
        for (int64_t v : *s)
            if (v < 0 || v > (int64_t(1) << 40)) {
                set_why(why, "dimension out of range");
                return RT_ERR_INVALID_ARG;
            }
    // element counts (and every offset derived from them) must stay far inside int64
    for (const Shape *s : {&a, &b})
        if (!numel_fits(*s)) {
            set_why(why, "tensor of more than 2^56 elements");
            return RT_ERR_INVALID_ARG;
        }
    return RT_OK;
}

// Allowed (lhs, rhs) pairs.  The first four are the reference's
// (ops/matmul.rs:454-467).  (Q4_K, F16) is this library's extension, and so
// is each mirrored pair, where the activations are the lhs and the quantized
// weight is the rhs read with trans_rhs ("x . W^T" spelled directly).
static bool pair_allowed(int lhs, int rhs) {
    if (is_float(lhs) && lhs == rhs) return true;
    if (is_quantized(lhs) && rhs == activation_dt(lhs)) return true;
    if (is_quantized(rhs) && lhs == activation_dt(rhs)) return true;
    return false;
}

rt_status validate(const rt_matmul_desc &d, std::string *why) {
    Shape a, b, bias, c;
    rt_status st = read_desc(d, a, b, bias, why);
    if (st != RT_OK) return st;
    // Matmul::new (ops/matmul.rs:258-272)
    if (d.has_bias && !is_vector(bias)) {
        set_why(why, "Bias must be a vector: " + shape_str(bias));
        return RT_ERR_INVALID_SHAPE;
    }
    if (is_quantized(d.lhs_dt) && d.trans_lhs) {
        set_why(why, "Transposed quantized inputs are not supported");
        return RT_ERR_UNSUPPORTED;
    }
    // OpGuards::check_shapes (ops/matmul.rs:442-451)
    st = compute_c_shape(a, b, d.trans_lhs, d.trans_rhs, d.trans_out, c, why);
    if (st != RT_OK) return st;
    if (!numel_fits(c)) {
        set_why(why, "output of more than 2^56 elements");
        return RT_ERR_INVALID_ARG;
    }
    // OpGuards::check_dtypes (ops/matmul.rs:453-478)
    if (!pair_allowed(d.lhs_dt, d.rhs_dt)) {
        set_why(why, "Failed to validate DTypes: lhs " + std::to_string(d.lhs_dt) + ", rhs " +
                         std::to_string(d.rhs_dt));
        return RT_ERR_DTYPE_MISMATCH;
    }
    const int act = is_quantized(d.rhs_dt) ? activation_dt(d.rhs_dt) : d.rhs_dt;
    if (d.has_bias && d.bias_dt != act) {
        set_why(why, "Failed to validate DTypes: bias " + std::to_string(d.bias_dt) + ", activation " +
                         std::to_string(act));
        return RT_ERR_DTYPE_MISMATCH;
    }
    // GEMMSpec::new (ops/matmul.rs:67-69)
    if (a.size() < 2 || b.size() < 2) {
        set_why(why, "MatMul: inputs must be at least 2D");
        return RT_ERR_INVALID_SHAPE;
    }
    if (is_quantized(d.rhs_dt) && !d.trans_rhs) {
        set_why(why, "a quantized rhs must be read with trans_rhs (weights stored [N, K])");
        return RT_ERR_UNSUPPORTED;
    }
    // GEMMSpec::new stack rule (ops/matmul.rs:83-94)
    const size_t rank = std::max(a.size(), b.size());
    Shape ap = a, bp = b;
    while (ap.size() < rank) ap.insert(ap.begin(), 1);
    while (bp.size() < rank) bp.insert(bp.begin(), 1);
    const size_t sd = c.size() - 2;
    const int64_t ls = numel(Shape(ap.begin(), ap.begin() + sd));
    const int64_t rs = numel(Shape(bp.begin(), bp.begin() + sd));
    const int64_t os = numel(Shape(c.begin(), c.begin() + sd));
    if (ls != 1 && rs != 1 && !(ls == rs && rs == os)) {
        set_why(why, "operand stacks must be equal, or one of them 1: lhs " + std::to_string(ls) + " rhs " +
                         std::to_string(rs) + " out " + std::to_string(os));
        return RT_ERR_INVALID_SHAPE;
    }
    int64_t m = ap[rank - 2], k = ap[rank - 1], n = bp[rank - 1];
    if (d.trans_lhs) std::swap(m, k);
    if (d.trans_rhs) n = bp[rank - 2];
    // Blocks of a quantized operand must not straddle its rows.
    const int qdt = is_quantized(d.lhs_dt) ? d.lhs_dt : d.rhs_dt;
    if (is_quantized(qdt) && k % block_numel(qdt) != 0) {
        set_why(why, "K = " + std::to_string(k) + " is not a multiple of the quantization block (" +
                         std::to_string(block_numel(qdt)) + ")");
        return RT_ERR_UNSUPPORTED;
    }
    // Bias indexes the lhs rows under trans_out, else the output columns
    // (ops/gemm.rs:466-476, ops/gemv.rs:310-314).
    if (d.has_bias) {
        const int64_t want = d.trans_out ? m : n;
        if (numel(bias) != want) {
            set_why(why, "bias has " + std::to_string(numel(bias)) + " elements, expected " + std::to_string(want));
            return RT_ERR_INVALID_SHAPE;
        }
    }
    return RT_OK;
}

rt_status infer(const rt_matmul_desc &d, Shape &out, int &out_dt, std::string *why) {
    Shape a, b, bias;
    rt_status st = read_desc(d, a, b, bias, why);
    if (st != RT_OK) return st;
    st = compute_c_shape(a, b, d.trans_lhs, d.trans_rhs, d.trans_out, out, why);
    if (st != RT_OK) return st;
    // Matmul::compute_view: dtype = rhs dtype (ops/matmul.rs:437); a quantized
    // rhs (extension) yields its activation dtype.
    out_dt = is_quantized(d.rhs_dt) ? activation_dt(d.rhs_dt) : d.rhs_dt;
    return RT_OK;
}

static int pick_kernel(const Problem &p) {
    if (p.stacks * p.M * p.N == 0) return RT_KERNEL_NONE;
    const bool b_kcontig = p.b_ks == 1 || p.K == 1;
    switch (p.a_dt) {
    case RT_Q8_0F:
    case RT_Q8_0H:
        if (p.N <= (p.a_dt == RT_Q8_0H ? kGemvQ8hMaxCols : kGemvMaxCols) && b_kcontig) return RT_KERNEL_GEMV_Q8;
        return p.a_dt == RT_Q8_0H ? RT_KERNEL_GEMM_F16 : RT_KERNEL_GEMM_F32;
    case RT_Q4_K:
        if (p.N <= kGemvQ4kMaxCols && b_kcontig) return RT_KERNEL_GEMV_Q4K;
        return RT_KERNEL_GEMM_F16;
    default:
        if (p.N <= kGemvMaxCols && b_kcontig && (p.a_ks == 1 || p.K == 1)) return RT_KERNEL_GEMV_FLOAT;
        return p.a_dt == RT_F16 ? RT_KERNEL_GEMM_F16 : RT_KERNEL_GEMM_F32;
    }
}

rt_status make_spec(const rt_matmul_desc &d, rt_gemm_spec &spec, Problem &p, std::string *why) {
    rt_status st = validate(d, why);
    if (st != RT_OK) return st;
    Shape a(d.lhs_shape, d.lhs_shape + d.lhs_rank), b(d.rhs_shape, d.rhs_shape + d.rhs_rank), c;
    compute_c_shape(a, b, d.trans_lhs, d.trans_rhs, d.trans_out, c, nullptr);
    const size_t rank = std::max(a.size(), b.size());
    while (a.size() < rank) a.insert(a.begin(), 1);
    while (b.size() < rank) b.insert(b.begin(), 1);
    const size_t sd = c.size() - 2;

    spec = rt_gemm_spec{};
    spec.lhs_stack = numel(Shape(a.begin(), a.begin() + sd));
    spec.rhs_stack = numel(Shape(b.begin(), b.begin() + sd));
    spec.out_stack = numel(Shape(c.begin(), c.begin() + sd));
    spec.lhs_shape[0] = a[rank - 2], spec.lhs_shape[1] = a[rank - 1];
    spec.rhs_shape[0] = b[rank - 2], spec.rhs_shape[1] = b[rank - 1];
    spec.out_shape[0] = c[sd], spec.out_shape[1] = c[sd + 1];
    spec.dim_lhs_outer = spec.out_shape[0];
    spec.dim_rhs_outer = spec.out_shape[1];
    spec.dim_inner = d.trans_lhs ? spec.lhs_shape[0] : spec.lhs_shape[1];
    // GEMVHeuristic (ops/matmul.rs:112-117)
    const int64_t arows = spec.lhs_shape[0], acols = spec.lhs_shape[1];
    if (arows > acols * 4) spec.heuristic = RT_HEUR_VERY_TALL;
    else if (arows > acols * 2) spec.heuristic = RT_HEUR_TALL;
    else if (acols > arows * 2) spec.heuristic = RT_HEUR_FAT;
    else spec.heuristic = RT_HEUR_SQUARE;
    // GEMMSpec::is_gemv (ops/matmul.rs:221-223)
    spec.is_gemv = is_vector(Shape{spec.rhs_shape[0], spec.rhs_shape[1]}) && !d.trans_lhs;

    // Lower to the strided problem.
    const int64_t ar = spec.lhs_shape[0], ac = spec.lhs_shape[1];
    const int64_t br = spec.rhs_shape[0], bc = spec.rhs_shape[1];
    const int64_t m = d.trans_lhs ? ac : ar, k = spec.dim_inner, n = d.trans_rhs ? br : bc;
    p = Problem{};
    p.stacks = spec.out_stack;
    p.K = k;
    p.has_bias = d.has_bias != 0;
    p.act_dt = is_quantized(d.rhs_dt) ? activation_dt(d.rhs_dt) : d.rhs_dt;
    // strides of op(lhs)[i,k] and op(rhs)[k,j] in their own buffers
    const int64_t l_is = d.trans_lhs ? 1 : ac, l_ks = d.trans_lhs ? ac : 1;
    const int64_t r_ks = d.trans_rhs ? 1 : bc, r_js = d.trans_rhs ? bc : 1;
    const int64_t out_i = d.trans_out ? 1 : n, out_j = d.trans_out ? m : 1; // out[m,n] or out[n,m]
    bool swap = is_quantized(d.rhs_dt);
    // Both operands plain floats with few lhs rows and many rhs columns, all
    // K-contiguous: stream the rhs as the row operand of the GEMV kernel.
    if (!swap && is_float(d.lhs_dt) && m <= kGemvMaxCols && n > kGemvMaxCols && (l_ks == 1 || k == 1) &&
        (r_ks == 1 || k == 1))
        swap = true;
    if (!swap) {
        p.a_dt = d.lhs_dt;
        p.M = m, p.N = n;
        p.a_stack = spec.lhs_stack, p.b_stack = spec.rhs_stack;
        p.a_bs = ar * ac, p.a_rs = l_is, p.a_ks = l_ks;
        p.b_bs = br * bc, p.b_ks = r_ks, p.b_js = r_js;
        p.o_is = out_i, p.o_js = out_j;
        p.bias_on_rows = d.trans_out != 0;
    } else {
        p.swapped = true;
        p.a_dt = d.rhs_dt;
        p.M = n, p.N = m;
        p.a_stack = spec.rhs_stack, p.b_stack = spec.lhs_stack;
        p.a_bs = br * bc, p.a_rs = r_js, p.a_ks = r_ks;
        p.b_bs = ar * ac, p.b_ks = l_ks, p.b_js = l_is;
        p.o_is = out_j, p.o_js = out_i;
        p.bias_on_rows = d.trans_out == 0;
    }
    p.o_bs = m * n;
    p.kernel = pick_kernel(p);
    spec.kernel = p.kernel;
    return RT_OK;
}

} // namespace rt
