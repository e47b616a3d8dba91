// CPU restatement, as C++ / OpenMP loop nests, of one BERT encoder layer forward + backward.
//
// TEST AND MEASUREMENT INFRASTRUCTURE ONLY: the timed CPU baseline of bench.py and a second opinion for the NumPy
// oracle. Nothing in the library or the Python package uses it.
//
// It writes out what the reference's "pure" expansions denote once DaCe has compiled them for the CPU: every NumPy
// statement of an expansion (daceml/onnx/op_implementations/pure_implementations.py - Add/Sub/Mul/Div :34-93,
// Erf :106-108, ReduceMean / ReduceSum :101-103,294-306, Softmax :309-319, Transpose, MatMul / Einsum :135-239) is
// one parallel map or one parallel reduction over a materialised temporary, in fp32, in the statement order of
// oracle/bert_layer.py (which follows the opset-12 export of HuggingFace's BertLayer,
// tests/torch/test_bert_encoder.py:13-52). The backward applies the reference's reverse nodes in the same style
// (DefaultEinsumBackward / DefaultSoftmaxBackward, daceml/autodiff/implementations/onnx_ops.py:25-138,237-275, and
// the reversed LayerNorm / GELU maps). Contractions are a cache-blocked OpenMP loop nest: the stand-in for the BLAS
// library node that `set_fast_implementations` (daceml/util/utils.py:226-229) selects on a machine without one to
// link against.
//
// Pinned by tests/test_oracle.py against oracle/bert_layer.py in fp64 (itself pinned against transformers' BertLayer
// and torch.autograd).
#include <algorithm>
#include <cmath>
#include <cstddef>
#include <cstdint>
#include <vector>

#include <omp.h>

namespace {

typedef std::vector<float> Buf;
typedef int64_t i64;

// ------------------------------------------------------------------------------------------------ maps and reductions
template <class F>
void map(float* out, i64 n, F f) {
#pragma omp parallel for schedule(static)
    for (i64 i = 0; i < n; ++i) out[i] = f(i);
}

// out[r, c] = f(r, c) over a [rows, cols] iteration space (row operand broadcasts are indexed by r, vectors by c)
template <class F>
void map2(float* out, i64 rows, i64 cols, F f) {
#pragma omp parallel for schedule(static)
    for (i64 r = 0; r < rows; ++r) {
        float* o = out + r * cols;
        for (i64 c = 0; c < cols; ++c) o[c] = f(r, c);
    }
}

// out[r] = reduction over the row
template <class F>
void reduce_rows(float* out, const float* in, i64 rows, i64 cols, float init, F f, float scale = 1.f) {
#pragma omp parallel for schedule(static)
    for (i64 r = 0; r < rows; ++r) {
        const float* p = in + r * cols;
        float acc = init;
        for (i64 c = 0; c < cols; ++c) acc = f(acc, p[c]);
        out[r] = acc * scale;
    }
}

// out[c] = sum over rows (ReduceSum over the leading axes)
void sum_columns(float* out, const float* in, i64 rows, i64 cols) {
#pragma omp parallel for schedule(static)
    for (i64 c0 = 0; c0 < cols; c0 += 64) {
        const i64 c1 = std::min(cols, c0 + 64);
        float acc[64] = {0};
        for (i64 r = 0; r < rows; ++r)
            for (i64 c = c0; c < c1; ++c) acc[c - c0] += in[r * cols + c];
        for (i64 c = c0; c < c1; ++c) out[c] = acc[c - c0];
    }
}

// Transpose of the last two axes of [batch, rows, cols]
void transpose_last2(float* out, const float* in, i64 batch, i64 rows, i64 cols) {
#pragma omp parallel for collapse(2) schedule(static)
    for (i64 b = 0; b < batch; ++b)
        for (i64 r0 = 0; r0 < rows; r0 += 32)
            for (i64 c0 = 0; c0 < cols; c0 += 32)
                for (i64 r = r0; r < std::min(rows, r0 + 32); ++r)
                    for (i64 c = c0; c < std::min(cols, c0 + 32); ++c)
                        out[(b * cols + c) * rows + r] = in[(b * rows + r) * cols + c];
}

// Transpose(perm = 0, 2, 1, 3) of [d0, d1, d2, d3] -> [d0, d2, d1, d3] (head split and merge)
void transpose_0213(float* out, const float* in, i64 d0, i64 d1, i64 d2, i64 d3) {
#pragma omp parallel for collapse(2) schedule(static)
    for (i64 a = 0; a < d0; ++a)
        for (i64 c = 0; c < d2; ++c)
            for (i64 b = 0; b < d1; ++b) {
                const float* src = in + ((a * d1 + b) * d2 + c) * d3;
                float* dst = out + ((a * d2 + c) * d1 + b) * d3;
                for (i64 e = 0; e < d3; ++e) dst[e] = src[e];
            }
}

// ------------------------------------------------------------------------------------------------ contraction
// C[b] = A[b] (M x K, row-major) * B[b] (K x N, row-major), batch matrices contiguous. Blocked for cache; every tile of
// C is owned by one thread, which walks K in blocks with a 4 x 16 register tile.
const i64 MB = 64, NB = 128, KB = 256, MR = 4, NR = 16;

void tile_product(const float* A, const float* B, float* C, i64 N, i64 K, i64 m0, i64 m1, i64 n0, i64 n1) {
    for (i64 k0 = 0; k0 < K; k0 += KB) {
        const i64 k1 = std::min(K, k0 + KB);
        for (i64 i0 = m0; i0 < m1; i0 += MR) {
            const i64 mr = std::min(MR, m1 - i0);
            for (i64 j0 = n0; j0 < n1; j0 += NR) {
                const i64 nr = std::min(NR, n1 - j0);
                float acc[MR][NR];
                for (i64 r = 0; r < MR; ++r)
                    for (i64 c = 0; c < NR; ++c) acc[r][c] = (k0 == 0 || r >= mr || c >= nr) ? 0.f : C[(i0 + r) * N + j0 + c];
                if (mr == MR && nr == NR) {
                    for (i64 k = k0; k < k1; ++k) {
                        const float* b = B + k * N + j0;
                        const float a0 = A[(i0 + 0) * K + k], a1 = A[(i0 + 1) * K + k], a2 = A[(i0 + 2) * K + k],
                                    a3 = A[(i0 + 3) * K + k];
#pragma omp simd
                        for (i64 c = 0; c < NR; ++c) {
                            acc[0][c] += a0 * b[c];
                            acc[1][c] += a1 * b[c];
                            acc[2][c] += a2 * b[c];
                            acc[3][c] += a3 * b[c];
                        }
                    }
                } else {
                    for (i64 k = k0; k < k1; ++k)
                        for (i64 r = 0; r < mr; ++r) {
                            const float a = A[(i0 + r) * K + k];
                            for (i64 c = 0; c < nr; ++c) acc[r][c] += a * B[k * N + j0 + c];
                        }
                }
                for (i64 r = 0; r < mr; ++r)
                    for (i64 c = 0; c < nr; ++c) C[(i0 + r) * N + j0 + c] = acc[r][c];
            }
        }
    }
}

void matmul(float* C, const float* A, const float* B, i64 batch, i64 M, i64 N, i64 K) {
    const i64 tm = (M + MB - 1) / MB, tn = (N + NB - 1) / NB;
#pragma omp parallel for collapse(3) schedule(dynamic, 1)
    for (i64 b = 0; b < batch; ++b)
        for (i64 ti = 0; ti < tm; ++ti)
            for (i64 tj = 0; tj < tn; ++tj)
                tile_product(A + b * M * K, B + b * K * N, C + b * M * N, N, K, ti * MB, std::min(M, ti * MB + MB), tj * NB,
                             std::min(N, tj * NB + NB));
}

// ------------------------------------------------------------------------------------------------ node chains
// Transpose(W) -> MatMul -> Add(bias, .): x [T, I], w [O, I], b [O] -> [T, O]
void linear(Buf& out, const float* x, const float* w, const float* b, i64 T, i64 I, i64 O) {
    Buf wt(I * O), mm(T * O);
    transpose_last2(wt.data(), w, 1, O, I);
    matmul(mm.data(), x, wt.data(), 1, T, O, I);
    out.resize(T * O);
    const float* m = mm.data();
    map2(out.data(), T, O, [=](i64 r, i64 c) { return b[c] + m[r * O + c]; });
}

// ReduceMean, Sub, Pow, ReduceMean, Add, Sqrt, Div, Mul, Add
void layernorm_chain(Buf& y, const float* x, const float* gamma, const float* beta, i64 rows, i64 cols, float eps) {
    Buf mean(rows), centered(rows * cols), squared(rows * cols), var(rows), shifted(rows), stddev(rows), normed(rows * cols),
        scaled(rows * cols);
    auto add = [](float a, float v) { return a + v; };
    reduce_rows(mean.data(), x, rows, cols, 0.f, add, 1.f / cols);
    const float *mu = mean.data(), *ce = centered.data(), *sq = squared.data(), *va = var.data(), *sh = shifted.data(),
                *sd = stddev.data(), *no = normed.data(), *sc = scaled.data();
    map2(centered.data(), rows, cols, [=](i64 r, i64 c) { return x[r * cols + c] - mu[r]; });
    map(squared.data(), rows * cols, [=](i64 i) { return ce[i] * ce[i]; });
    reduce_rows(var.data(), sq, rows, cols, 0.f, add, 1.f / cols);
    map(shifted.data(), rows, [=](i64 i) { return va[i] + eps; });
    map(stddev.data(), rows, [=](i64 i) { return std::sqrt(sh[i]); });
    map2(normed.data(), rows, cols, [=](i64 r, i64 c) { return ce[r * cols + c] / sd[r]; });
    map2(scaled.data(), rows, cols, [=](i64 r, i64 c) { return no[r * cols + c] * gamma[c]; });
    y.resize(rows * cols);
    map2(y.data(), rows, cols, [=](i64 r, i64 c) { return sc[r * cols + c] + beta[c]; });
}

// the reversed LayerNorm maps: dx, dgamma [cols], dbeta [cols]
void layernorm_backward(Buf& dx, float* dgamma, float* dbeta, const float* dy, const float* x, const float* gamma, i64 rows,
                        i64 cols, float eps) {
    const i64 n = rows * cols;
    Buf mean(rows), centered(n), squared(n), var(rows), rstd(rows), xhat(n), t1(n), g(n), gm(rows), t2(n), gxm(rows);
    auto add = [](float a, float v) { return a + v; };
    reduce_rows(mean.data(), x, rows, cols, 0.f, add, 1.f / cols);
    const float *mu = mean.data(), *ce = centered.data(), *sq = squared.data(), *va = var.data(), *rs = rstd.data(),
                *xh = xhat.data(), *gp = g.data(), *gmp = gm.data(), *gxp = gxm.data();
    map2(centered.data(), rows, cols, [=](i64 r, i64 c) { return x[r * cols + c] - mu[r]; });
    map(squared.data(), n, [=](i64 i) { return ce[i] * ce[i]; });
    reduce_rows(var.data(), sq, rows, cols, 0.f, add, 1.f / cols);
    map(rstd.data(), rows, [=](i64 i) { return 1.f / std::sqrt(va[i] + eps); });
    map2(xhat.data(), rows, cols, [=](i64 r, i64 c) { return ce[r * cols + c] * rs[r]; });
    map(t1.data(), n, [=](i64 i) { return dy[i] * xh[i]; });
    sum_columns(dgamma, t1.data(), rows, cols);
    sum_columns(dbeta, dy, rows, cols);
    map2(g.data(), rows, cols, [=](i64 r, i64 c) { return dy[r * cols + c] * gamma[c]; });
    reduce_rows(gm.data(), gp, rows, cols, 0.f, add, 1.f / cols);
    map(t2.data(), n, [=](i64 i) { return gp[i] * xh[i]; });
    reduce_rows(gxm.data(), t2.data(), rows, cols, 0.f, add, 1.f / cols);
    dx.resize(n);
    map2(dx.data(), rows, cols, [=](i64 r, i64 c) {
        const i64 i = r * cols + c;
        return (gp[i] - gmp[r] - xh[i] * gxp[r]) * rs[r];
    });
}

// Div(x, sqrt 2), Erf, Add 1, Mul x, Mul 0.5
void gelu_chain(Buf& out, const float* x, i64 n) {
    Buf scaled(n), e(n), shifted(n), prod(n);
    const float *sc = scaled.data(), *ep = e.data(), *sh = shifted.data(), *pr = prod.data();
    const float root2 = std::sqrt(2.f);
    map(scaled.data(), n, [=](i64 i) { return x[i] / root2; });
    map(e.data(), n, [=](i64 i) { return std::erf(sc[i]); });
    map(shifted.data(), n, [=](i64 i) { return ep[i] + 1.f; });
    map(prod.data(), n, [=](i64 i) { return x[i] * sh[i]; });
    out.resize(n);
    map(out.data(), n, [=](i64 i) { return pr[i] * 0.5f; });
}

// dy * (Phi(x) + x * phi(x))
void gelu_backward(Buf& out, const float* dy, const float* x, i64 n) {
    Buf cdf(n), pdf(n);
    const float *cp = cdf.data(), *pp = pdf.data();
    const float root2 = std::sqrt(2.f), norm = std::sqrt(2.f * 3.14159265358979323846f);
    map(cdf.data(), n, [=](i64 i) { return 0.5f * (1.f + std::erf(x[i] / root2)); });
    map(pdf.data(), n, [=](i64 i) { return std::exp(-0.5f * x[i] * x[i]) / norm; });
    out.resize(n);
    map(out.data(), n, [=](i64 i) { return dy[i] * (cp[i] + x[i] * pp[i]); });
}

// reverse of Transpose(W) -> MatMul -> Add: weight gradient 'aij,aik->jk', bias gradient, input gradient 'aij,jk->aik'
void linear_backward(Buf& dinp, float* gw, float* gb, const float* dout, const float* inp, const float* w, i64 T, i64 I, i64 O) {
    Buf dt(O * T);
    transpose_last2(dt.data(), dout, 1, T, O);
    matmul(gw, dt.data(), inp, 1, O, I, T);
    sum_columns(gb, dout, T, O);
    dinp.resize(T * I);
    matmul(dinp.data(), dout, w, 1, T, I, O);
}

}  // namespace

// Parameters and their gradients in the order q_w q_b k_w k_b v_w v_b o_w o_b ffn1_w ffn1_b ffn2_w ffn2_b ln1_g ln1_b
// ln2_g ln2_b (weights [out, in]). x, dy, y, dx: [batch, seq, hidden]. Returns 0, or 1 for shapes it cannot take.
extern "C" int bert_layer_loops(const float* x, const float* dy, const float* const* p, float* y_out, float* dx_out,
                                float* const* g, int batch, int seq, int hidden, int heads, int ffn, float eps) {
    if (batch <= 0 || seq <= 0 || hidden <= 0 || heads <= 0 || ffn <= 0 || hidden % heads) return 1;
    const i64 B = batch, S = seq, H = hidden, NH = heads, F = ffn, D = H / NH, T = B * S, BH = B * NH;
    enum { QW, QB, KW, KB_, VW, VB, OW, OB, F1W, F1B, F2W, F2B, L1G, L1B, L2G, L2B };
    const float root_d = std::sqrt((float)D);

    // ---------------------------------------------------------------- forward
    Buf lin, q(T * H), k(T * H), v(T * H);
    linear(lin, x, p[QW], p[QB], T, H, H);
    transpose_0213(q.data(), lin.data(), B, S, NH, D);
    linear(lin, x, p[KW], p[KB_], T, H, H);
    transpose_0213(k.data(), lin.data(), B, S, NH, D);
    linear(lin, x, p[VW], p[VB], T, H, H);
    transpose_0213(v.data(), lin.data(), B, S, NH, D);

    const i64 NS = BH * S * S;
    Buf probs(NS);
    {
        Buf kt(T * H), scores(NS), scaled(NS), maximum(BH * S), shifted(NS), exponent(NS), total(BH * S);
        transpose_last2(kt.data(), k.data(), BH, S, D);
        matmul(scores.data(), q.data(), kt.data(), BH, S, S, D);
        const float *sc = scores.data(), *sl = scaled.data(), *mx = maximum.data(), *sh = shifted.data(), *ex = exponent.data(),
                    *to = total.data();
        map(scaled.data(), NS, [=](i64 i) { return sc[i] / root_d; });
        reduce_rows(maximum.data(), sl, BH * S, S, -INFINITY, [](float a, float v) { return std::max(a, v); });
        map2(shifted.data(), BH * S, S, [=](i64 r, i64 c) { return sl[r * S + c] - mx[r]; });
        map(exponent.data(), NS, [=](i64 i) { return std::exp(sh[i]); });
        reduce_rows(total.data(), ex, BH * S, S, 0.f, [](float a, float v) { return a + v; });
        map2(probs.data(), BH * S, S, [=](i64 r, i64 c) { return ex[r * S + c] / to[r]; });
    }
    Buf ctx(T * H), ctx2(T * H);
    matmul(ctx.data(), probs.data(), v.data(), BH, S, D, S);
    transpose_0213(ctx2.data(), ctx.data(), B, NH, S, D);

    Buf res1(T * H), h1, pre, act, res2(T * H), y;
    linear(lin, ctx2.data(), p[OW], p[OB], T, H, H);
    {
        const float* l = lin.data();
        map(res1.data(), T * H, [=](i64 i) { return l[i] + x[i]; });
    }
    layernorm_chain(h1, res1.data(), p[L1G], p[L1B], T, H, eps);
    linear(pre, h1.data(), p[F1W], p[F1B], T, H, F);
    gelu_chain(act, pre.data(), T * F);
    linear(lin, act.data(), p[F2W], p[F2B], T, F, H);
    {
        const float *l = lin.data(), *h = h1.data();
        map(res2.data(), T * H, [=](i64 i) { return l[i] + h[i]; });
    }
    layernorm_chain(y, res2.data(), p[L2G], p[L2B], T, H, eps);
    std::copy(y.begin(), y.end(), y_out);
    if (!dy) return 0;

    // ---------------------------------------------------------------- backward
    Buf dres2, dact, dpre, dlin, dh1(T * H), dres1, dctx2;
    layernorm_backward(dres2, g[L2G], g[L2B], dy, res2.data(), p[L2G], T, H, eps);
    linear_backward(dact, g[F2W], g[F2B], dres2.data(), act.data(), p[F2W], T, F, H);
    gelu_backward(dpre, dact.data(), pre.data(), T * F);
    linear_backward(dlin, g[F1W], g[F1B], dpre.data(), h1.data(), p[F1W], T, H, F);
    {
        const float *a = dres2.data(), *b = dlin.data();
        map(dh1.data(), T * H, [=](i64 i) { return a[i] + b[i]; });
    }
    layernorm_backward(dres1, g[L1G], g[L1B], dh1.data(), res1.data(), p[L1G], T, H, eps);
    linear_backward(dctx2, g[OW], g[OB], dres1.data(), ctx2.data(), p[OW], T, H, H);

    Buf dctx(T * H), dq(T * H), dk(T * H), dv(T * H);
    transpose_0213(dctx.data(), dctx2.data(), B, S, NH, D);
    {
        Buf vt(T * H), dprobs(NS), pt(NS), prod(NS), sums(BH * S), ig(NS), dscaled(NS), dscores(NS), dst(NS);
        transpose_last2(vt.data(), v.data(), BH, S, D);
        matmul(dprobs.data(), dctx.data(), vt.data(), BH, S, S, D);
        transpose_last2(pt.data(), probs.data(), BH, S, S);
        matmul(dv.data(), pt.data(), dctx.data(), BH, S, D, S);
        const float *pr = probs.data(), *dp = dprobs.data(), *pd = prod.data(), *su = sums.data(), *igp = ig.data(),
                    *ds = dscaled.data();
        map(prod.data(), NS, [=](i64 i) { return pr[i] * dp[i]; });
        reduce_rows(sums.data(), pd, BH * S, S, 0.f, [](float a, float v) { return a + v; });
        map2(ig.data(), BH * S, S, [=](i64 r, i64 c) { return pr[r * S + c] * su[r]; });
        map(dscaled.data(), NS, [=](i64 i) { return pd[i] - igp[i]; });
        map(dscores.data(), NS, [=](i64 i) { return ds[i] / root_d; });
        matmul(dq.data(), dscores.data(), k.data(), BH, S, D, S);
        transpose_last2(dst.data(), dscores.data(), BH, S, S);
        matmul(dk.data(), dst.data(), q.data(), BH, S, D, S);
    }
    Buf merged(T * H), dx_q, dx_k, dx_v;
    transpose_0213(merged.data(), dq.data(), B, NH, S, D);
    linear_backward(dx_q, g[QW], g[QB], merged.data(), x, p[QW], T, H, H);
    transpose_0213(merged.data(), dk.data(), B, NH, S, D);
    linear_backward(dx_k, g[KW], g[KB_], merged.data(), x, p[KW], T, H, H);
    transpose_0213(merged.data(), dv.data(), B, NH, S, D);
    linear_backward(dx_v, g[VW], g[VB], merged.data(), x, p[VW], T, H, H);
    {
        // Sum(dres1, dx_v, dx_q, dx_k): the variadic Sum adds its inputs in order
        const float *a = dres1.data(), *b = dx_v.data(), *c = dx_q.data(), *d = dx_k.data();
        map(dx_out, T * H, [=](i64 i) { return ((a[i] + b[i]) + c[i]) + d[i]; });
    }
    return 0;
}

extern "C" int bert_layer_loops_threads() { return omp_get_max_threads(); }
