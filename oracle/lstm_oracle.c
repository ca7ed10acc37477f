/* CPU restatement of the LSTM forward + BPTT path -- TEST INFRASTRUCTURE, NOT PRODUCT CODE.
 *
 * Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may build, load or call
 * this file; the shipped library (flashlstm_poc_amd/) never links or falls back to it.
 *
 * Plain C, double precision arithmetic, PyTorch tensor layouts, gate order i,f,g,o.  Each function
 * names the reference lines it restates:
 *   oracle_lstm_forward   pointwise cell of src/kernels.cu:86-164 (gates = x W_ih^T + h W_hh^T + b_ih
 *                         + b_hh, sigmoid/tanh, c' = f c + i g, h' = o tanh c'), step order and h0/c0
 *                         handling of src/lstm.cu:1241-1339,1930-1941; optional fp16 rounding of the
 *                         operands and of the fed-back h as in src/kernels.cu:150-155
 *   oracle_lstm_backward  closed-form BPTT of flashlstm_v2/src/lstm_backward.cu:199-211 (pointwise),
 *                         :1083-1097 (dh = dG W_hh), :1112-1172 (dW_ih, dW_hh, db, dX), :1218-1246
 *                         (db_ih == db_hh, dh0/dc0) -- with c taken from the forward pass instead of
 *                         the atanh reconstruction of :188-197; flag bit3 rounds the pre-activation
 *                         gradients dG to fp16 before the products that consume them, as the fp16 copy
 *                         written at :213-222 for the half-operand GEMMs does
 *   oracle_pack_weights_v1 layout of src/kernels.cu:57-84 with stride = align_up(I+H, 8)
 *                         (src/lstm.cu:698-699)
 *   oracle_checkpoints    "entry k = state before step k*R" of flashlstm_v2/src/lstm_forward.cu:370-375,
 *                         727-783
 *   oracle_chunk_steps    src/lstm.cu:144-153 (chunk <= 0 or > T means the whole sequence)
 *
 * Pinned by tests/test_oracle.py against torch.nn.LSTM (CPU, fp64 autograd), central finite
 * differences, closed forms (W_hh = 0, zero input) and committed golden vectors (tests/golden/).
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

static double sigmoid(double x) { return 1.0 / (1.0 + exp(-x)); }

/* round-to-nearest-even float -> IEEE binary16 -> double */
static double round_fp16(double v) {
    float f = (float)v;
    uint32_t x;
    memcpy(&x, &f, 4);
    uint32_t sign = x & 0x80000000u;
    uint32_t ax = x & 0x7fffffffu;
    if (ax >= 0x7f800000u) return v;                 /* inf / nan */
    if (ax >= 0x477ff000u) {                         /* >= 65520 rounds to inf */
        return sign ? -INFINITY : INFINITY;
    }
    float a = fabsf(f), r;
    if (ax < 0x38800000u) {                          /* subnormal half: quantum 2^-24 */
        r = (float)(rint((double)a * 16777216.0) / 16777216.0);
    } else {
        int e;
        (void)frexpf(a, &e);                         /* a = m * 2^e, m in [0.5,1) */
        double q = ldexp(1.0, e - 11);               /* 11 significant bits */
        r = (float)(rint((double)a / q) * q);
    }
    return sign ? -(double)r : (double)r;
}

double oracle_round_fp16(double v) { return round_fp16(v); }

size_t oracle_chunk_steps(int chunk, size_t T) {
    if (chunk <= 0 || (size_t)chunk > T) return T;
    return (size_t)chunk;
}

/* flags: bit0 = round x, W_ih, W_hh to fp16 before use; bit1 = feed h back through an fp16 cast;
 *        bit2 = round stored y / h_all to fp16 (what an fp16 output tensor holds).
 * Outputs (any may be NULL): y (T,B,H); hn, cn (B,H); gates (T,B,4H) activated i,f,g,o in PyTorch
 * order [gate*H + j]; h_all, c_all (T+1,B,H) with entry t = state before step t. */
int oracle_lstm_forward(size_t T, size_t B, size_t I, size_t H, const double* x, const double* w_ih,
                        const double* w_hh, const double* b_ih, const double* b_hh, const double* h0,
                        const double* c0, int flags, double* y, double* hn, double* cn, double* gates,
                        double* h_all, double* c_all) {
    const size_t G = 4 * H;
    double* wi = (double*)malloc(sizeof(double) * G * I + 8);
    double* wh = (double*)malloc(sizeof(double) * G * H + 8);
    double* h = (double*)calloc(B * H + 1, sizeof(double));
    double* c = (double*)calloc(B * H + 1, sizeof(double));
    double* hnext = (double*)calloc(B * H + 1, sizeof(double));
    double* z = (double*)malloc(sizeof(double) * G + 8);
    if (!wi || !wh || !h || !c || !hnext || !z) return 1;
    for (size_t k = 0; k < G * I; ++k) wi[k] = (flags & 1) ? round_fp16(w_ih[k]) : w_ih[k];
    for (size_t k = 0; k < G * H; ++k) wh[k] = (flags & 1) ? round_fp16(w_hh[k]) : w_hh[k];
    for (size_t k = 0; k < B * H; ++k) {
        h[k] = h0 ? h0[k] : 0.0;
        c[k] = c0 ? c0[k] : 0.0;
        if (flags & 2) h[k] = round_fp16(h[k]);
    }
    for (size_t t = 0; t < T; ++t) {
        if (h_all) memcpy(h_all + t * B * H, h, sizeof(double) * B * H);
        if (c_all) memcpy(c_all + t * B * H, c, sizeof(double) * B * H);
        for (size_t b = 0; b < B; ++b) {
            const double* xt = x + (t * B + b) * I;
            for (size_t r = 0; r < G; ++r) {
                double s = (b_ih ? b_ih[r] : 0.0) + (b_hh ? b_hh[r] : 0.0);
                const double* wr = wi + r * I;
                for (size_t k = 0; k < I; ++k) s += ((flags & 1) ? round_fp16(xt[k]) : xt[k]) * wr[k];
                const double* hr = wh + r * H;
                for (size_t k = 0; k < H; ++k) s += h[b * H + k] * hr[k];
                z[r] = s;
            }
            for (size_t j = 0; j < H; ++j) {
                const double ig = sigmoid(z[j]), fg = sigmoid(z[H + j]);
                const double gg = tanh(z[2 * H + j]), og = sigmoid(z[3 * H + j]);
                const double cv = fg * c[b * H + j] + ig * gg;
                double hv = og * tanh(cv);
                c[b * H + j] = cv;
                if (gates) {
                    double* gt = gates + (t * B + b) * G;
                    gt[j] = ig; gt[H + j] = fg; gt[2 * H + j] = gg; gt[3 * H + j] = og;
                }
                if (y) y[(t * B + b) * H + j] = (flags & 4) ? round_fp16(hv) : hv;
                hnext[b * H + j] = (flags & 2) ? round_fp16(hv) : hv;
            }
        }
        memcpy(h, hnext, sizeof(double) * B * H);
    }
    if (h_all) memcpy(h_all + T * B * H, h, sizeof(double) * B * H);
    if (c_all) memcpy(c_all + T * B * H, c, sizeof(double) * B * H);
    if (hn) memcpy(hn, h, sizeof(double) * B * H);
    if (cn) memcpy(cn, c, sizeof(double) * B * H);
    free(wi); free(wh); free(h); free(c); free(hnext); free(z);
    return 0;
}

/* BPTT.  gates (T,B,4H), h_all / c_all (T+1,B,H) come from oracle_lstm_forward.  dY (T,B,H);
 * d_hn / d_cn (B,H) may be NULL.  Outputs (any may be NULL): dx (T,B,I), dw_ih (4H,I), dw_hh (4H,H),
 * db (4H) (the gradient of b_ih and of b_hh alike), dh0, dc0 (B,H).
 * flags bit0: use fp16-rounded W_ih / W_hh in the products (matches forward flag bit0). */
int oracle_lstm_backward(size_t T, size_t B, size_t I, size_t H, const double* x, const double* w_ih,
                         const double* w_hh, const double* gates, const double* h_all, const double* c_all,
                         const double* dY, const double* d_hn, const double* d_cn, int flags, double* dx,
                         double* dw_ih, double* dw_hh, double* db, double* dh0, double* dc0) {
    const size_t G = 4 * H;
    double* dh = (double*)calloc(B * H + 1, sizeof(double));
    double* dc = (double*)calloc(B * H + 1, sizeof(double));
    double* dhp = (double*)calloc(B * H + 1, sizeof(double));
    double* dg = (double*)malloc(sizeof(double) * B * G + 8);
    double* wi = (double*)malloc(sizeof(double) * G * I + 8);
    double* wh = (double*)malloc(sizeof(double) * G * H + 8);
    if (!dh || !dc || !dhp || !dg || !wi || !wh) return 1;
    for (size_t k = 0; k < G * I; ++k) wi[k] = (flags & 1) ? round_fp16(w_ih[k]) : w_ih[k];
    for (size_t k = 0; k < G * H; ++k) wh[k] = (flags & 1) ? round_fp16(w_hh[k]) : w_hh[k];
    if (dw_ih) memset(dw_ih, 0, sizeof(double) * G * I);
    if (dw_hh) memset(dw_hh, 0, sizeof(double) * G * H);
    if (db) memset(db, 0, sizeof(double) * G);
    for (size_t k = 0; k < B * H; ++k) {
        dh[k] = d_hn ? d_hn[k] : 0.0;
        dc[k] = d_cn ? d_cn[k] : 0.0;
    }
    for (size_t t = T; t-- > 0;) {
        for (size_t b = 0; b < B; ++b) {
            const double* gt = gates + (t * B + b) * G;
            for (size_t j = 0; j < H; ++j) {
                const double ig = gt[j], fg = gt[H + j], gg = gt[2 * H + j], og = gt[3 * H + j];
                const double cprev = c_all[(t * B + b) * H + j];
                const double tc = tanh(c_all[((t + 1) * B + b) * H + j]);
                const double dht = dh[b * H + j] + dY[(t * B + b) * H + j];
                const double dov = dht * tc;
                const double dcv = dc[b * H + j] + dht * og * (1.0 - tc * tc);
                double* d = dg + b * G;
                d[j] = dcv * gg * ig * (1.0 - ig);
                d[H + j] = dcv * cprev * fg * (1.0 - fg);
                d[2 * H + j] = dcv * ig * (1.0 - gg * gg);
                d[3 * H + j] = dov * og * (1.0 - og);
                dc[b * H + j] = dcv * fg;
                if (flags & 8) {   /* the GEMMs that consume dG take fp16 operands */
                    d[j] = round_fp16(d[j]);
                    d[H + j] = round_fp16(d[H + j]);
                    d[2 * H + j] = round_fp16(d[2 * H + j]);
                    d[3 * H + j] = round_fp16(d[3 * H + j]);
                }
            }
        }
        memset(dhp, 0, sizeof(double) * B * H);
        for (size_t b = 0; b < B; ++b) {
            const double* d = dg + b * G;
            const double* xt = x + (t * B + b) * I;
            const double* hp = h_all + (t * B + b) * H;
            for (size_t r = 0; r < G; ++r) {
                const double v = d[r];
                if (db) db[r] += v;
                for (size_t k = 0; k < H; ++k) dhp[b * H + k] += v * wh[r * H + k];
                if (dw_hh) for (size_t k = 0; k < H; ++k) dw_hh[r * H + k] += v * hp[k];
                if (dw_ih) for (size_t k = 0; k < I; ++k) dw_ih[r * I + k] += v * xt[k];
                if (dx) {
                    double* dxt = dx + (t * B + b) * I;
                    if (r == 0) memset(dxt, 0, sizeof(double) * I);
                    for (size_t k = 0; k < I; ++k) dxt[k] += v * wi[r * I + k];
                }
            }
        }
        memcpy(dh, dhp, sizeof(double) * B * H);
    }
    if (dh0) memcpy(dh0, dh, sizeof(double) * B * H);
    if (dc0) memcpy(dc0, dc, sizeof(double) * B * H);
    free(dh); free(dc); free(dhp); free(dg); free(wi); free(wh);
    return 0;
}

/* packed[4H][stride], stride = align_up(I+H, 8): row r = [W_ih[r][0..I), W_hh[r][0..H), zeros]. */
size_t oracle_pack_stride_v1(size_t I, size_t H) { return (I + H + 7) / 8 * 8; }
void oracle_pack_weights_v1(size_t I, size_t H, const double* w_ih, const double* w_hh, double* packed) {
    const size_t stride = oracle_pack_stride_v1(I, H);
    for (size_t r = 0; r < 4 * H; ++r)
        for (size_t col = 0; col < stride; ++col) {
            double v = 0.0;
            if (col < I) v = w_ih[r * I + col];
            else if (col < I + H) v = w_hh[r * H + (col - I)];
            packed[r * stride + col] = round_fp16(v);
        }
}

/* out[k] = all[k*R] for k < ceil(T/R); all is (T+1,B,H). */
void oracle_checkpoints(size_t T, size_t B, size_t H, size_t R, const double* all, double* out) {
    const size_t n = (T + R - 1) / R;
    for (size_t k = 0; k < n; ++k) memcpy(out + k * B * H, all + k * R * B * H, sizeof(double) * B * H);
}
