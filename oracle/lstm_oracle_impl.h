/*
 * TEST INFRASTRUCTURE ONLY -- CPU restatement of the LSTM forward/backward
 * algorithm of the reference's persistent path.  Nothing in the product
 * (fastlstm_amd/) may include, link or call this file; it exists so that the
 * HIP path can be checked against an independent implementation and so that
 * bench.py can time a CPU baseline next to the GPU number.
 *
 * This header is a "template": it is included twice by lstm_oracle.c with
 * REAL = double / float and SUF = f64 / f32.
 *
 * Reference lines followed (paths relative to the reference checkout):
 *   forward maths, gate order i,f,g,o ....... fastlstm/lstm.py:1101-1104
 *   time loop, out[0]/cell[0] = initial state  fastlstm/lstm.py:1123-1136, 84-90
 *   x.Wx^T + bx + bh for all timesteps ....... fastlstm/lstm.py:66-68
 *   stored pre-activations ifgo[T,B,4H] ....... fastlstm/kernels.py:631-640
 *   rounding points of the 16-bit path ........ fastlstm/kernels.py:631-657
 *   backward point-wise formulas .............. fastlstm/lstm.py:1143-1166,
 *                                               fastlstm/kernels.py:1301-1316
 *   reverse time loop, dh[s] + dh_rec ......... fastlstm/lstm.py:1204-1221
 *   dh_rec = d_ifgo . Wh (K = 4H) ............. fastlstm/kernels.py:1362-1383
 *   dx, db, dWx, dWh ........................... fastlstm/lstm.py:294, 494-501
 *
 * Parity pinning (tests/test_oracle.py): every output of both functions is
 * checked against torch.nn.LSTM / torch.nn.LSTMCell autograd in float64 on
 * ragged shapes, against central finite differences on tiny inputs, and
 * against closed-form special cases (T=1, Wh=0, zero initial state); the
 * 16-bit round modes of both functions by representability of every stored
 * value and, for the backward, by the matrix identities that tie dx, dWx,
 * dWh and db to the rounded d_ifgo it returns.
 */

#define CAT_(a, b) a##_##b
#define CAT(a, b) CAT_(a, b)
#define FN(name) CAT(name, SUF)

static inline REAL FN(sigm)(REAL v) { return (REAL)1 / ((REAL)1 + (REAL)exp(-(double)v)); }

/*
 * Forward.  out, cell: [T+1, B, H] (slot 0 = initial state, zeros when h0/c0
 * are NULL); ifgo: [T, B, 4H], gate blocks i,f,g,o along the last axis.
 * round_mode: 0 = keep REAL precision, 1 = round every stored ifgo/c/h value
 * to IEEE fp16, 2 = to bfloat16 (the gates are still evaluated on the
 * unrounded pre-activations and c is carried unrounded, h is re-read rounded).
 */
void FN(oracle_lstm_fwd)(int T, int B, int I, int H, const REAL *x, const REAL *h0,
                         const REAL *c0, const REAL *Wx, const REAL *bx, const REAL *Wh,
                         const REAL *bh, REAL *out, REAL *cell, REAL *ifgo, int round_mode) {
    const size_t BH = (size_t)B * H, G = (size_t)4 * H;
    REAL *c_run = (REAL *)malloc(BH * sizeof(REAL)); /* unrounded carried cell state */
    for (size_t i = 0; i < BH; ++i) {
        out[i] = h0 ? h0[i] : (REAL)0;
        cell[i] = c0 ? c0[i] : (REAL)0;
        c_run[i] = cell[i];
    }
    for (int t = 0; t < T; ++t) {
        const REAL *xt = x + (size_t)t * B * I;
        const REAL *hp = out + (size_t)t * BH;
        REAL *hn = out + (size_t)(t + 1) * BH;
        REAL *cn = cell + (size_t)(t + 1) * BH;
        REAL *pt = ifgo + (size_t)t * B * G;
#pragma omp parallel for schedule(static)
        for (int b = 0; b < B; ++b) {
            const REAL *xb = xt + (size_t)b * I;
            const REAL *hb = hp + (size_t)b * H;
            REAL *pb = pt + (size_t)b * G;
            for (size_t r = 0; r < G; ++r) {
                const REAL *wx = Wx + r * I;
                const REAL *wh = Wh + r * H;
                REAL acc = bx[r] + bh[r];
                REAL ax = 0, ah = 0;
#pragma omp simd reduction(+ : ax)
                for (int k = 0; k < I; ++k) ax += xb[k] * wx[k];
#pragma omp simd reduction(+ : ah)
                for (int k = 0; k < H; ++k) ah += hb[k] * wh[k];
                pb[r] = acc + ax + ah;
            }
            for (int u = 0; u < H; ++u) {
                REAL pi = pb[u], pf = pb[H + u], pg = pb[2 * H + u], po = pb[3 * H + u];
                size_t idx = (size_t)b * H + u;
                REAL c1 = FN(sigm)(pf) * c_run[idx] + FN(sigm)(pi) * (REAL)tanh((double)pg);
                REAL h1 = FN(sigm)(po) * (REAL)tanh((double)c1);
                c_run[idx] = c1;
                cn[idx] = (REAL)round_to((double)c1, round_mode);
                hn[idx] = (REAL)round_to((double)h1, round_mode);
            }
            if (round_mode)
                for (size_t r = 0; r < G; ++r) pb[r] = (REAL)round_to((double)pb[r], round_mode);
        }
    }
    free(c_run);
}

/*
 * Backward.  dout: [T,B,H] upstream gradient of out[1:]; dh_n, dc_n: [B,H]
 * gradients flowing into the last hidden/cell state (NULL = zeros).
 * Outputs: dx [T,B,I], dh0, dc0 [B,H], dWx [4H,I], dWh [4H,H], db [4H],
 * d_ifgo [T,B,4H].  round_mode as above applies to the stored d_ifgo (which
 * is also what the recurrent product and the weight-gradient sums consume).
 * The carried dc and dh_rec stay unrounded (the reference's default kernel
 * rounds them through 16-bit buffers every step, kernels.py:1337-1342,
 * 1388-1390; the HIP path keeps them in fp32 registers, so the checker does too).
 */
void FN(oracle_lstm_bwd)(int T, int B, int I, int H, const REAL *dout, const REAL *dh_n,
                         const REAL *dc_n, const REAL *x, const REAL *out, const REAL *cell,
                         const REAL *ifgo, const REAL *Wx, const REAL *Wh, REAL *dx, REAL *dh0,
                         REAL *dc0, REAL *dWx, REAL *dWh, REAL *db, REAL *d_ifgo, int round_mode) {
    const size_t BH = (size_t)B * H, G = (size_t)4 * H;
    REAL *dh = (REAL *)malloc(BH * sizeof(REAL));
    REAL *dc = (REAL *)malloc(BH * sizeof(REAL));
    for (size_t i = 0; i < BH; ++i) {
        dh[i] = dh_n ? dh_n[i] : (REAL)0;
        dc[i] = dc_n ? dc_n[i] : (REAL)0;
    }
    memset(dWx, 0, G * I * sizeof(REAL));
    memset(dWh, 0, G * H * sizeof(REAL));
    memset(db, 0, G * sizeof(REAL));
    for (int t = T - 1; t >= 0; --t) {
        const REAL *pt = ifgo + (size_t)t * B * G;
        const REAL *c0t = cell + (size_t)t * BH;
        const REAL *c1t = cell + (size_t)(t + 1) * BH;
        const REAL *dot = dout + (size_t)t * BH;
        const REAL *xt = x + (size_t)t * B * I;
        const REAL *hprev = out + (size_t)t * BH;
        REAL *dpt = d_ifgo + (size_t)t * B * G;
        REAL *dxt = dx + (size_t)t * B * I;
#pragma omp parallel for schedule(static)
        for (int b = 0; b < B; ++b) {
            const REAL *pb = pt + (size_t)b * G;
            REAL *dpb = dpt + (size_t)b * G;
            for (int u = 0; u < H; ++u) {
                size_t idx = (size_t)b * H + u;
                REAL si = FN(sigm)(pb[u]), sf = FN(sigm)(pb[H + u]);
                REAL tg = (REAL)tanh((double)pb[2 * H + u]), so = FN(sigm)(pb[3 * H + u]);
                REAL tc = (REAL)tanh((double)c1t[idx]);
                REAL dht = dh[idx] + dot[idx];
                REAL dc1 = dc[idx] + dht * so * ((REAL)1 - tc * tc);
                REAL d_o = dht * tc * so * ((REAL)1 - so);
                REAL d_f = dc1 * c0t[idx] * sf * ((REAL)1 - sf);
                REAL d_i = dc1 * tg * si * ((REAL)1 - si);
                REAL d_g = dc1 * si * ((REAL)1 - tg * tg);
                REAL dcp = dc1 * sf;
                dc[idx] = dcp;
                dpb[u] = (REAL)round_to((double)d_i, round_mode);
                dpb[H + u] = (REAL)round_to((double)d_f, round_mode);
                dpb[2 * H + u] = (REAL)round_to((double)d_g, round_mode);
                dpb[3 * H + u] = (REAL)round_to((double)d_o, round_mode);
            }
            /* dh_rec[b,:] = d_ifgo[t,b,:] . Wh   and   dx[t,b,:] = d_ifgo[t,b,:] . Wx */
            REAL *dhb = dh + (size_t)b * H;
            REAL *dxb = dxt + (size_t)b * I;
            for (int k = 0; k < H; ++k) dhb[k] = 0;
            for (int k = 0; k < I; ++k) dxb[k] = 0;
            for (size_t r = 0; r < G; ++r) {
                const REAL d = dpb[r];
                const REAL *wh = Wh + r * H;
                const REAL *wx = Wx + r * I;
#pragma omp simd
                for (int k = 0; k < H; ++k) dhb[k] += d * wh[k];
#pragma omp simd
                for (int k = 0; k < I; ++k) dxb[k] += d * wx[k];
            }
        }
        /* weight gradients: sums over batch (and, through the t loop, over time) */
#pragma omp parallel for schedule(static)
        for (size_t r = 0; r < G; ++r) {
            REAL *gx = dWx + r * I;
            REAL *gh = dWh + r * H;
            REAL s = 0;
            for (int b = 0; b < B; ++b) {
                const REAL d = dpt[(size_t)b * G + r];
                const REAL *xb = xt + (size_t)b * I;
                const REAL *hb = hprev + (size_t)b * H;
                s += d;
#pragma omp simd
                for (int k = 0; k < I; ++k) gx[k] += d * xb[k];
#pragma omp simd
                for (int k = 0; k < H; ++k) gh[k] += d * hb[k];
            }
            db[r] += s;
        }
    }
    for (size_t i = 0; i < BH; ++i) {
        dh0[i] = dh[i];
        dc0[i] = dc[i];
    }
    free(dh);
    free(dc);
}

#undef FN
#undef CAT
#undef CAT_
