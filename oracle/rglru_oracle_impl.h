/*
 * TEST INFRASTRUCTURE, NOT PRODUCT CODE.
 *
 * Body of the CPU restatement of Hawk's RG-LRU scan, temporal conv1d and decode step.
 * Included twice by rglru_oracle.c, once with REAL=double (suffix _f64, the ground truth)
 * and once with REAL=float (suffix _f32, the timed scalar CPU port).
 *
 * Every function states the reference lines it follows (paths under the upstream tree,
 * hawk/...).  All tensors are dense row-major: activations [B,T,D], Lambda [D],
 * conv weight [W,D], conv bias [D], conv state [B,W-1,D].
 */

#ifndef REAL
#error "define REAL and SUFFIX before including"
#endif

#define CAT_(a, b) a##b
#define CAT(a, b) CAT_(a, b)
#define FN(name) CAT(name, SUFFIX)

/* hawk/scan_fused.py:18-20 (softplus_fwd), evaluated without overflow for large x. */
static REAL FN(softplus)(REAL x) {
    if (x > (REAL)30) return x;
    return (REAL)log1p(exp((double)x));
}

/* logistic function, the tl.sigmoid of hawk/scan_fused.py:65-66 and softplus_bwd of :23-25 */
static REAL FN(sigmoid)(REAL x) {
    if (x >= 0) {
        return (REAL)(1.0 / (1.0 + exp(-(double)x)));
    } else {
        double e = exp((double)x);
        return (REAL)(e / (1.0 + e));
    }
}

/* hawk/scan_fused.py:10-15: derivative of sqrt with the argument floored so that the
 * derivative never exceeds MAX_SQRT_GRADIENT=1000:  1/sqrt(max(4z, 1e-6)). */
static REAL FN(clipped_sqrt_grad)(REAL z) {
    const REAL min_value = (REAL)(1.0 / (1000.0 * 1000.0));
    REAL scaled = (REAL)4 * z;
    REAL clipped = scaled > min_value ? scaled : min_value;
    return (REAL)1 / (REAL)sqrt((double)clipped);
}

/*
 * Forward scan.  hawk/scan_fused.py:44-109.
 *   r = sigmoid(a_rg_lru), i = sigmoid(x_rg_lru)          (:65-66, :93-94)
 *   log_a = -8 * r * softplus(Lambda)                      (:44, :68, :96)
 *   alpha = exp(log_a), a2 = exp(2 log_a), m = sqrt(1-a2)  (:69-71, :97-101)
 *   beta = (x*i) * m                                       (:73-75, :103-105)
 *   h_0 = beta_0                                           (:79)
 *   h_t = alpha_t * h_{t-1} + beta_t                       (:107)
 */
void FN(oracle_rglru_scan_fwd)(const REAL* x, const REAL* xg, const REAL* ag, const REAL* lam,
                               REAL* h, int B, int T, int D) {
    for (int b = 0; b < B; ++b) {
        for (int d = 0; d < D; ++d) {
            const REAL s = FN(softplus)(lam[d]);
            REAL state = 0;
            for (int t = 0; t < T; ++t) {
                const size_t k = ((size_t)b * T + t) * D + d;
                const REAL r = FN(sigmoid)(ag[k]);
                const REAL i = FN(sigmoid)(xg[k]);
                const REAL log_a = (REAL)-8 * r * s;
                const REAL alpha = (REAL)exp((double)log_a);
                const REAL a2 = (REAL)exp((double)((REAL)2 * log_a));
                const REAL m = (REAL)sqrt((double)((REAL)1 - a2));
                const REAL beta = (x[k] * i) * m;
                state = (t == 0) ? beta : alpha * state + beta;
                h[k] = state;
            }
        }
    }
}

/*
 * Backward scan.  hawk/scan_fused.py:123-317 and the batch reduction at :424.
 *   g_{T-1} = gout_{T-1}; g_t = gout_t + alpha_{t+1} g_{t+1}          (:153, :213-219, :273-276)
 *   d_alpha_t = g_t * h_{t-1}, absent at t = 0                        (:160, :221, :303)
 *   dlog_a_t = d_alpha_t*alpha_t + g_t*(i_t x_t)*csg(1-a2_t)*(-2 a2_t) (:175-184, :244-252)
 *   da_rg_lru_t = sigmoid'(a_rg_lru_t) * dlog_a_t * (-8) * softplus(Lambda)   (:186, :254)
 *   dx_t = g_t * m_t * i_t                                            (:188, :240)
 *   dx_rg_lru_t = g_t * m_t * x_t * sigmoid'(x_rg_lru_t)              (:190, :242)
 *   dLambda = sum_{b,t} dlog_a_t * (-8) * r_t * sigmoid(Lambda)       (:192, :256, :311, :424)
 * The upstream kernel is only meaningful for T >= 2 (its t = T-1 peel reads row T-2 of
 * h_saved); T = 1 is handled here as the single step t = 0 with d_alpha absent.
 */
void FN(oracle_rglru_scan_bwd)(const REAL* x, const REAL* xg, const REAL* ag, const REAL* lam,
                               const REAL* h_saved, const REAL* gout, REAL* dx, REAL* dxg,
                               REAL* dag, REAL* dlam, int B, int T, int D) {
    for (int d = 0; d < D; ++d) dlam[d] = 0;
    for (int b = 0; b < B; ++b) {
        for (int d = 0; d < D; ++d) {
            const REAL s = FN(softplus)(lam[d]);
            const REAL dsoftplus = FN(sigmoid)(lam[d]);
            REAL g = 0;
            REAL alpha_next = 0;
            REAL acc = 0;
            for (int t = T - 1; t >= 0; --t) {
                const size_t k = ((size_t)b * T + t) * D + d;
                g = gout[k] + alpha_next * g;
                const REAL r = FN(sigmoid)(ag[k]);
                const REAL i = FN(sigmoid)(xg[k]);
                const REAL log_a = (REAL)-8 * r * s;
                const REAL alpha = (REAL)exp((double)log_a);
                const REAL a2 = (REAL)exp((double)((REAL)2 * log_a));
                const REAL m = (REAL)sqrt((double)((REAL)1 - a2));
                const REAL d_alpha = (t > 0) ? g * h_saved[k - D] : (REAL)0;
                REAL dlog_a = d_alpha * alpha;
                dlog_a += g * (i * x[k]) * FN(clipped_sqrt_grad)((REAL)1 - a2) * ((REAL)-2 * a2);
                dag[k] = (r * ((REAL)1 - r)) * dlog_a * (REAL)-8 * s;
                dx[k] = g * m * i;
                dxg[k] = g * m * x[k] * (i * ((REAL)1 - i));
                acc += dlog_a * (REAL)-8 * r * dsoftplus;
                alpha_next = alpha;
            }
            dlam[d] += acc;
        }
    }
}

/*
 * Temporal conv1d forward.  hawk/external.py:49-95 with :100-136:
 *   y[b,t,c] = bias[c] + sum_{s=0}^{min(W,T+S)-1} w[W-1-s, c] * x[b, t-s, c]
 * where rows before t = 0 are zero in training (prompt_len = 0, zero left pad of :123-136).
 * With `state` (the [B,W-1,D] rows that precede t = 0, oldest first, as the decode path
 * of hawk/hawk.py:169 concatenates them) those rows are read from it instead.
 */
void FN(oracle_conv1d_fwd)(const REAL* x, const REAL* w, const REAL* bias, const REAL* state,
                           REAL* y, int B, int T, int D, int W) {
    for (int b = 0; b < B; ++b)
        for (int t = 0; t < T; ++t)
            for (int c = 0; c < D; ++c) {
                REAL acc = 0;
                for (int s = 0; s < W; ++s) {
                    const int tt = t - s;
                    REAL xv;
                    if (tt >= 0)
                        xv = x[((size_t)b * T + tt) * D + c];
                    else if (state)
                        xv = state[((size_t)b * (W - 1) + (W - 1 + tt)) * D + c];
                    else
                        xv = 0;
                    acc += xv * w[(size_t)(W - 1 - s) * D + c];
                }
                y[((size_t)b * T + t) * D + c] = acc + bias[c];
            }
}

/*
 * Temporal conv1d backward: the adjoint of the map above (upstream has no hand-written
 * backward; autograd differentiates hawk/external.py:78-93).
 *   dx[b,t,c]    = sum_{s} w[W-1-s,c] * gy[b,t+s,c]      (t+s < T)
 *   dw[W-1-s,c]  = sum_{b,t} gy[b,t,c] * x[b,t-s,c]      (t-s >= 0, zero history)
 *   db[c]        = sum_{b,t} gy[b,t,c]
 */
void FN(oracle_conv1d_bwd)(const REAL* gy, const REAL* x, const REAL* w, REAL* dx, REAL* dw,
                           REAL* db, int B, int T, int D, int W) {
    for (int k = 0; k < W * D; ++k) dw[k] = 0;
    for (int c = 0; c < D; ++c) db[c] = 0;
    for (int b = 0; b < B; ++b)
        for (int t = 0; t < T; ++t)
            for (int c = 0; c < D; ++c) {
                REAL acc = 0;
                for (int s = 0; s < W; ++s) {
                    if (t + s < T)
                        acc += w[(size_t)(W - 1 - s) * D + c] * gy[((size_t)b * T + t + s) * D + c];
                }
                dx[((size_t)b * T + t) * D + c] = acc;
                const REAL g = gy[((size_t)b * T + t) * D + c];
                db[c] += g;
                for (int s = 0; s < W; ++s) {
                    if (t - s >= 0)
                        dw[(size_t)(W - 1 - s) * D + c] += g * x[((size_t)b * T + t - s) * D + c];
                }
            }
}

/*
 * One decode step of the RG-LRU.  hawk/hawk.py:137-151 and :196:
 *   a = exp(-8 sigmoid(a_gate) softplus(Lambda)); mult = sqrt(1 - exp(2 log_a))
 *   h = a * recc_state + (x * sigmoid(i_gate)) * mult
 * state_in/h_out are [B,D]; h_out may alias state_in.
 */
void FN(oracle_rglru_step)(const REAL* x, const REAL* xg, const REAL* ag, const REAL* lam,
                           const REAL* state_in, REAL* h_out, int B, int D) {
    for (int b = 0; b < B; ++b)
        for (int d = 0; d < D; ++d) {
            const size_t k = (size_t)b * D + d;
            const REAL s = FN(softplus)(lam[d]);
            const REAL r = FN(sigmoid)(ag[k]);
            const REAL i = FN(sigmoid)(xg[k]);
            const REAL log_a = (REAL)-8 * r * s;
            const REAL a = (REAL)exp((double)log_a);
            const REAL mult = (REAL)sqrt((double)((REAL)1 - (REAL)exp((double)((REAL)2 * log_a))));
            h_out[k] = a * state_in[k] + (x[k] * i) * mult;
        }
}

/*
 * One decode step of the temporal conv.  hawk/hawk.py:169-179 with hawk/cache.py:37-43:
 * the window is concat(conv_state, x_new); the state is rolled up by one row and x_new is
 * written into its last row; the output is the last row of the conv over the window.
 * conv_state is [B,W-1,D] (oldest row first) and is updated in place.
 */
void FN(oracle_conv1d_step)(REAL* conv_state, const REAL* x_new, const REAL* w, const REAL* bias,
                            REAL* y, int B, int D, int W) {
    for (int b = 0; b < B; ++b)
        for (int c = 0; c < D; ++c) {
            REAL* st = conv_state + (size_t)b * (W - 1) * D + c;
            const REAL xn = x_new[(size_t)b * D + c];
            REAL acc = xn * w[(size_t)(W - 1) * D + c];
            for (int j = 0; j < W - 1; ++j) acc += st[(size_t)j * D] * w[(size_t)j * D + c];
            y[(size_t)b * D + c] = acc + bias[c];
            for (int j = 0; j + 1 < W - 1; ++j) st[(size_t)j * D] = st[(size_t)(j + 1) * D];
            if (W > 1) st[(size_t)(W - 2) * D] = xn;
        }
}

#undef FN
#undef CAT
#undef CAT_
