// CPU oracle, LSTM layer -- TEST INFRASTRUCTURE ONLY (see oracle_common.h).
//
// Restates /root/reference/CURRENNT_codes/currennt_lib/src/layers/LstmLayer.cu:
//   weight vector layout           LstmLayer.cu:1136-1169, 1218-1268 (LstmLayer.hpp:36-55)
//   forward cell update            LstmLayer.cu:57-185   (driver 1743-1949)
//   output interleave (BLSTM)      LstmLayer.cu:187-208
//   output-error split (BLSTM)     LstmLayer.cu:210-235
//   gate / cell errors             LstmLayer.cu:237-405  (driver 2066-2255)
//   error to the preceding layer   LstmLayer.cu:2298-2334
//   weight updates                 LstmLayer.cu:407-648  (driver 2337-2375)
// The ClockLSTM branch is not restated.
#include "currennt_oracle.h"
#include "oracle_common.h"

#include <cstring>

static int g_threads = 1;
namespace orc {
int threads() { return g_threads; }
}  // namespace orc

namespace {

struct Geometry {
    int P, L, H, S, T, Tmin, ndir, n;  // n = S*H, the stride between time steps
    float bias;
    size_t off_bias, off_int, off_peep;
    explicit Geometry(const orc_lstm_desc &d) {
        P = d.P; L = d.L; ndir = d.bidir ? 2 : 1; H = L / ndir; S = d.S; T = d.T; Tmin = d.Tmin;
        n = S * H; bias = d.bias;
        off_bias = (size_t)4 * P * L;
        off_int = off_bias + (size_t)4 * L;
        off_peep = off_int + (size_t)4 * L * H;
    }
    // P x H column-major block of gate g, direction dir
    const float *w_in(const float *w, int g, int dir) const { return w + (size_t)g * P * L + (size_t)dir * P * H; }
    const float *w_bias(const float *w, int g, int dir) const { return w + off_bias + (size_t)g * L + dir * H; }
    // H x H column-major block [from + to*H]
    const float *w_int(const float *w, int g, int dir) const {
        return w + off_int + (size_t)g * L * H + (size_t)dir * H * H;
    }
    // k: 0 input gate, 1 forget gate, 2 output gate
    const float *w_peep(const float *w, int k, int dir) const { return w + off_peep + (size_t)k * L + dir * H; }
};

void forward_direction(const Geometry &G, const float *W, const char *pat, const float *x, orc_lstm_dir *st,
                       int dir) {
    const int H = G.H, S = G.S, T = G.T, n = G.n;
    float *act[4] = {st->ni, st->ig, st->fg, st->og};
    for (int g = 0; g < 4; ++g)
        orc::mat_product(act[g], H, T * S, G.P, G.w_in(W, g, dir), true, x, false, false);

    const float *b_ni = G.w_bias(W, 0, dir), *b_ig = G.w_bias(W, 1, dir);
    const float *b_fg = G.w_bias(W, 2, dir), *b_og = G.w_bias(W, 3, dir);
    const float *p_ig = G.w_peep(W, 0, dir), *p_fg = G.w_peep(W, 1, dir), *p_og = G.w_peep(W, 2, dir);

    for (int step = 0; step < T; ++step) {
        const int t = dir ? (T - 1 - step) : step;
        const int prev = dir ? t + 1 : t - 1;
        const bool first = (step == 0);
        const bool check = (t >= G.Tmin);
        if (!first)
            for (int g = 0; g < 4; ++g)
                orc::mat_product(act[g] + (size_t)t * n, H, S, H, G.w_int(W, g, dir), true,
                                 st->h + (size_t)prev * n, false, true);
        for (int s = 0; s < S; ++s) {
            const bool dummy = check && pat[t * S + s] == orc::PAT_NONE;
            for (int j = 0; j < H; ++j) {
                const size_t i = (size_t)t * n + (size_t)s * H + j;
                if (dummy) {
                    if (dir) st->c[i] = 0.0f;  // only the time-reversed direction clears the cell
                    st->h[i] = 0.0f;
                    continue;
                }
                const size_t ip = (size_t)prev * n + (size_t)s * H + j;
                float a_ni = st->ni[i] + G.bias * b_ni[j];
                float a_ig = st->ig[i] + G.bias * b_ig[j];
                float a_fg = st->fg[i] + G.bias * b_fg[j];
                float a_og = st->og[i] + G.bias * b_og[j];
                if (!first) {
                    const float cp = st->c[ip];
                    a_ig += cp * p_ig[j];
                    a_fg += cp * p_fg[j];
                }
                const float ni = orc::tanh_act(a_ni);
                const float ig = orc::logistic(a_ig);
                const float fg = orc::logistic(a_fg);
                st->ni[i] = ni; st->ig[i] = ig; st->fg[i] = fg;
                float c = ni * ig;
                if (!first) c += st->c[ip] * fg;
                st->c[i] = c;
                a_og += c * p_og[j];
                const float og = orc::logistic(a_og);
                st->og[i] = og;
                st->h[i] = orc::tanh_act(c) * og;
            }
        }
    }
}

void backward_direction(const Geometry &G, const float *W, const char *pat, orc_lstm_dir *st, int dir) {
    const int H = G.H, S = G.S, T = G.T, n = G.n;
    float *delta[4] = {st->dni, st->dig, st->dfg, st->dog};
    const float *p_ig = G.w_peep(W, 0, dir), *p_fg = G.w_peep(W, 1, dir), *p_og = G.w_peep(W, 2, dir);

    // The error recursion runs against the direction's forward order.
    for (int step = 0; step < T; ++step) {
        const int t = dir ? step : (T - 1 - step);
        const int later = dir ? t - 1 : t + 1;    // the slot handled in the previous iteration
        const int earlier = dir ? t + 1 : t - 1;  // the slot the forward pass came from
        const bool first = (step == 0);
        const bool last = (step == T - 1);
        const bool check = (t >= G.Tmin);
        if (!first)
            for (int g = 0; g < 4; ++g)
                orc::mat_product(st->herr + (size_t)t * n, H, S, H, G.w_int(W, g, dir), false,
                                 delta[g] + (size_t)later * n, false, true);
        for (int s = 0; s < S; ++s) {
            const bool dummy = check && pat[t * S + s] == orc::PAT_NONE;
            for (int j = 0; j < H; ++j) {
                const size_t i = (size_t)t * n + (size_t)s * H + j;
                if (dummy) {
                    st->dni[i] = 0.0f; st->dig[i] = 0.0f; st->dfg[i] = 0.0f; st->dog[i] = 0.0f;
                    st->cerr[i] = 0.0f;
                    continue;
                }
                const float e = st->herr[i];
                const float ni = st->ni[i], ig = st->ig[i], og = st->og[i], c = st->c[i];
                const float tc = orc::tanh_act(c);
                // the stored output-gate delta is read back before it is overwritten
                const float d_og = (orc::logistic_deriv(og) * tc * e) + st->dog[i];
                float ce = og * orc::tanh_deriv(tc) * e + p_og[j] * d_og;
                if (!first) {
                    const size_t il = (size_t)later * n + (size_t)s * H + j;
                    ce += (st->fg[il] * st->cerr[il] + p_ig[j] * st->dig[il] + p_fg[j] * st->dfg[il]);
                }
                const float d_ni = ig * orc::tanh_deriv(ni) * ce;
                float d_fg = 0.0f;
                if (!last) {
                    const size_t ie = (size_t)earlier * n + (size_t)s * H + j;
                    d_fg = orc::logistic_deriv(st->fg[i]) * st->c[ie] * ce;
                }
                const float d_ig = orc::logistic_deriv(ig) * ni * ce;
                st->dni[i] = orc::clip1(d_ni);
                st->dig[i] = orc::clip1(d_ig);
                st->dfg[i] = orc::clip1(d_fg);
                st->dog[i] = orc::clip1(d_og);
                st->cerr[i] = ce;
            }
        }
    }
}

// One weight = one pattern-ordered sum, as in the reference's per-weight functor.
void weight_updates(const Geometry &G, const float *x, orc_lstm_dir *const dirs[2], float *dW) {
    const int P = G.P, L = G.L, H = G.H, S = G.S;
    const int N = G.T * S;
    for (int dir = 0; dir < G.ndir; ++dir) {
        const orc_lstm_dir *st = dirs[dir];
        const float *delta[4] = {st->dni, st->dig, st->dfg, st->dog};
        for (int g = 0; g < 4; ++g) {
            const float *dl = delta[g];
            // input weights
#pragma omp parallel for collapse(2) schedule(static) num_threads(orc::threads()) if (orc::threads() > 1)
            for (int u = 0; u < H; ++u)
                for (int p = 0; p < P; ++p) {
                    float wu = 0.0f;
                    for (int i = 0; i < N; ++i) wu += x[p + (size_t)i * P] * dl[u + (size_t)i * H];
                    dW[(size_t)g * P * L + (size_t)(dir * H + u) * P + p] = wu;
                }
            // bias weights
            for (int u = 0; u < H; ++u) {
                float wu = 0.0f;
                for (int i = 0; i < N; ++i) wu += G.bias * dl[u + (size_t)i * H];
                dW[G.off_bias + (size_t)g * L + dir * H + u] = wu;
            }
            // recurrent weights: source is the block output of the step the forward pass came from
#pragma omp parallel for collapse(2) schedule(static) num_threads(orc::threads()) if (orc::threads() > 1)
            for (int u = 0; u < H; ++u)
                for (int src = 0; src < H; ++src) {
                    float wu = 0.0f;
                    if (dir == 0) {
                        for (int i = S; i < N; ++i) wu += st->h[src + (size_t)(i - S) * H] * dl[u + (size_t)i * H];
                    } else {
                        for (int i = 0; i < N - S; ++i) wu += st->h[src + (size_t)(i + S) * H] * dl[u + (size_t)i * H];
                    }
                    dW[G.off_int + (size_t)g * L * H + (size_t)dir * H * H + (size_t)u * H + src] = wu;
                }
        }
        // peepholes: input and forget gate see the earlier cell state, the output gate the current one
        for (int k = 0; k < 3; ++k) {
            const float *dl = delta[k + 1];
            for (int u = 0; u < H; ++u) {
                float wu = 0.0f;
                if (k == 2) {
                    for (int i = 0; i < N; ++i) wu += st->c[u + (size_t)i * H] * dl[u + (size_t)i * H];
                } else if (dir == 0) {
                    for (int i = S; i < N; ++i) wu += st->c[u + (size_t)(i - S) * H] * dl[u + (size_t)i * H];
                } else {
                    for (int i = 0; i < N - S; ++i) wu += st->c[u + (size_t)(i + S) * H] * dl[u + (size_t)i * H];
                }
                dW[G.off_peep + (size_t)k * L + dir * H + u] = wu;
            }
        }
    }
}

}  // namespace

extern "C" {

long orc_lstm_weight_count(int P, int L, int bidir) {
    const long H = L / (bidir ? 2 : 1);
    return 4L * P * L + 4L * L + 4L * L * H + 3L * L;
}

void orc_lstm_forward(const orc_lstm_desc *d, const float *weights, const char *patTypes, const float *x,
                      orc_lstm_dir *fw, orc_lstm_dir *bw, float *out) {
    const Geometry G(*d);
    forward_direction(G, weights, patTypes, x, fw, 0);
    if (G.ndir == 2) {
        forward_direction(G, weights, patTypes, x, bw, 1);
        const size_t N = (size_t)G.T * G.S;
        for (size_t p = 0; p < N; ++p)
            for (int v = 0; v < G.L; ++v)
                out[p * G.L + v] = (v < G.H) ? fw->h[p * G.H + v] : bw->h[p * G.H + v - G.H];
    } else if (out != fw->h) {
        std::memcpy(out, fw->h, sizeof(float) * (size_t)G.T * G.S * G.H);
    }
}

void orc_lstm_backward(const orc_lstm_desc *d, const float *weights, const char *patTypes, const float *x,
                       const float *outerr, orc_lstm_dir *fw, orc_lstm_dir *bw, float *ex,
                       float *weightUpdates) {
    const Geometry G(*d);
    const size_t N = (size_t)G.T * G.S;
    orc_lstm_dir *dirs[2] = {fw, bw};
    if (G.ndir == 2) {
        for (size_t p = 0; p < N; ++p)
            for (int v = 0; v < G.L; ++v) {
                if (v < G.H) fw->herr[p * G.H + v] = outerr[p * G.L + v];
                else bw->herr[p * G.H + v - G.H] = outerr[p * G.L + v];
            }
    } else if (outerr != fw->herr) {
        std::memcpy(fw->herr, outerr, sizeof(float) * N * G.H);
    }
    for (int dir = 0; dir < G.ndir; ++dir) backward_direction(G, weights, patTypes, dirs[dir], dir);

    if (ex) {
        bool assigned = false;
        for (int dir = 0; dir < G.ndir; ++dir) {
            const float *delta[4] = {dirs[dir]->dni, dirs[dir]->dig, dirs[dir]->dfg, dirs[dir]->dog};
            for (int g = 0; g < 4; ++g) {
                orc::mat_product(ex, G.P, (int)N, G.H, G.w_in(weights, g, dir), false, delta[g], false, assigned);
                assigned = true;
            }
        }
    }
    weight_updates(G, x, dirs, weightUpdates);
}

void orc_set_threads(int n) { g_threads = n < 1 ? 1 : n; }
int orc_get_threads() { return g_threads; }

float orc_logistic(float x) { return orc::logistic(x); }
float orc_tanh(float x) { return orc::tanh_act(x); }
float orc_safe_exp(float x) { return orc::safe_exp(x); }
float orc_safe_log(float x) { return orc::safe_log(x); }
float orc_log_add(float x, float y) { return orc::log_add(x, y); }

void orc_mat_product(float *C, int m, int n, int k, const float *A, int tA, const float *B, int tB,
                     int accumulate) {
    orc::mat_product(C, m, n, k, A, tA != 0, B, tB != 0, accumulate != 0);
}

}  // extern "C"
