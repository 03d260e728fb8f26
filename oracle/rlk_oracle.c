/*
 * Double-precision C restatement of the fused linear-logprob path.
 * TEST INFRASTRUCTURE ONLY: loaded by tests/, __graft_entry__.smoke() and the
 * cpu_baseline leg of bench.py; never by the product package.
 *
 * It is deliberately written as naive loops so that it shares no code, no
 * blocking and no library routine with either the torch restatement
 * (oracle/oracle.py) or the HIP kernels: agreement between the three is the
 * pin.  Reference lines each routine follows are cited per function (paths are
 * relative to the reference tree).
 *
 * Parity pins: tests/test_oracle_pins.py checks these routines against the
 * known answers held by the reference's own tests
 * (tests/test_reference_ops.py:18-28,60-71,79-105; tests/test_grpo_loss.py:110-117).
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>

/* z = (h.W^T + b)/T ; logp = z_t - logsumexp(z) ; ignored rows -> 0.
 * rl_engine/kernels/ops/pytorch/loss/linear_logp.py:514-520 and
 * rl_engine/testing/reference_ops.py:15-47 (temperature, ignore-index). */
int rlk_oracle_linear_logp_f64(const double *hidden, const double *weight, const double *bias,
                               const int64_t *targets, int64_t n, int64_t h, int64_t v,
                               double temperature, int64_t ignore_index, int use_ignore,
                               double *logp, double *lse)
{
    if (!(temperature > 0.0)) return -1;
    double *z = (double *)malloc(sizeof(double) * (size_t)v);
    if (!z) return -2;
    for (int64_t r = 0; r < n; ++r) {
        double zmax = -INFINITY;
        for (int64_t c = 0; c < v; ++c) {
            double acc = 0.0;
            for (int64_t k = 0; k < h; ++k) acc += hidden[r * h + k] * weight[c * h + k];
            if (bias) acc += bias[c];
            z[c] = acc / temperature;
            if (z[c] > zmax) zmax = z[c];
        }
        double s = 0.0;
        for (int64_t c = 0; c < v; ++c) s += exp(z[c] - zmax);
        double l = zmax + log(s);
        if (lse) lse[r] = l;
        int64_t t = targets[r];
        if (use_ignore && t == ignore_index) {
            logp[r] = 0.0;
        } else if (t < 0 || t >= v) {
            free(z);
            return -3;
        } else {
            logp[r] = z[t] - l;
        }
    }
    free(z);
    return 0;
}

/* dz = g (onehot - softmax(z)) / T ; dH = dz W ; dW = dz^T H ; db = sum_rows dz.
 * rl_engine/kernels/ops/pytorch/loss/linear_logp.py:408-434. */
int rlk_oracle_linear_logp_bwd_f64(const double *grad, const double *hidden, const double *weight,
                                   const double *bias, const int64_t *targets, int64_t n,
                                   int64_t h, int64_t v, double temperature, int64_t ignore_index,
                                   int use_ignore, double *d_hidden, double *d_weight,
                                   double *d_bias)
{
    if (!(temperature > 0.0)) return -1;
    double *z = (double *)malloc(sizeof(double) * (size_t)v);
    if (!z) return -2;
    for (int64_t i = 0; i < v * h; ++i) d_weight[i] = 0.0;
    if (d_bias)
        for (int64_t c = 0; c < v; ++c) d_bias[c] = 0.0;
    for (int64_t r = 0; r < n; ++r) {
        for (int64_t k = 0; k < h; ++k) d_hidden[r * h + k] = 0.0;
        int64_t t = targets[r];
        double g = grad[r];
        if (use_ignore && t == ignore_index) continue;
        if (t < 0 || t >= v) {
            free(z);
            return -3;
        }
        double zmax = -INFINITY;
        for (int64_t c = 0; c < v; ++c) {
            double acc = 0.0;
            for (int64_t k = 0; k < h; ++k) acc += hidden[r * h + k] * weight[c * h + k];
            if (bias) acc += bias[c];
            z[c] = acc / temperature;
            if (z[c] > zmax) zmax = z[c];
        }
        double s = 0.0;
        for (int64_t c = 0; c < v; ++c) s += exp(z[c] - zmax);
        for (int64_t c = 0; c < v; ++c) {
            double p = exp(z[c] - zmax) / s;
            double dz = g * ((c == t ? 1.0 : 0.0) - p) / temperature;
            if (d_bias) d_bias[c] += dz;
            for (int64_t k = 0; k < h; ++k) {
                d_hidden[r * h + k] += dz * weight[c * h + k];
                d_weight[c * h + k] += dz * hidden[r * h + k];
            }
        }
    }
    free(z);
    return 0;
}

/* logits -> selected logp; out-of-range target -> 0
 * (csrc/fused_logp_kernel.cu:147-155). */
void rlk_oracle_logp_from_logits_f64(const double *logits, const int64_t *ids, int64_t n,
                                     int64_t v, double *out)
{
    for (int64_t r = 0; r < n; ++r) {
        const double *row = logits + r * v;
        double m = -INFINITY;
        for (int64_t c = 0; c < v; ++c)
            if (row[c] > m) m = row[c];
        double s = 0.0;
        for (int64_t c = 0; c < v; ++c) s += exp(row[c] - m);
        int64_t t = ids[r];
        out[r] = (t >= 0 && t < v) ? row[t] - m - log(s) : 0.0;
    }
}

/* Per-group (x - mean)/sqrt(max(E[x^2]-mean^2, eps^2)) over CSR boundaries.
 * rl_engine/kernels/ops/pytorch/loss/grpo_loss.py:70-84. */
void rlk_oracle_group_advantages_f64(const double *rewards, const int64_t *bounds,
                                     int64_t num_groups, double eps, double *adv)
{
    for (int64_t g = 0; g < num_groups; ++g) {
        double s1 = 0.0, s2 = 0.0;
        int64_t a = bounds[g], b = bounds[g + 1];
        for (int64_t i = a; i < b; ++i) {
            s1 += rewards[i];
            s2 += rewards[i] * rewards[i];
        }
        double cnt = (double)(b - a);
        double mean = s1 / cnt;
        double var = s2 / cnt - mean * mean;
        if (var < eps * eps) var = eps * eps;
        double sd = sqrt(var);
        for (int64_t i = a; i < b; ++i) adv[i] = (rewards[i] - mean) / sd;
    }
}

/* loss = mean_mask(-min(rA, clip(r)A)) + beta*mean_mask(e^d - d - 1), and dloss/dcur.
 * rl_engine/testing/reference_ops.py:71-106 chained as in
 * rl_engine/kernels/ops/pytorch/loss/grpo_loss.py:110-125.
 * out3 = {loss, policy_loss, kl}. */
void rlk_oracle_grpo_from_logp_f64(const double *cur, const double *old_lp, const double *ref_lp,
                                   const double *adv_tok, const uint8_t *mask, int64_t n,
                                   double clip_eps, double beta, double *out3, double *dcur)
{
    double cnt = 0.0, pol = 0.0, kl = 0.0;
    const double lo = 1.0 - clip_eps, hi = 1.0 + clip_eps;
    for (int64_t i = 0; i < n; ++i)
        if (mask[i]) cnt += 1.0;
    double denom = cnt < 1e-8 ? 1e-8 : cnt;
    for (int64_t i = 0; i < n; ++i) {
        if (!mask[i]) {
            if (dcur) dcur[i] = 0.0;
            continue;
        }
        double r = exp(cur[i] - old_lp[i]);
        double rc = r < lo ? lo : (r > hi ? hi : r);
        double a = adv_tok[i];
        double un = r * a, cl = rc * a;
        pol += -(un < cl ? un : cl);
        double d = ref_lp[i] - cur[i];
        kl += exp(d) - d - 1.0;
        if (dcur) {
            double inside = (r >= lo && r <= hi) ? 1.0 : 0.0;
            double w_un = un < cl ? 1.0 : (un == cl ? 0.5 : 0.0);
            double gp = -(w_un * a * r + (1.0 - w_un) * a * r * inside);
            dcur[i] = (gp + beta * (1.0 - exp(d))) / denom;
        }
    }
    out3[1] = pol / denom;
    out3[2] = kl / denom;
    out3[0] = out3[1] + beta * out3[2];
}
