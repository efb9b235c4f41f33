/*
 * TEST INFRASTRUCTURE ONLY - body of the CPU oracle, included twice by
 * cs_oracle.c: once with REAL = float (the opmath type ATen uses for float,
 * half and bfloat16 storage) and once with REAL = double.  FN(name) appends
 * the suffix (_f32 / _f64).
 *
 * Every function restates, in scalar C, what one reference task body
 * computes; file:line citations are into the CoreScheduler tree.  Where the
 * task body is a single ATen call the formula is ATen's documented one and
 * the tests pin this file against the installed ATen CPU kernels.
 *
 * Row and column sums are accumulated in double and narrowed to REAL once:
 * the result is the correctly rounded statistic that every fp32 summation
 * order approximates, so it can judge any of them.
 */

/* ---- AdamW: src/optimizer/adamw.cu:45-59 (plain), :72-89 (amsgrad) ------
 * Operation order and types as the kernel: everything in REAL, m and v are
 * stored back and the update continues from the unrounded values.  The bias
 * corrections come from the host in double and are narrowed (adamw.cu:116-117). */
void FN(oracle_adamw_step)(REAL *w, const REAL *dw, REAL *m, REAL *v, REAL *v_max, int64_t n,
                           double lr_d, double beta1_d, double beta2_d, double eps_d,
                           double wd_d, int64_t t) {
  const REAL lr = (REAL)lr_d, beta1 = (REAL)beta1_d, beta2 = (REAL)beta2_d, eps = (REAL)eps_d,
             wd = (REAL)wd_d;
  const REAL inv_bc1 = (REAL)(1. / (1. - pow(beta1_d, (double)t)));
  const REAL inv_bc2 = (REAL)(1. / (1. - pow(beta2_d, (double)t)));
  const REAL one = (REAL)1;
  for (int64_t i = 0; i < n; ++i) {
    const REAL g_t = dw[i];
    const REAL theta_t = w[i] - lr * wd * w[i];
    const REAL m_t = beta1 * m[i] + (one - beta1) * g_t;
    m[i] = m_t;
    const REAL v_t = beta2 * v[i] + (one - beta2) * g_t * g_t;
    v[i] = v_t;
    const REAL m_hat_t = m_t * inv_bc1;
    REAL v_hat_t = v_t * inv_bc2;
    if (v_max) {
      v_hat_t = v_max[i] > v_hat_t ? v_max[i] : v_hat_t;
      v_max[i] = v_hat_t;
    }
    w[i] = theta_t - lr * m_hat_t / (SQRT(v_hat_t) + eps);
  }
}

/* ---- gradient clipping: src/compute/utils.cpp:700-746 (Utils::clip_grad_norm_)
 * total = || hstack(all gradients) ||_p for p = 2 (inf_norm == 0) or +infinity
 * (inf_norm != 0); coefficient = min(1, max_norm / (total + 1e-6)) in the tensors'
 * arithmetic type; every gradient is multiplied by it in place when `scale` is set.
 * The sum of squares is accumulated in double and narrowed once (see the header). */
void FN(oracle_clip_grad_norm)(REAL *const *grads, const int64_t *sizes, int64_t n_tensors,
                               int inf_norm, double max_norm_d, int scale, REAL *total_norm,
                               REAL *clip_coef) {
  double acc = 0.;
  for (int64_t t = 0; t < n_tensors; ++t) {
    for (int64_t i = 0; i < sizes[t]; ++i) {
      const double g = (double)grads[t][i];
      if (inf_norm) {
        acc = fabs(g) > acc ? fabs(g) : acc;
      } else {
        acc += g * g;
      }
    }
  }
  const REAL total = (REAL)(inf_norm ? acc : sqrt(acc));
  REAL coef = (REAL)max_norm_d / (total + (REAL)1e-6);
  if (coef > (REAL)1) coef = (REAL)1;
  *total_norm = total;
  *clip_coef = coef;
  if (scale) {
    for (int64_t t = 0; t < n_tensors; ++t)
      for (int64_t i = 0; i < sizes[t]; ++i) grads[t][i] = grads[t][i] * coef;
  }
}

/* ---- GeLU: src/compute/gelu.cpp:39 (at::gelu), :61-62 (at::gelu_backward)
 * mode 0 = exact: x * 0.5 * (1 + erf(x / sqrt 2)); derivative cdf + x * pdf.
 * mode 1 = at::gelu(x, "tanh"): 0.5 x (1 + tanh(kBeta (x + kKappa x^3))),
 * kBeta = sqrt(2) * (2/sqrt(pi)) * 0.5, kKappa = 0.044715 (ATen Gelu.h). */
void FN(oracle_gelu_forward)(const REAL *x, REAL *y, int64_t n, int mode) {
  const REAL kBeta = (REAL)(M_SQRT2 * M_2_SQRTPI * 0.5), kKappa = (REAL)0.044715;
  for (int64_t i = 0; i < n; ++i) {
    const REAL xi = x[i];
    if (mode == 0) {
      y[i] = xi * (REAL)0.5 * ((REAL)1 + ERF(xi * (REAL)M_SQRT1_2));
    } else {
      const REAL inner = kBeta * (xi + kKappa * (xi * xi * xi));
      y[i] = (REAL)0.5 * xi * ((REAL)1 + TANH(inner));
    }
  }
}

void FN(oracle_gelu_backward)(const REAL *dy, const REAL *x, REAL *dx, int64_t n, int mode) {
  const REAL kBeta = (REAL)(M_SQRT2 * M_2_SQRTPI * 0.5), kKappa = (REAL)0.044715;
  for (int64_t i = 0; i < n; ++i) {
    const REAL xi = x[i];
    if (mode == 0) {
      const REAL cdf = (REAL)0.5 * ((REAL)1 + ERF(xi * (REAL)M_SQRT1_2));
      const REAL pdf = EXP((REAL)-0.5 * xi * xi) * (REAL)(M_2_SQRTPI * M_SQRT1_2 * 0.5);
      dx[i] = dy[i] * (cdf + xi * pdf);
    } else {
      const REAL x_sq = xi * xi;
      const REAL inner = kBeta * (xi + kKappa * (x_sq * xi));
      const REAL th = TANH(inner);
      const REAL left = (REAL)0.5 * xi, right = (REAL)1 + th;
      const REAL left_d = (REAL)0.5 * right;
      const REAL tanh_d = (REAL)1 - th * th;
      const REAL inner_d = kBeta * ((REAL)1 + (REAL)3 * kKappa * x_sq);
      dx[i] = dy[i] * (left_d + left * tanh_d * inner_d);
    }
  }
}

/* ---- LayerNorm forward: at::native_layer_norm, src/compute/layer_norm.cpp:163-169
 * mean, biased variance, rstd = 1/sqrt(var + eps); y = (x-mean)*rstd*gamma + beta.
 * beta may be NULL (the bias=false path, :198-204). */
void FN(oracle_layernorm_forward)(const REAL *x, const REAL *gamma, const REAL *beta, REAL *y,
                                  REAL *mean, REAL *rstd, int64_t rows, int64_t C, double eps) {
  for (int64_t r = 0; r < rows; ++r) {
    const REAL *xr = x + r * C;
    double s = 0;
    for (int64_t c = 0; c < C; ++c) s += xr[c];
    const double mu = s / (double)C;
    double q = 0;
    for (int64_t c = 0; c < C; ++c) q += (xr[c] - mu) * (xr[c] - mu);
    const double rs = 1.0 / sqrt(q / (double)C + eps);
    mean[r] = (REAL)mu;
    rstd[r] = (REAL)rs;
    for (int64_t c = 0; c < C; ++c) {
      const REAL xh = (xr[c] - (REAL)mu) * (REAL)rs;
      y[r * C + c] = xh * gamma[c] + (beta ? beta[c] : (REAL)0);
    }
  }
}

/* ---- LayerNorm backward: at::native_layer_norm_backward,
 * src/compute/layer_norm.cpp:263-266 (dx) and :321-334 (dgamma, dbeta; += into
 * an existing gradient when accumulate is set).  Any output may be NULL. */
void FN(oracle_layernorm_backward)(const REAL *dy, const REAL *x, const REAL *mean,
                                   const REAL *rstd, const REAL *gamma, REAL *dx, REAL *dgamma,
                                   REAL *dbeta, int64_t rows, int64_t C, int accumulate) {
  double *ag = (double *)calloc((size_t)C, sizeof(double));
  double *ab = (double *)calloc((size_t)C, sizeof(double));
  for (int64_t r = 0; r < rows; ++r) {
    const REAL *dyr = dy + r * C, *xr = x + r * C;
    const double mu = mean[r], rs = rstd[r];
    double s1 = 0, s2 = 0;
    for (int64_t c = 0; c < C; ++c) {
      const double xh = (xr[c] - mu) * rs;
      const double g = gamma ? (double)dyr[c] * gamma[c] : (double)dyr[c];
      s1 += g;
      s2 += g * xh;
      ag[c] += (double)dyr[c] * xh;
      ab[c] += dyr[c];
    }
    s1 /= (double)C;
    s2 /= (double)C;
    if (dx) {
      for (int64_t c = 0; c < C; ++c) {
        const double xh = (xr[c] - mu) * rs;
        const double g = gamma ? (double)dyr[c] * gamma[c] : (double)dyr[c];
        dx[r * C + c] = (REAL)(rs * (g - s1 - xh * s2));
      }
    }
  }
  for (int64_t c = 0; c < C; ++c) {
    if (dgamma) dgamma[c] = (REAL)(ag[c] + (accumulate ? (double)dgamma[c] : 0.0));
    if (dbeta) dbeta[c] = (REAL)(ab[c] + (accumulate ? (double)dbeta[c] : 0.0));
  }
  free(ag);
  free(ab);
}

/* ---- Embedding forward: torch::embedding, src/compute/embedding.cpp:117-121
 * A copy.  An index outside [0, V) gives a zero row (the GPU library's
 * documented choice; ATen raises instead). */
void FN(oracle_embedding_forward)(const REAL *weight, const int64_t *ids, REAL *out, int64_t n,
                                  int64_t C, int64_t V) {
  for (int64_t i = 0; i < n; ++i) {
    const int64_t id = ids[i];
    for (int64_t c = 0; c < C; ++c)
      out[i * C + c] = (id >= 0 && id < V) ? weight[id * C + c] : (REAL)0;
  }
}

/* token + position: two gathers, broadcast_to and add,
 * example/gpt2/gpt2_single_device.cpp:541-545 */
void FN(oracle_embedding_forward_add)(const REAL *wte, const REAL *wpe, const int64_t *ids,
                                      REAL *out, int64_t B, int64_t T, int64_t C, int64_t V) {
  for (int64_t b = 0; b < B; ++b)
    for (int64_t t = 0; t < T; ++t) {
      const int64_t i = b * T + t, id = ids[i];
      for (int64_t c = 0; c < C; ++c)
        out[i * C + c] = (id >= 0 && id < V) ? wte[id * C + c] + wpe[t * C + c] : (REAL)0;
    }
}

/* ---- Embedding backward: at::embedding_backward (dense, with and without
 * scale_grad_by_freq) and the += of an existing gradient,
 * src/compute/embedding.cpp:147-157.  Rows equal to padding_idx get nothing;
 * padding_idx < 0 means none. */
void FN(oracle_embedding_backward)(const REAL *dout, const int64_t *ids, REAL *dweight,
                                   int64_t n, int64_t C, int64_t V, int64_t padding_idx,
                                   int accumulate, int scale_grad_by_freq) {
  double *acc = (double *)calloc((size_t)(V * C), sizeof(double));
  int64_t *count = (int64_t *)calloc((size_t)V, sizeof(int64_t));
  for (int64_t i = 0; i < n; ++i) {
    const int64_t id = ids[i];
    if (id < 0 || id >= V || id == padding_idx) continue;
    count[id] += 1;
    for (int64_t c = 0; c < C; ++c) acc[id * C + c] += dout[i * C + c];
  }
  /* scale_grad_by_freq: every contribution to row k weighs 1 / (entries naming k) */
  for (int64_t k = 0; k < V * C; ++k) {
    const double scale = (scale_grad_by_freq && count[k / C] > 0) ? 1.0 / (double)count[k / C] : 1.0;
    dweight[k] = (REAL)(acc[k] * scale + (accumulate ? (double)dweight[k] : 0.0));
  }
  free(count);
  free(acc);
}

/* Utils::sum(dx, 0) then wpe->backward with arange positions,
 * example/gpt2/gpt2_single_device.cpp:565-566 */
void FN(oracle_embedding_backward_positions)(const REAL *dout, REAL *dwpe, int64_t B, int64_t T,
                                             int64_t C, int accumulate) {
  for (int64_t f = 0; f < T * C; ++f) {
    double a = accumulate ? (double)dwpe[f] : 0.0;
    for (int64_t b = 0; b < B; ++b) a += dout[b * T * C + f];
    dwpe[f] = (REAL)a;
  }
}

/* ---- Cross entropy: at::log_softmax + at::nll_loss_forward
 * (src/compute/cross_entropy.cpp:57-63), then at::nll_loss_backward with
 * ones_like(loss) + at::_log_softmax_backward_data (:103-109).
 * logits [N, stride], classes are columns [0, V).  reduction: 0 none, 1 mean,
 * 2 sum (at::Reduction).  row_loss [N]; loss 1 value (mean / sum);
 * total_weight = rows not ignored; dlogits [N, stride] or NULL, with
 * dlogits = (softmax - onehot) * dloss / total_weight (mean) or * dloss.
 * A target outside [0, V) that is not ignore_index is treated as ignored
 * (the GPU library's documented choice; ATen raises instead). */
void FN(oracle_cross_entropy)(const REAL *logits, const int64_t *targets, REAL *row_loss,
                              REAL *loss, REAL *total_weight, REAL *dlogits, int64_t N, int64_t V,
                              int64_t stride, int64_t ignore_index, int reduction, double dloss,
                              const REAL *class_weight) {
  /* class_weight (at::nll_loss's `weight`, src/compute/cross_entropy.cpp:52-63; NULL: all 1):
   * a row's loss and gradient carry the weight of its target, the mean is over the sum of
   * those weights, which is also what total_weight returns */
  double count = 0;
  for (int64_t i = 0; i < N; ++i) {
    const int64_t t = targets[i];
    if (t != ignore_index && t >= 0 && t < V) count += class_weight ? (double)class_weight[t] : 1.0;
  }
  const double scale = reduction == 1 ? dloss / count : dloss;
  double total = 0;
  for (int64_t i = 0; i < N; ++i) {
    const REAL *x = logits + i * stride;
    const int64_t t = targets[i];
    const int live = t != ignore_index && t >= 0 && t < V;
    if (!live) {
      if (row_loss) row_loss[i] = (REAL)0;
      if (dlogits)
        for (int64_t c = 0; c < stride; ++c) dlogits[i * stride + c] = (REAL)0;
      continue;
    }
    const double w = class_weight ? (double)class_weight[t] : 1.0;
    double mx = x[0];
    for (int64_t c = 1; c < V; ++c) mx = x[c] > mx ? x[c] : mx;
    double s = 0;
    for (int64_t c = 0; c < V; ++c) s += exp((double)x[c] - mx);
    const double lse = mx + log(s);
    const double li = (lse - (double)x[t]) * w;
    if (row_loss) row_loss[i] = (REAL)li;
    total += li;
    if (dlogits) {
      for (int64_t c = 0; c < stride; ++c) {
        double o = 0;
        if (c < V) o = (exp((double)x[c] - lse) - (c == t ? 1.0 : 0.0)) * scale * w;
        dlogits[i * stride + c] = (REAL)o;
      }
    }
  }
  if (loss) *loss = (REAL)(reduction == 1 ? total / count : total);
  if (total_weight) *total_weight = (REAL)count;
}
