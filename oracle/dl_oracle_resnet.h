/* TEST INFRASTRUCTURE — whole-network restatement for layer lists that contain
 * the reference's residual blocks (pre-activation ResNet form), float only.
 * Included at the end of dl_oracle.c; uses the _f32 leaves defined there.
 *
 * A list entry is {LAYER::FULLY_CONNECTED, units} or {LAYER::RESIDUAL, depth}; a
 * RESIDUAL entry is followed by `depth` fully-connected entries, the layers of
 * its block (compile.cpp:127-170, run/deep-learning/v1/custom.cpp:449-470).  The
 * zero-padding of the shortcut is derived from the widths (compile.cpp:495-510).  What the reference does with it (paths under lib/deep-learning/
 * v1/learner/):
 *
 *  forward of a block layer, K -> H (Forward_Pass__Residual__FC__Loop,
 *  fwp_st.cpp:4049-4442): [normalization of the INPUT, K units] -> [activation
 *  and dropout of that, K units each; skipped for the first layer of the block]
 *  -> weights (+ bias when not normalized).  The layer's output is its summation.
 *  forward of the block (Forward_Pass__Residual__Loop, fwp_st.cpp:3876-4010):
 *  the layers in turn, [block-level normalization of the last layer's output],
 *  then the zero-padded identity shortcut with the output of the layer that
 *  feeds the block (fwp_st.cpp:5051-5112).
 *  backward (bwp_st.cpp:80-185, 345-541, 1112-1175): the transposed chain; the
 *  activation derivative sees the post-dropout values and the gradient is not
 *  masked, as everywhere in the reference.
 *
 *  Unit counts, hence the parameter layout (allocate.cpp:1150-1330,
 *  compile.cpp:283-520): normalization / activation / dropout units of a block
 *  layer are as many as its INPUTS; a RESIDUAL entry has as many normalization
 *  units as its block's last layer has outputs, max(shortcut width, that) outputs
 *  and no weights or bias.  Parameters: [weights of every FC layer | biases of
 *  every FC layer | gamma of every entry | beta of every entry].
 */
#define DLO_LAYER_FC 3
#define DLO_LAYER_RESIDUAL 9

typedef struct {
  size_t n_layers;
  int *type;         /* [n] LAYER::TYPE */
  size_t *n_out;     /* [n] outputs of the entry */
  size_t *n_in;      /* [n] inputs of an FC entry (0 for entry 0 and RESIDUAL) */
  size_t *n_unit;    /* [n] normalization (= activation = dropout) units */
  size_t *feed;      /* [n] index of the entry whose outputs are this entry's input */
  size_t *depth, *padding; /* RESIDUAL entries */
  int *in_block, *block_first; /* FC entries inside a block / first of its block */
  int *act, *norm, *drop;
  float *keep;
  uint8_t **mask;    /* [n][n_unit] */
  float momentum, eps, r_max, d_max;
  size_t P, n_units_total, n_weights, n_bias;
  size_t *w_off, *b_off, *u_off;
  float *param, *dparam, *mov_mean, *mov_std;
  size_t max_batch;
  /* [max_batch, .] buffers per entry */
  float **out;    /* outputs [n_out] */
  float **Z;      /* summations [n_out] (FC) */
  float **xhat, **nrm; /* normalization buffers [n_unit] */
  float **tin;    /* block layer: what the weights see [n_in] */
  float **dOut;   /* gradient with respect to the outputs [n_out] */
  float **dZ;     /* gradient with respect to the summations [n_out] (FC) */
  float **mean, **stdv, **r, **d; /* [n_unit] */
  float *X0;
  double loss_sum, n_correct;
} dlo_net;

static size_t dlo_net_max(size_t a, size_t b) { return a > b ? a : b; }

void dlo_net_destroy(dlo_net *m);

dlo_net *dlo_net_create(size_t n, int const *types, size_t const *units, size_t const *padding) {
  dlo_net *m = (dlo_net *)calloc(1, sizeof(dlo_net));
  m->n_layers = n;
#define DLO_NET_ARR(field, T) m->field = (T *)calloc(n, sizeof(T))
  DLO_NET_ARR(type, int); DLO_NET_ARR(n_out, size_t); DLO_NET_ARR(n_in, size_t); DLO_NET_ARR(n_unit, size_t);
  DLO_NET_ARR(feed, size_t); DLO_NET_ARR(depth, size_t); DLO_NET_ARR(padding, size_t);
  DLO_NET_ARR(in_block, int); DLO_NET_ARR(block_first, int);
  DLO_NET_ARR(act, int); DLO_NET_ARR(norm, int); DLO_NET_ARR(drop, int); DLO_NET_ARR(keep, float);
  DLO_NET_ARR(mask, uint8_t *); DLO_NET_ARR(w_off, size_t); DLO_NET_ARR(b_off, size_t); DLO_NET_ARR(u_off, size_t);
#undef DLO_NET_ARR
  /* pass 1: types, feeding entries, sizes */
  size_t prev_feed = 0; /* entry whose outputs feed the next entry */
  for (size_t l = 0; l < n; ++l) {
    m->type[l] = types[l];
    m->act[l] = 18;
  }
  m->n_out[0] = m->n_unit[0] = units[0];
  for (size_t l = 1; l < n;) {
    if (types[l] == DLO_LAYER_RESIDUAL) {
      size_t const r = l, D = units[l];
      m->depth[r] = D;
      (void)padding; /* the reference derives it from the two widths, below */
      m->feed[r] = prev_feed;
      size_t cur = prev_feed;
      for (size_t d2 = 1; d2 <= D; ++d2) {
        size_t const i = r + d2;
        m->in_block[i] = 1;
        m->block_first[i] = d2 == 1;
        m->feed[i] = cur;
        m->n_in[i] = m->n_out[cur];
        m->n_out[i] = units[i];
        m->n_unit[i] = m->n_in[i];
        cur = i;
      }
      m->n_unit[r] = m->n_out[r + D];
      m->n_out[r] = dlo_net_max(m->n_out[prev_feed], m->n_out[r + D]);
      /* compile.cpp:495-510: padding = (|shortcut width - block width| + 1) / 2 */
      {
        size_t const a = m->n_out[prev_feed], b = m->n_out[r + D];
        m->padding[r] = ((a > b ? a - b : b - a) + 1) / 2;
      }
      prev_feed = r;
      l = r + D + 1;
    } else {
      m->feed[l] = prev_feed;
      m->n_in[l] = m->n_out[prev_feed];
      m->n_out[l] = m->n_unit[l] = units[l];
      prev_feed = l;
      ++l;
    }
  }
  /* pass 2: offsets */
  size_t nw = 0, nb = 0, nu = 0;
  for (size_t l = 0; l < n; ++l) {
    m->u_off[l] = nu;
    nu += m->n_unit[l];
    if (l > 0 && m->type[l] == DLO_LAYER_FC) {
      m->w_off[l] = nw;
      nw += m->n_out[l] * m->n_in[l];
    }
  }
  for (size_t l = 1; l < n; ++l)
    if (m->type[l] == DLO_LAYER_FC) {
      m->b_off[l] = nw + nb;
      nb += m->n_out[l];
    }
  m->n_weights = nw; m->n_bias = nb; m->n_units_total = nu;
  m->P = nw + nb + 2 * nu;
  m->param = (float *)calloc(m->P, sizeof(float));
  m->dparam = (float *)calloc(m->P, sizeof(float));
  m->mov_mean = (float *)calloc(nu, sizeof(float));
  m->mov_std = (float *)calloc(nu, sizeof(float));
  for (size_t i = 0; i < nu; ++i) {
    m->param[nw + nb + i] = 1.0f;
    m->mov_std[i] = 1.0f;
  }
  m->momentum = 0.999f; m->eps = 1e-5f; m->r_max = 1.0f; m->d_max = 0.0f;
  return m;
}

size_t dlo_net_total_parameters(dlo_net const *m) { return m->P; }
size_t dlo_net_total_units(dlo_net const *m) { return m->n_units_total; }
/* out[0] type, [1] outputs, [2] first weight index, [3] one past the last, [4] bias
 * index, [5] uses a bias, [6] normalization units, [7] gamma index, [8] moving-
 * statistic index, [9] activation units, [10] block depth, [11] padding */
void dlo_net_layer_info(dlo_net const *m, size_t l, size_t *out) {
  int const fc = l > 0 && m->type[l] == DLO_LAYER_FC;
  out[0] = (size_t)m->type[l];
  out[1] = m->n_out[l];
  out[2] = fc ? m->w_off[l] : 0;
  out[3] = fc ? m->w_off[l] + m->n_out[l] * m->n_in[l] : 0;
  out[4] = fc ? m->b_off[l] : 0;
  out[5] = m->norm[l] == DLO_NORM_NONE;
  out[6] = m->n_unit[l];
  out[7] = m->n_weights + m->n_bias + m->u_off[l];
  out[8] = m->u_off[l];
  out[9] = m->type[l] == DLO_LAYER_RESIDUAL ? 0 : (m->in_block[l] ? (m->block_first[l] ? 0 : m->n_unit[l]) : m->n_out[l]);
  out[10] = m->depth[l];
  out[11] = m->padding[l];
}
void dlo_net_set_layer(dlo_net *m, size_t l, int act, int norm, int drop, float keep, uint8_t const *mask) {
  m->act[l] = act; m->norm[l] = norm; m->drop[l] = drop; m->keep[l] = keep;
  free(m->mask[l]);
  m->mask[l] = NULL;
  if (mask) {
    m->mask[l] = (uint8_t *)malloc(m->n_unit[l]);
    memcpy(m->mask[l], mask, m->n_unit[l]);
  }
}
void dlo_net_set_norm_hyper(dlo_net *m, float momentum, float eps, float r_max, float d_max) {
  m->momentum = momentum; m->eps = eps; m->r_max = r_max; m->d_max = d_max;
}
float *dlo_net_parameters(dlo_net *m) { return m->param; }
float *dlo_net_dparameters(dlo_net *m) { return m->dparam; }
float *dlo_net_moving_mean(dlo_net *m) { return m->mov_mean; }
float *dlo_net_moving_std(dlo_net *m) { return m->mov_std; }

static float **dlo_net_alloc(dlo_net const *m, size_t rows, size_t const *width) {
  float **p = (float **)calloc(m->n_layers, sizeof(float *));
  for (size_t l = 0; l < m->n_layers; ++l) p[l] = (float *)calloc((rows ? rows : 1) * (width[l] ? width[l] : 1), sizeof(float));
  return p;
}
static void dlo_net_free(dlo_net const *m, float **p) {
  if (!p) return;
  for (size_t l = 0; l < m->n_layers; ++l) free(p[l]);
  free(p);
}

void dlo_net_prepare(dlo_net *m, size_t B) {
  m->max_batch = B;
  m->out = dlo_net_alloc(m, B, m->n_out);
  m->Z = dlo_net_alloc(m, B, m->n_out);
  m->dOut = dlo_net_alloc(m, B, m->n_out);
  m->dZ = dlo_net_alloc(m, B, m->n_out);
  m->xhat = dlo_net_alloc(m, B, m->n_unit);
  m->nrm = dlo_net_alloc(m, B, m->n_unit);
  m->tin = dlo_net_alloc(m, B, m->n_unit);
  m->mean = dlo_net_alloc(m, 1, m->n_unit);
  m->stdv = dlo_net_alloc(m, 1, m->n_unit);
  m->r = dlo_net_alloc(m, 1, m->n_unit);
  m->d = dlo_net_alloc(m, 1, m->n_unit);
  m->X0 = (float *)calloc(B * m->n_out[0], sizeof(float));
}

/* normalization of x [B, n_unit(l)] with entry l's units -> m->nrm[l] */
static void dlo_net_norm_fwd(dlo_net *m, int nt, int state, size_t B, size_t l, float const *x) {
  size_t const U = m->n_unit[l];
  float const *gamma = m->param + m->n_weights + m->n_bias + m->u_off[l];
  float const *beta = gamma + m->n_units_total;
  if (state >= 1)
    dlo_norm_fwd_train_f32(nt, m->norm[l] == DLO_NORM_BRN, B, U, m->momentum, m->eps, m->r_max, m->d_max, x, gamma, beta,
                           m->mean[l], m->stdv[l], m->mov_mean + m->u_off[l], m->mov_std + m->u_off[l], m->r[l], m->d[l],
                           m->xhat[l], m->nrm[l]);
  else
    dlo_norm_fwd_infer_f32(nt, B, U, x, gamma, beta, m->mov_mean + m->u_off[l], m->mov_std + m->u_off[l], m->nrm[l]);
}
/* dropout of v [B, U] with entry l's settings (fwp_st.cpp:657-732) */
static void dlo_net_dropout(dlo_net *m, int nt, int state, size_t B, size_t l, size_t U, float *v) {
  if (state == 1) {
    if (m->drop[l] == DLO_DROP_BERNOULLI)
      dlo_dropout_fwd_f32(nt, 1, 0, B, U, m->mask[l], 0.0f, v);
    else if (m->drop[l] == DLO_DROP_BERNOULLI_INVERTED)
      dlo_dropout_fwd_f32(nt, 0, 0, B, U, m->mask[l], m->keep[l] == 0.0f ? 0.0f : 1.0f / m->keep[l], v);
  } else if (m->drop[l] == DLO_DROP_BERNOULLI) {
    dlo_dropout_fwd_f32(nt, 2, 0, B, U, NULL, m->keep[l], v);
  }
}

void dlo_net_forward(dlo_net *m, int nt, int state, size_t B, float const *X) {
  size_t const n = m->n_layers;
  memcpy(m->X0, X, B * m->n_out[0] * sizeof(float));
  memcpy(m->out[0], X, B * m->n_out[0] * sizeof(float));
  for (size_t l = 1; l < n; ++l) {
    if (m->type[l] == DLO_LAYER_RESIDUAL) continue; /* finished when its last block layer is */
    size_t const K = m->n_in[l], H = m->n_out[l];
    float const *in = m->out[m->feed[l]];
    float const *W = m->param + m->w_off[l];
    if (m->in_block[l]) {
      /* fwp_st.cpp:4049-4442 */
      float const *t = in;
      if (m->norm[l] != DLO_NORM_NONE) {
        dlo_net_norm_fwd(m, nt, state, B, l, t);
        t = m->nrm[l];
      }
      if (!m->block_first[l]) {
        dlo_act_fwd_f32(nt, m->act[l], B, K, t, m->tin[l]);
        dlo_net_dropout(m, nt, state, B, l, K, m->tin[l]);
        t = m->tin[l];
      } else if (t != m->tin[l]) {
        memcpy(m->tin[l], t, B * K * sizeof(float));
        t = m->tin[l];
      }
      dlo_fc_fwd_f32(nt, B, K, H, t, W, m->Z[l]);
      if (m->norm[l] == DLO_NORM_NONE) dlo_bias_fwd_f32(nt, B, H, m->param + m->b_off[l], m->Z[l]);
      memcpy(m->out[l], m->Z[l], B * H * sizeof(float));
      /* last layer of its block: finish the block (fwp_st.cpp:3876-4010) */
      size_t r = l;
      while (m->type[r] != DLO_LAYER_RESIDUAL) --r;
      if (l == r + m->depth[r]) {
        float const *blk = m->out[l];
        if (m->norm[r] != DLO_NORM_NONE) {
          dlo_net_norm_fwd(m, nt, state, B, r, blk);
          blk = m->nrm[r];
        }
        size_t const f = m->feed[r];
        if (m->padding[r] == 0)
          dlo_identity_add_f32(nt, B, m->n_out[r], m->out[f], blk, m->out[r]);
        else
          dlo_zero_padded_identity_fwd_f32(nt, B, m->n_out[f], H, m->padding[r], m->out[f], blk, m->out[r]);
      }
    } else {
      /* plain layer, normalization before the activation: fwp_st.cpp:298-733 */
      float *cur;
      dlo_fc_fwd_f32(nt, B, K, H, in, W, m->Z[l]);
      if (m->norm[l] == DLO_NORM_NONE) dlo_bias_fwd_f32(nt, B, H, m->param + m->b_off[l], m->Z[l]);
      cur = m->Z[l];
      if (m->norm[l] != DLO_NORM_NONE) {
        dlo_net_norm_fwd(m, nt, state, B, l, cur);
        cur = m->nrm[l];
      }
      if (m->act[l] == DLO_ACT_SOFTMAX)
        dlo_softmax_fwd_f32(nt, B, H, cur, m->out[l]);
      else
        dlo_act_fwd_f32(nt, m->act[l], B, H, cur, m->out[l]);
      dlo_net_dropout(m, nt, state, B, l, H, m->out[l]);
    }
  }
}

/* normalization backward of entry l: dN [B,U] -> dx [B,U]; x = what was normalized */
static void dlo_net_norm_bwd(dlo_net *m, int nt, size_t B, size_t l, float const *x, float const *dN, float *dx) {
  size_t const U = m->n_unit[l];
  float const *gamma = m->param + m->n_weights + m->n_bias + m->u_off[l];
  float *dgamma = m->dparam + m->n_weights + m->n_bias + m->u_off[l];
  float *dbeta = dgamma + m->n_units_total;
  float *dmean = (float *)calloc(U, sizeof(float)), *dstd = (float *)calloc(U, sizeof(float));
  dlo_norm_bwd_f32(nt, m->norm[l] == DLO_NORM_BRN, B, U, m->mean[l], m->stdv[l], gamma, m->r[l], x, m->xhat[l], dN, dgamma,
                   dbeta, dmean, dstd, dx);
  free(dmean);
  free(dstd);
}

void dlo_net_backward(dlo_net *m, int nt, size_t B, float const *Y) {
  size_t const n = m->n_layers;
  for (size_t l = 0; l < n; ++l) memset(m->dOut[l], 0, m->max_batch * m->n_out[l] * sizeof(float));
  size_t const o = n - 1;
  for (size_t l = o; l >= 1; --l) {
    if (m->type[l] == DLO_LAYER_RESIDUAL) continue; /* handled with its last block layer */
    size_t const K = m->n_in[l], H = m->n_out[l];
    float const *W = m->param + m->w_off[l];
    if (!m->in_block[l]) {
      if (l == o) {
        dlo_softmax_ce_seed_f32(nt, B, H, m->out[o], Y, m->dZ[o], &m->loss_sum, &m->n_correct);
      } else {
        float const *pre = m->norm[l] != DLO_NORM_NONE ? m->nrm[l] : m->Z[l];
        float *dAF = (float *)calloc(B * H, sizeof(float));
        dlo_act_bwd_f32(nt, m->act[l], B, H, pre, m->out[l], m->dOut[l], dAF);
        if (m->norm[l] != DLO_NORM_NONE)
          dlo_net_norm_bwd(m, nt, B, l, m->Z[l], dAF, m->dZ[l]);
        else
          memcpy(m->dZ[l], dAF, B * H * sizeof(float));
        free(dAF);
      }
      dlo_fc_bwd_dw_f32(nt, B, K, H, m->out[m->feed[l]], m->dZ[l], m->dparam + m->w_off[l],
                        m->norm[l] == DLO_NORM_NONE ? m->dparam + m->b_off[l] : NULL);
      if (m->feed[l] != 0) dlo_fc_bwd_dx_f32(nt, B, H, K, m->dZ[l], W, m->dOut[m->feed[l]]);
    } else {
      /* l is the last layer of a block (the loop skips the others below) */
      size_t r = l;
      while (m->type[r] != DLO_LAYER_RESIDUAL) --r;
      size_t const D = m->depth[r], f = m->feed[r], HD = m->n_out[r + D];
      /* shortcut and block shares of the gradient (bwp_st.cpp:345-454, 1112-1175) */
      if (f != 0) dlo_residual_bwd_f32(nt, B, m->n_out[r], m->n_out[f], m->padding[r], m->dOut[r], m->dOut[f]);
      float *g = (float *)calloc(B * HD, sizeof(float));
      dlo_residual_bwd_f32(nt, B, m->n_out[r], HD, m->padding[r], m->dOut[r], g);
      if (m->norm[r] != DLO_NORM_NONE) {
        float *gx = (float *)calloc(B * HD, sizeof(float));
        dlo_net_norm_bwd(m, nt, B, r, m->out[r + D], g, gx);
        free(g);
        g = gx;
      }
      for (size_t i = r + D; i > r; --i) {
        size_t const Ki = m->n_in[i], Hi = m->n_out[i];
        memcpy(m->dZ[i], g, B * Hi * sizeof(float));
        free(g);
        dlo_fc_bwd_dw_f32(nt, B, Ki, Hi, m->tin[i], m->dZ[i], m->dparam + m->w_off[i],
                          m->norm[i] == DLO_NORM_NONE ? m->dparam + m->b_off[i] : NULL);
        float *dt = (float *)calloc(B * Ki, sizeof(float));
        dlo_fc_bwd_dx_f32(nt, B, Hi, Ki, m->dZ[i], m->param + m->w_off[i], dt);
        if (!m->block_first[i]) {
          float const *pre = m->norm[i] != DLO_NORM_NONE ? m->nrm[i] : m->out[m->feed[i]];
          float *da = (float *)calloc(B * Ki, sizeof(float));
          dlo_act_bwd_f32(nt, m->act[i], B, Ki, pre, m->tin[i], dt, da);
          free(dt);
          dt = da;
        }
        if (m->norm[i] != DLO_NORM_NONE) {
          float *dx = (float *)calloc(B * Ki, sizeof(float));
          dlo_net_norm_bwd(m, nt, B, i, m->out[m->feed[i]], dt, dx);
          free(dt);
          dt = dx;
        }
        g = dt;
      }
      /* g: gradient with respect to the block's input through its first layer */
      if (f != 0) dlo_identity_add_f32(nt, B, m->n_out[f], m->dOut[f], g, m->dOut[f]);
      free(g);
      l = r; /* continue below the RESIDUAL entry */
    }
    if (l == 1) break;
  }
}

float const *dlo_net_layer_output(dlo_net const *m, size_t l) { return m->out[l]; }
float const *dlo_net_layer_error(dlo_net const *m, size_t l) { return m->dZ[l]; }
double dlo_net_loss_sum(dlo_net const *m) { return m->loss_sum; }
double dlo_net_n_correct(dlo_net const *m) { return m->n_correct; }

void dlo_net_destroy(dlo_net *m) {
  if (!m) return;
  float **bufs[] = {m->out, m->Z, m->dOut, m->dZ, m->xhat, m->nrm, m->tin, m->mean, m->stdv, m->r, m->d};
  for (size_t i = 0; i < sizeof(bufs) / sizeof(bufs[0]); ++i) dlo_net_free(m, bufs[i]);
  for (size_t l = 0; l < m->n_layers; ++l) free(m->mask[l]);
  free(m->mask); free(m->X0);
  free(m->type); free(m->n_out); free(m->n_in); free(m->n_unit); free(m->feed); free(m->depth); free(m->padding);
  free(m->in_block); free(m->block_first); free(m->act); free(m->norm); free(m->drop); free(m->keep);
  free(m->w_off); free(m->b_off); free(m->u_off);
  free(m->param); free(m->dparam); free(m->mov_mean); free(m->mov_std);
  free(m);
}
