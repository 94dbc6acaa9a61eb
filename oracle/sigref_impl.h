/*
 * sigref_impl.h -- type-generic body of the CPU oracle (TEST INFRASTRUCTURE ONLY).
 *
 * Included twice by sigref.c, once with REAL=float / SUF=_f and once with
 * REAL=double / SUF=_d.  Every function restates, in plain C, what one function
 * of the reference CPU library computes; the reference location is cited above
 * each function (paths relative to the reference repository root).
 *
 * Buffers called "full" carry the scalar term at index 0 and level k starts at
 * offset lvl[k] = (d^k - 1)/(d - 1).
 */

#define CAT_(a, b) a##b
#define CAT(a, b) CAT_(a, b)
#define FN(name) CAT(name, SUF)

/* Virtual augmented path: siglib/cpsig/cp_path.h:46-62 (dims), :207-385 (points).
 * lead-lag: point i has lag = x[i/2], lead = x[i/2 + (i odd)]; time is the last
 * channel.  The reference keeps `time` as a running value advanced by
 * += time_step / -= time_step from the position the iterator was created at;
 * callers below reproduce that by carrying the time of each of their two
 * cursors themselves and passing it in. */
typedef struct {
    const REAL *x;
    uint64_t d_raw, len_raw;
    uint64_t d, len;
    int time_aug, lead_lag;
    REAL time_step;
} FN(vpath);

static void FN(vpath_init)(FN(vpath) *p, const REAL *x, uint64_t d_raw, uint64_t len_raw,
                           int time_aug, int lead_lag, REAL end_time)
{
    p->x = x;
    p->d_raw = d_raw;
    p->len_raw = len_raw;
    p->time_aug = time_aug;
    p->lead_lag = lead_lag;
    p->d = (lead_lag ? 2 * d_raw : d_raw) + (time_aug ? 1 : 0);
    p->len = lead_lag ? 2 * len_raw - 1 : len_raw;
    p->time_step = p->len > 1 ? end_time / (REAL)(p->len - 1) : (REAL)0;
}

/* value of channel c of augmented point i, given that point's running time */
static inline REAL FN(vpath_at)(const FN(vpath) *p, uint64_t i, uint64_t c, REAL time)
{
    if (!p->lead_lag) {
        if (c < p->d_raw) return p->x[i * p->d_raw + c];
        return time;
    }
    const uint64_t row = i / 2, odd = i & 1;
    if (c < p->d_raw) return p->x[row * p->d_raw + c];
    if (c < 2 * p->d_raw) return p->x[(row + odd) * p->d_raw + (c - p->d_raw)];
    return time;
}

/* siglib/cpsig/cp_signature.h:365-389 linear_signature_: exp of one segment,
 * level k = level (k-1) (x) z / k.  `full` layout. */
static void FN(segment_exp)(const REAL *z, REAL *out, uint64_t d, uint64_t degree, const uint64_t *lvl)
{
    out[0] = (REAL)1;
    if (degree == 0) return;
    for (uint64_t i = 0; i < d; ++i) out[1 + i] = z[i];
    for (uint64_t k = 2; k <= degree; ++k) {
        const REAL inv = (REAL)1 / (REAL)k;
        const REAL *left = out + lvl[k - 1];
        REAL *res = out + lvl[k];
        const uint64_t nleft = lvl[k] - lvl[k - 1];
        for (uint64_t i = 0; i < nleft; ++i) {
            const REAL s = left[i] * inv;
            for (uint64_t j = 0; j < d; ++j) res[i * d + j] = out[1 + j] * s;
        }
    }
}

/* siglib/cpsig/cp_signature.h:464-499 (loop body of signature_horner_) and
 * :549-603 signature_horner_step_: S <- S (x) exp(z), Horner form, in place,
 * descending target level so lower levels still hold the old values.
 * `h` needs d^(degree-1) entries. */
static void FN(horner_step)(REAL *S, const REAL *z, uint64_t d, uint64_t degree,
                            const uint64_t *lvl, REAL *h)
{
    for (uint64_t t = degree; t > 1; --t) {
        const REAL inv_t = (REAL)1 / (REAL)t;
        for (uint64_t i = 0; i < d; ++i) h[i] = z[i] * inv_t;
        for (uint64_t l = 1; l + 1 < t; ++l) {
            const uint64_t n = lvl[l + 1] - lvl[l];
            const REAL inv = (REAL)1 / (REAL)(t - l);
            const REAL *Sl = S + lvl[l];
            for (uint64_t i = n; i-- > 0;) {
                const REAL s = (h[i] + Sl[i]) * inv;
                for (uint64_t j = 0; j < d; ++j) h[i * d + j] = z[j] * s;
            }
        }
        const uint64_t n = lvl[t] - lvl[t - 1];
        const REAL *Sl = S + lvl[t - 1];
        REAL *St = S + lvl[t];
        for (uint64_t i = n; i-- > 0;) {
            const REAL s = h[i] + Sl[i];
            for (uint64_t j = 0; j < d; ++j) St[i * d + j] += z[j] * s;
        }
    }
    for (uint64_t j = 0; j < d; ++j) S[1 + j] += z[j];
}

/* siglib/cpsig/cp_sig_combine.h:35-66 sig_combine_inplace_: a <- a (x) b. */
static void FN(chen_inplace)(REAL *a, const REAL *b, uint64_t degree, const uint64_t *lvl)
{
    a[0] = (REAL)1;
    for (uint64_t t = degree; t > 0; --t) {
        REAL *res = a + lvl[t];
        for (uint64_t left = t - 1; left > 0; --left) {
            const uint64_t right = t - left;
            const uint64_t nl = lvl[left + 1] - lvl[left];
            const uint64_t nr = lvl[right + 1] - lvl[right];
            const REAL *al = a + lvl[left];
            const REAL *br = b + lvl[right];
            for (uint64_t i = 0; i < nl; ++i)
                for (uint64_t j = 0; j < nr; ++j) res[i * nr + j] += al[i] * br[j];
        }
        const uint64_t nt = lvl[t + 1] - lvl[t];
        for (uint64_t j = 0; j < nt; ++j) res[j] += b[lvl[t] + j];
    }
}

/* One path, full layout.  horner != 0: siglib/cpsig/cp_signature.h:426-500
 * signature_horner_; horner == 0: :391-424 signature_naive_.  Requires
 * p->len >= 2 and degree >= 2. */
static int FN(one_path_sig)(const FN(vpath) *p, REAL *out, uint64_t degree, int horner)
{
    const uint64_t d = p->d;
    uint64_t *lvl = (uint64_t *)malloc((degree + 2) * sizeof(uint64_t));
    REAL *z = (REAL *)malloc(d * sizeof(REAL));
    if (!lvl || !z) { free(lvl); free(z); return 1; }
    sigref_level_index(lvl, d, degree + 2);
    const uint64_t full = lvl[degree + 1];
    const uint64_t hsz = horner ? (lvl[degree] - lvl[degree - 1]) : full;
    REAL *work = (REAL *)malloc(hsz * sizeof(REAL));
    if (!work) { free(lvl); free(z); return 1; }

    REAL t_prev = (REAL)0, t_next = p->time_step; /* cursors start at indices 0 and 1 */
    for (uint64_t i = 0; i < d; ++i) z[i] = FN(vpath_at)(p, 1, i, t_next) - FN(vpath_at)(p, 0, i, t_prev);
    FN(segment_exp)(z, out, d, degree, lvl);

    for (uint64_t s = 1; s + 1 < p->len; ++s) {
        t_prev += p->time_step;
        t_next += p->time_step;
        for (uint64_t i = 0; i < d; ++i)
            z[i] = FN(vpath_at)(p, s + 1, i, t_next) - FN(vpath_at)(p, s, i, t_prev);
        if (horner) {
            FN(horner_step)(out, z, d, degree, lvl, work);
        } else {
            FN(segment_exp)(z, work, d, degree, lvl);
            FN(chen_inplace)(out, work, degree, lvl);
        }
    }
    free(work); free(z); free(lvl);
    return 0;
}

/* siglib/cpsig/cp_signature.h:1098-1203 sig_backprop_inplace_: reverse sweep for
 * one path.  S (full layout, signature of the whole path) and G (full layout,
 * upstream gradient, scalar slot ignored) are both overwritten.  out has
 * len_raw*d_raw entries, already zeroed. */
static int FN(one_path_backprop)(const FN(vpath) *p, REAL *out, REAL *G, REAL *S, uint64_t degree)
{
    const uint64_t d = p->d, dr = p->d_raw;
    uint64_t *lvl = (uint64_t *)malloc((degree + 2) * sizeof(uint64_t));
    if (!lvl) return 1;
    sigref_level_index(lvl, d, degree + 2);
    const uint64_t top = lvl[degree] - lvl[degree - 1]; /* d^(degree-1) */
    REAL *h = (REAL *)malloc((lvl[degree] ? lvl[degree] : 1) * sizeof(REAL));
    REAL *hd = (REAL *)malloc((top ? top : 1) * sizeof(REAL));
    REAL *z = (REAL *)malloc(3 * d * sizeof(REAL));
    REAL *hs = (REAL *)malloc((top ? top : 1) * sizeof(REAL));
    if (!h || !hd || !z || !hs) { free(lvl); free(h); free(hd); free(z); free(hs); return 1; }
    REAL *dz = z + d, *part = z + 2 * d;

    /* cursors: prev at index len-2, next at len-1; both iterators were created
     * at end() (time = len*time_step) and walked back with -= time_step */
    REAL t_next = (REAL)p->len * p->time_step;
    REAL t_prev = t_next;
    t_prev -= p->time_step; t_prev -= p->time_step;
    t_next -= p->time_step;
    uint64_t pos = p->len_raw - 1; /* raw row that receives +dz */
    int parity = 0;

    for (uint64_t s = p->len - 1; s > 0; --s) { /* segment (s-1) -> s */
        for (uint64_t i = 0; i < d; ++i)
            z[i] = FN(vpath_at)(p, s - 1, i, t_prev) - FN(vpath_at)(p, s, i, t_next);
        FN(horner_step)(S, z, d, degree, lvl, hs); /* un-multiply: S <- S (x) exp(-dx) */
        for (uint64_t i = 0; i < d; ++i) { z[i] = -z[i]; dz[i] = G[1 + i]; }

        for (uint64_t T = 2; T <= degree; ++T) {
            const REAL inv_T = (REAL)1 / (REAL)T;
            for (uint64_t i = 0; i < d; ++i) h[1 + i] = z[i] * inv_T;
            for (uint64_t l = 1; l + 1 < T; ++l) {
                const uint64_t n = lvl[l + 1] - lvl[l];
                const REAL sc = (REAL)1 / (REAL)(T - l);
                for (uint64_t i = 0; i < n; ++i) {
                    const REAL v = (h[lvl[l] + i] + S[lvl[l] + i]) * sc;
                    for (uint64_t j = 0; j < d; ++j) h[lvl[l + 1] + i * d + j] = z[j] * v;
                }
            }
            const REAL *incoming = G + lvl[T];
            for (uint64_t l = T - 1; l > 0; --l) {
                const uint64_t n = lvl[l + 1] - lvl[l];
                const REAL sc = (REAL)1 / (REAL)(T - l);
                for (uint64_t j = 0; j < d; ++j) part[j] = (REAL)0;
                for (uint64_t i = 0; i < n; ++i) {
                    const REAL v = (h[lvl[l] + i] + S[lvl[l] + i]) * sc;
                    const REAL *row = incoming + i * d;
                    REAL red = (REAL)0;
                    for (uint64_t j = 0; j < d; ++j) {
                        part[j] += row[j] * v;
                        red += row[j] * z[j];
                    }
                    red *= sc;
                    hd[i] = red;
                    G[lvl[l] + i] += red;
                }
                for (uint64_t j = 0; j < d; ++j) dz[j] += part[j];
                incoming = hd;
            }
            for (uint64_t i = 0; i < d; ++i) dz[i] += hd[i] * inv_T;
        }

        /* siglib/cpsig/cp_signature.h:1189-1201: raw channels only; with lead-lag
         * the odd->even segment moved the lag half, the even->odd one the lead half */
        const REAL *src = dz + ((p->lead_lag && parity) ? dr : 0);
        for (uint64_t c = 0; c < dr; ++c) {
            out[pos * dr + c] += src[c];
            out[(pos - 1) * dr + c] -= src[c];
        }
        if (s > 1) {
            t_prev -= p->time_step;
            t_next -= p->time_step;
            if (!p->lead_lag || parity) --pos;
            parity = !parity;
        }
    }
    free(lvl); free(h); free(hd); free(z); free(hs);
    return 0;
}

/* ---- batch drivers -------------------------------------------------------- */

typedef struct {
    const REAL *path; REAL *out;
    const REAL *derivs; const REAL *sig;
    uint64_t d_raw, len_raw, degree;
    int time_aug, lead_lag, horner, scalar_term;
    REAL end_time;
    uint64_t full_len, stride;
    int status;
} FN(job);

static void FN(sig_worker)(void *ctx, uint64_t b0, uint64_t b1)
{
    FN(job) *J = (FN(job) *)ctx;
    REAL *buf = NULL;
    if (!J->scalar_term) {
        buf = (REAL *)malloc(J->full_len * sizeof(REAL));
        if (!buf) { J->status = 1; return; }
    }
    for (uint64_t b = b0; b < b1; ++b) {
        FN(vpath) p;
        FN(vpath_init)(&p, J->path + b * J->d_raw * J->len_raw, J->d_raw, J->len_raw,
                       J->time_aug, J->lead_lag, J->end_time);
        REAL *o = J->out + b * J->stride;
        if (J->degree == 1) {
            /* siglib/cpsig/cp_signature.h:845-851,863-868: endpoint difference */
            /* the end() cursor holds len*time_step and is stepped back once */
            const REAL t_last = (REAL)p.len * p.time_step - p.time_step;
            if (J->scalar_term) *o++ = (REAL)1;
            for (uint64_t c = 0; c < p.d; ++c)
                o[c] = FN(vpath_at)(&p, p.len - 1, c, t_last) - FN(vpath_at)(&p, 0, c, (REAL)0);
            continue;
        }
        REAL *dst = J->scalar_term ? o : buf;
        const int rc = FN(one_path_sig)(&p, dst, J->degree, J->horner);
        if (rc) { J->status = rc; break; }
        if (!J->scalar_term) memcpy(o, buf + 1, (J->full_len - 1) * sizeof(REAL));
    }
    free(buf);
}

/* siglib/cpsig/cp_signature.h:719-889 signature_ (the correction path and the
 * small-dimension batch-SIMD path are alternative schedules of the same
 * arithmetic and are not restated). */
int FN(sigref_signature)(const REAL *path, REAL *out, uint64_t batch, uint64_t d_raw,
                         uint64_t len_raw, uint64_t degree, int time_aug, int lead_lag,
                         REAL end_time, int horner, int scalar_term, int n_jobs)
{
    if (d_raw == 0) return 2;
    if (n_jobs == 0) return 2;
    FN(vpath) p0;
    FN(vpath_init)(&p0, NULL, d_raw, len_raw, time_aug, lead_lag, end_time);
    const uint64_t full = sigref_sig_length(p0.d, degree);
    if (full == 0) return 10;
    const uint64_t stride = scalar_term ? full : full - 1;

    if (len_raw == 0 || p0.len <= 1) {
        for (uint64_t i = 0; i < stride * batch; ++i) out[i] = (REAL)0;
        if (scalar_term)
            for (uint64_t b = 0; b < batch; ++b) out[b * stride] = (REAL)1;
        return 0;
    }
    if (degree == 0) {
        if (scalar_term)
            for (uint64_t b = 0; b < batch; ++b) out[b] = (REAL)1;
        return 0;
    }
    if (p0.d == 1) {
        /* siglib/cpsig/cp_signature.h:770-784: d == 1 closed form Delta^k / k! */
        for (uint64_t b = 0; b < batch; ++b) {
            const REAL *x = path + b * len_raw;
            const REAL inc = x[len_raw - 1] - x[0];
            REAL v = (REAL)1;
            REAL *o = out + b * stride;
            if (scalar_term) *o++ = v;
            for (uint64_t k = 1; k <= degree; ++k) { v *= inc / (REAL)k; *o++ = v; }
        }
        return 0;
    }
    FN(job) J;
    memset(&J, 0, sizeof J);
    J.path = path; J.out = out; J.d_raw = d_raw; J.len_raw = len_raw; J.degree = degree;
    J.time_aug = time_aug; J.lead_lag = lead_lag; J.horner = horner; J.scalar_term = scalar_term;
    J.end_time = end_time; J.full_len = full; J.stride = stride; J.status = 0;
    sigref_run_batch(batch, n_jobs, &J, FN(sig_worker));
    return J.status;
}

static void FN(bp_worker)(void *ctx, uint64_t b0, uint64_t b1)
{
    FN(job) *J = (FN(job) *)ctx;
    REAL *S = (REAL *)malloc(2 * J->full_len * sizeof(REAL));
    if (!S) { J->status = 1; return; }
    REAL *G = S + J->full_len;
    for (uint64_t b = b0; b < b1; ++b) {
        /* siglib/cpsig/cp_signature.h:958-975: work on private full-size copies,
         * prepending sig[0] = 1 and deriv[0] = 0 when the scalar term is absent */
        if (J->scalar_term) {
            memcpy(S, J->sig + b * J->stride, J->full_len * sizeof(REAL));
            memcpy(G, J->derivs + b * J->stride, J->full_len * sizeof(REAL));
        } else {
            S[0] = (REAL)1; G[0] = (REAL)0;
            memcpy(S + 1, J->sig + b * J->stride, J->stride * sizeof(REAL));
            memcpy(G + 1, J->derivs + b * J->stride, J->stride * sizeof(REAL));
        }
        FN(vpath) p;
        FN(vpath_init)(&p, J->path + b * J->d_raw * J->len_raw, J->d_raw, J->len_raw,
                       J->time_aug, J->lead_lag, J->end_time);
        const int rc = FN(one_path_backprop)(&p, J->out + b * J->d_raw * J->len_raw, G, S, J->degree);
        if (rc) { J->status = rc; break; }
    }
    free(S);
}

/* siglib/cpsig/cp_signature.h:909-1019 sig_backprop_ (general path; the
 * small-signature batch-SIMD variant :42-227 is an alternative schedule of the
 * same arithmetic and is not restated). */
int FN(sigref_sig_backprop)(const REAL *path, REAL *out, const REAL *sig_derivs, const REAL *sig,
                            uint64_t batch, uint64_t d_raw, uint64_t len_raw, uint64_t degree,
                            int time_aug, int lead_lag, REAL end_time, int scalar_term, int n_jobs)
{
    for (uint64_t i = 0; i < batch * d_raw * len_raw; ++i) out[i] = (REAL)0;
    if (d_raw == 0) return 2;
    if (n_jobs == 0) return 2;
    FN(vpath) p0;
    FN(vpath_init)(&p0, NULL, d_raw, len_raw, time_aug, lead_lag, end_time);
    const uint64_t full = sigref_sig_length(p0.d, degree);
    if (full == 0) return 10;
    if (len_raw == 0 || p0.len <= 1 || degree == 0) return 0;

    FN(job) J;
    memset(&J, 0, sizeof J);
    J.path = path; J.out = out; J.derivs = sig_derivs; J.sig = sig;
    J.d_raw = d_raw; J.len_raw = len_raw; J.degree = degree;
    J.time_aug = time_aug; J.lead_lag = lead_lag; J.scalar_term = scalar_term;
    J.end_time = end_time; J.full_len = full; J.stride = scalar_term ? full : full - 1; J.status = 0;
    sigref_run_batch(batch, n_jobs, &J, FN(bp_worker));
    return J.status;
}


/* ---- operators either side of the signature path -------------------------- */

/* siglib/cpsig/cp_sig_combine.h:126-176 uncombine_sig_deriv (full layout):
 * given dF/d(a (x) b) in `da` (overwritten with dF/da) computes dF/db into `db`. */
static void FN(chen_pullback)(const REAL *a, const REAL *b, REAL *da, REAL *db, uint64_t degree, const uint64_t *lvl)
{
    const uint64_t full = lvl[degree + 1];
    memcpy(db, da, full * sizeof(REAL));
    for (uint64_t t = degree; t > 0; --t) {
        for (uint64_t left = t - 1; left > 0; --left) {
            const uint64_t right = t - left;
            const uint64_t nl = lvl[left + 1] - lvl[left], nr = lvl[right + 1] - lvl[right];
            const REAL *res = da + lvl[t];
            REAL *dbr = db + lvl[right];
            for (uint64_t i = 0; i < nl; ++i)
                for (uint64_t j = 0; j < nr; ++j) dbr[j] += res[i * nr + j] * a[lvl[left] + i];
        }
    }
    for (uint64_t left = 1; left < degree; ++left) {
        for (uint64_t t = left + 1; t <= degree; ++t) {
            const uint64_t right = t - left;
            const uint64_t nl = lvl[left + 1] - lvl[left], nr = lvl[right + 1] - lvl[right];
            const REAL *res = da + lvl[t];
            for (uint64_t i = 0; i < nl; ++i) {
                REAL acc = (REAL)0;
                for (uint64_t j = 0; j < nr; ++j) acc += res[i * nr + j] * b[lvl[right] + j];
                da[lvl[left] + i] += acc;
            }
        }
    }
}

/* siglib/cpsig/cp_sig_combine.h:266-316 sig_combine_ / batch_sig_combine_ */
int FN(sigref_sig_combine)(const REAL *sig1, const REAL *sig2, REAL *out, uint64_t batch, uint64_t d,
                           uint64_t degree, int scalar_term)
{
    if (d == 0) return 2;
    const uint64_t full = sigref_sig_length(d, degree);
    if (full == 0) return 10;
    const uint64_t stride = scalar_term ? full : full - 1;
    uint64_t *lvl = (uint64_t *)malloc((degree + 2) * sizeof(uint64_t));
    REAL *a = (REAL *)malloc(2 * full * sizeof(REAL));
    if (!lvl || !a) { free(lvl); free(a); return 1; }
    REAL *b = a + full;
    sigref_level_index(lvl, d, degree + 2);
    const uint64_t off = scalar_term ? 0 : 1;
    for (uint64_t i = 0; i < batch; ++i) {
        a[0] = b[0] = (REAL)1;
        memcpy(a + off, sig1 + i * stride, stride * sizeof(REAL));
        memcpy(b + off, sig2 + i * stride, stride * sizeof(REAL));
        FN(chen_inplace)(a, b, degree, lvl);
        memcpy(out + i * stride, a + off, stride * sizeof(REAL));
    }
    free(lvl); free(a);
    return 0;
}

/* siglib/cpsig/cp_sig_combine.h:318-400 sig_combine_backprop_ / batch_sig_combine_backprop_:
 * scalar slots of both gradients are 0. */
int FN(sigref_sig_combine_backprop)(const REAL *dout, REAL *d1, REAL *d2, const REAL *sig1, const REAL *sig2,
                                    uint64_t batch, uint64_t d, uint64_t degree, int scalar_term)
{
    if (d == 0) return 2;
    const uint64_t full = sigref_sig_length(d, degree);
    if (full == 0) return 10;
    const uint64_t stride = scalar_term ? full : full - 1;
    uint64_t *lvl = (uint64_t *)malloc((degree + 2) * sizeof(uint64_t));
    REAL *a = (REAL *)malloc(4 * full * sizeof(REAL));
    if (!lvl || !a) { free(lvl); free(a); return 1; }
    REAL *b = a + full, *da = a + 2 * full, *db = a + 3 * full;
    sigref_level_index(lvl, d, degree + 2);
    const uint64_t off = scalar_term ? 0 : 1;
    for (uint64_t i = 0; i < batch; ++i) {
        a[0] = b[0] = (REAL)1; da[0] = (REAL)0;
        memcpy(a + off, sig1 + i * stride, stride * sizeof(REAL));
        memcpy(b + off, sig2 + i * stride, stride * sizeof(REAL));
        memcpy(da + off, dout + i * stride, stride * sizeof(REAL));
        FN(chen_pullback)(a, b, da, db, degree, lvl);
        da[0] = db[0] = (REAL)0;
        memcpy(d1 + i * stride, da + off, stride * sizeof(REAL));
        memcpy(d2 + i * stride, db + off, stride * sizeof(REAL));
    }
    free(lvl); free(a);
    return 0;
}

/* siglib/cpsig/cp_path_transforms.h:36-142 transform_path_ (materialised augmentation) */
int FN(sigref_transform_path)(const REAL *in, REAL *out, uint64_t batch, uint64_t d, uint64_t len,
                              int time_aug, int lead_lag, REAL end_time)
{
    if (d == 0) return 2;
    FN(vpath) p;
    for (uint64_t b = 0; b < batch; ++b) {
        FN(vpath_init)(&p, in + b * d * len, d, len, time_aug, lead_lag, end_time);
        REAL *o = out + b * p.d * p.len;
        const REAL scale = p.len > 1 ? end_time / (REAL)(p.len - 1) : (REAL)0;
        for (uint64_t i = 0; i < p.len; ++i)
            for (uint64_t c = 0; c < p.d; ++c) o[i * p.d + c] = FN(vpath_at)(&p, i, c, (REAL)i * scale);
    }
    return 0;
}

/* siglib/cpsig/cp_path_transforms.h:182-243 transform_path_backprop_ */
int FN(sigref_transform_path_backprop)(const REAL *derivs, REAL *out, uint64_t batch, uint64_t d, uint64_t len,
                                       int time_aug, int lead_lag)
{
    if (d == 0) return 2;
    const uint64_t td = (lead_lag ? 2 * d : d) + (time_aug ? 1 : 0);
    const uint64_t tl = lead_lag ? 2 * len - 1 : len;
    for (uint64_t b = 0; b < batch; ++b) {
        const REAL *g = derivs + b * td * tl;
        REAL *o = out + b * d * len;
        for (uint64_t k = 0; k < len; ++k)
            for (uint64_t j = 0; j < d; ++j) {
                if (!lead_lag) { o[k * d + j] = g[k * td + j]; continue; }
                REAL v = g[(2 * k) * td + j];
                if (k + 1 < len) v += g[(2 * k + 1) * td + j];
                v += g[(2 * k) * td + d + j];
                if (k >= 1) v += g[(2 * k - 1) * td + d + j];
                o[k * d + j] = v;
            }
    }
    return 0;
}

/* siglib/cpsig/cp_sig_combine.h:232-263 linear_sig_deriv_to_increment_deriv: e = exp(z) (full layout),
 * de = dF/de (destroyed), dz = dF/dz.  Level k = level (k-1) (x) z / k, pulled back from the top level down. */
static void FN(exp_pullback)(const REAL *e, REAL *de, REAL *dz, uint64_t d, uint64_t degree, const uint64_t *lvl)
{
    for (uint64_t j = 0; j < d; ++j) dz[j] = (REAL)0;
    for (uint64_t k = degree; k > 1; --k) {
        const REAL inv = (REAL)1 / (REAL)k;
        const uint64_t nleft = lvl[k] - lvl[k - 1];
        for (uint64_t i = 0; i < nleft; ++i) {
            const REAL *g = de + lvl[k] + i * d;
            const REAL s = e[lvl[k - 1] + i] * inv;
            REAL dot = (REAL)0;
            for (uint64_t j = 0; j < d; ++j) {
                dot += g[j] * e[1 + j];
                dz[j] += g[j] * s;
            }
            de[lvl[k - 1] + i] += dot * inv;
        }
    }
    if (degree >= 1)
        for (uint64_t j = 0; j < d; ++j) dz[j] += de[1 + j];
}

/* siglib/cpsig/cp_sig_join.h:62-104 linear_sig_ / batch_linear_sig_ */
int FN(sigref_linear_sig)(const REAL *disp, REAL *out, uint64_t batch, uint64_t d, uint64_t degree, int scalar_term)
{
    if (d == 0) return 2;
    const uint64_t full = sigref_sig_length(d, degree);
    if (full == 0) return 10;
    const uint64_t stride = scalar_term ? full : full - 1;
    uint64_t *lvl = (uint64_t *)malloc((degree + 2) * sizeof(uint64_t));
    REAL *e = (REAL *)malloc(full * sizeof(REAL));
    if (!lvl || !e) { free(lvl); free(e); return 1; }
    sigref_level_index(lvl, d, degree + 2);
    const uint64_t off = scalar_term ? 0 : 1;
    for (uint64_t i = 0; i < batch; ++i) {
        FN(segment_exp)(disp + i * d, e, d, degree, lvl);
        memcpy(out + i * stride, e + off, stride * sizeof(REAL));
    }
    free(lvl); free(e);
    return 0;
}

/* siglib/cpsig/cp_sig_join.h:107-160 sig_join_: out = sig (x) exp(z), or exp(z) (x) sig when prepending */
int FN(sigref_sig_join)(const REAL *sig, const REAL *disp, REAL *out, uint64_t batch, uint64_t d, uint64_t degree,
                        int prepend, int scalar_term)
{
    if (d == 0) return 2;
    const uint64_t full = sigref_sig_length(d, degree);
    if (full == 0) return 10;
    const uint64_t stride = scalar_term ? full : full - 1;
    uint64_t *lvl = (uint64_t *)malloc((degree + 2) * sizeof(uint64_t));
    REAL *a = (REAL *)malloc(2 * full * sizeof(REAL));
    if (!lvl || !a) { free(lvl); free(a); return 1; }
    REAL *e = a + full;
    sigref_level_index(lvl, d, degree + 2);
    const uint64_t off = scalar_term ? 0 : 1;
    for (uint64_t i = 0; i < batch; ++i) {
        a[0] = (REAL)1;
        memcpy(a + off, sig + i * stride, stride * sizeof(REAL));
        FN(segment_exp)(disp + i * d, e, d, degree, lvl);
        if (prepend) {
            FN(chen_inplace)(e, a, degree, lvl);
            memcpy(out + i * stride, e + off, stride * sizeof(REAL));
        } else {
            FN(chen_inplace)(a, e, degree, lvl);
            memcpy(out + i * stride, a + off, stride * sizeof(REAL));
        }
    }
    free(lvl); free(a);
    return 0;
}

/* siglib/cpsig/cp_sig_join.h:163-238 sig_join_backprop_ */
int FN(sigref_sig_join_backprop)(const REAL *dout, REAL *dsig, REAL *ddisp, const REAL *sig, const REAL *disp,
                                 uint64_t batch, uint64_t d, uint64_t degree, int prepend, int scalar_term)
{
    if (d == 0) return 2;
    const uint64_t full = sigref_sig_length(d, degree);
    if (full == 0) return 10;
    const uint64_t stride = scalar_term ? full : full - 1;
    uint64_t *lvl = (uint64_t *)malloc((degree + 2) * sizeof(uint64_t));
    REAL *a = (REAL *)malloc(4 * full * sizeof(REAL));
    if (!lvl || !a) { free(lvl); free(a); return 1; }
    REAL *e = a + full, *da = e + full, *de = da + full;
    sigref_level_index(lvl, d, degree + 2);
    const uint64_t off = scalar_term ? 0 : 1;
    for (uint64_t i = 0; i < batch; ++i) {
        a[0] = (REAL)1;
        memcpy(a + off, sig + i * stride, stride * sizeof(REAL));
        FN(segment_exp)(disp + i * d, e, d, degree, lvl);
        if (prepend) {      /* out = e (x) a */
            de[0] = (REAL)0;
            memcpy(de + off, dout + i * stride, stride * sizeof(REAL));
            FN(chen_pullback)(e, a, de, da, degree, lvl);
        } else {            /* out = a (x) e */
            da[0] = (REAL)0;
            memcpy(da + off, dout + i * stride, stride * sizeof(REAL));
            FN(chen_pullback)(a, e, da, de, degree, lvl);
        }
        da[0] = de[0] = (REAL)0;
        memcpy(dsig + i * stride, da + off, stride * sizeof(REAL));
        FN(exp_pullback)(e, de, ddisp + i * d, d, degree, lvl);
    }
    free(lvl); free(a);
    return 0;
}

/* siglib/cpsig/cp_sig_coef_impl.cpp:35-84 single_sig_coef_: coefficients of the prefixes of ONE word, swept over the
 * path with the per-word Horner step (:296-305):  c_i += z_{i-1} * (((1/i!) z_0 + c_1/(i-1)!) z_1 + ...). */
static void FN(word_sweep)(const FN(vpath) *p, const uint64_t *word, uint64_t k, REAL *c /* k + 1 */, REAL *z /* k */,
                           const REAL *inv_fact)
{
    c[0] = (REAL)1;
    for (uint64_t i = 1; i <= k; ++i) c[i] = (REAL)0;
    const REAL step = p->time_step;
    REAL t_prev = (REAL)0;
    for (uint64_t s = 0; s + 1 < p->len; ++s) {
        const REAL t_next = t_prev + step;
        for (uint64_t i = 0; i < k; ++i) z[i] = FN(vpath_at)(p, s + 1, word[i], t_next) - FN(vpath_at)(p, s, word[i], t_prev);
        for (uint64_t i = k; i > 0; --i) {
            REAL acc = inv_fact[i];
            for (uint64_t j = 0; j + 1 < i; ++j) acc = acc * z[j] + c[j + 1] * inv_fact[i - j - 1];
            c[i] += acc * z[i - 1];
        }
        t_prev = t_next;
    }
}

/* siglib/cpsig/cp_sig_coef_impl.cpp:138-348 sig_coef_: out row = per word either its coefficient or, with prefixes,
 * the coefficients of all its non-empty prefixes (the empty word yields one entry, 1). */
int FN(sigref_sig_coef)(const REAL *path, REAL *out, const uint64_t *multi_idx, uint64_t num_words, const uint64_t *degrees,
                        uint64_t batch, uint64_t d_raw, uint64_t len_raw, int time_aug, int lead_lag, REAL end_time,
                        int prefixes)
{
    if (d_raw == 0) return 2;
    FN(vpath) p0;
    FN(vpath_init)(&p0, NULL, d_raw, len_raw ? len_raw : 1, time_aug, lead_lag, end_time);
    uint64_t kmax = 0, total = 0, row = 0;
    for (uint64_t w = 0; w < num_words; ++w) {
        if (degrees[w] > kmax) kmax = degrees[w];
        total += degrees[w];
        row += prefixes ? (degrees[w] ? degrees[w] : 1) : 1;
    }
    if (len_raw == 0) {     /* no points: every non-empty word has coefficient 0 */
        for (uint64_t b = 0; b < batch; ++b) {
            REAL *o = out + b * row;
            for (uint64_t w = 0; w < num_words; ++w) {
                const uint64_t cnt = prefixes && degrees[w] ? degrees[w] : 1;
                for (uint64_t i = 0; i < cnt; ++i) *o++ = degrees[w] ? (REAL)0 : (REAL)1;
            }
        }
        return 0;
    }
    for (uint64_t i = 0; i < total; ++i) if (multi_idx[i] >= p0.d) return 2;
    REAL *c = (REAL *)malloc((3 * kmax + 3) * sizeof(REAL));
    if (!c) return 1;
    REAL *z = c + kmax + 1, *inv_fact = z + kmax + 1;
    inv_fact[0] = (REAL)1;
    for (uint64_t i = 1; i <= kmax; ++i) inv_fact[i] = inv_fact[i - 1] / (REAL)i;
    for (uint64_t b = 0; b < batch; ++b) {
        FN(vpath) p;
        FN(vpath_init)(&p, path + b * d_raw * len_raw, d_raw, len_raw, time_aug, lead_lag, end_time);
        REAL *o = out + b * row;
        const uint64_t *word = multi_idx;
        for (uint64_t w = 0; w < num_words; ++w) {
            const uint64_t k = degrees[w];
            if (k == 0) { *o++ = (REAL)1; continue; }
            FN(word_sweep)(&p, word, k, c, z, inv_fact);
            if (prefixes) { for (uint64_t i = 1; i <= k; ++i) *o++ = c[i]; }
            else *o++ = c[k];
            word += k;
        }
    }
    free(c);
    return 0;
}

/* siglib/cpsig/cp_sig_coef_impl.cpp:360-485,546-664 sig_coef_backprop_: reverse sweep per word.  Per step the prefix
 * coefficients are taken back one step with the increment negated (uncombine_coefs_), then the adjoint goes through the
 * Horner step (backprop_horner_): `g` (dF/d prefix coefficients) is updated in place and the increment gradient of
 * every letter is scattered to the two path points of the step.  coefs / derivs have the prefixes layout; words of
 * degree 0 own one (ignored) entry. */
int FN(sigref_sig_coef_backprop)(const REAL *path, REAL *out, const REAL *coefs, const REAL *derivs,
                                 const uint64_t *multi_idx, uint64_t num_words, const uint64_t *degrees, uint64_t batch,
                                 uint64_t d_raw, uint64_t len_raw, int time_aug, int lead_lag, REAL end_time)
{
    if (d_raw == 0) return 2;
    FN(vpath) p0;
    FN(vpath_init)(&p0, NULL, d_raw, len_raw, time_aug, lead_lag, end_time);
    uint64_t kmax = 0, total = 0, row = 0;
    for (uint64_t w = 0; w < num_words; ++w) {
        if (degrees[w] > kmax) kmax = degrees[w];
        total += degrees[w];
        row += degrees[w] ? degrees[w] : 1;
    }
    if (len_raw == 0) return 0;
    for (uint64_t i = 0; i < total; ++i) if (multi_idx[i] >= p0.d) return 2;
    REAL *c = (REAL *)malloc((6 * kmax + 6) * sizeof(REAL));
    REAL *dx = (REAL *)malloc((p0.len ? p0.len : 1) * p0.d * sizeof(REAL));      /* gradient w.r.t. the augmented path */
    if (!c || !dx) { free(c); free(dx); return 1; }
    REAL *z = c + kmax + 1, *inv_fact = z + kmax + 1, *g = inv_fact + kmax + 1, *st = g + kmax + 1, *dz = st + kmax + 1;
    inv_fact[0] = (REAL)1;
    for (uint64_t i = 1; i <= kmax; ++i) inv_fact[i] = inv_fact[i - 1] / (REAL)i;
    for (uint64_t b = 0; b < batch; ++b) {
        FN(vpath) p;
        FN(vpath_init)(&p, path + b * d_raw * len_raw, d_raw, len_raw, time_aug, lead_lag, end_time);
        for (uint64_t i = 0; i < p.len * p.d; ++i) dx[i] = (REAL)0;
        const REAL step = p.time_step;
        const uint64_t *word = multi_idx;
        const REAL *crow = coefs + b * row, *grow = derivs + b * row;
        for (uint64_t w = 0; w < num_words; ++w) {
            const uint64_t k = degrees[w];
            if (k == 0) { ++crow; ++grow; continue; }
            c[0] = (REAL)1;
            for (uint64_t i = 1; i <= k; ++i) { c[i] = crow[i - 1]; g[i] = grow[i - 1]; }
            for (uint64_t s = p.len - 1; s >= 1; --s) {      /* step s-1 -> s */
                const REAL t_next = (REAL)s * step, t_prev = (REAL)(s - 1) * step;
                for (uint64_t i = 0; i < k; ++i) z[i] = FN(vpath_at)(&p, s, word[i], t_next) - FN(vpath_at)(&p, s - 1, word[i], t_prev);
                /* coefficients before the step: multiply by exp(-z) */
                for (uint64_t i = k; i > 0; --i) {
                    REAL acc = (i & 1) ? -inv_fact[i] : inv_fact[i];
                    for (uint64_t j = 0; j + 1 < i; ++j) {
                        const uint64_t m = i - j - 1;
                        acc = acc * z[j] + c[j + 1] * ((m & 1) ? -inv_fact[m] : inv_fact[m]);
                    }
                    c[i] += acc * z[i - 1];
                }
                for (uint64_t i = 0; i < k; ++i) dz[i] = (REAL)0;
                for (uint64_t i = 1; i <= k; ++i) {
                    st[0] = inv_fact[i];
                    for (uint64_t j = 0; j + 1 < i; ++j) st[j + 1] = st[j] * z[j] + c[j + 1] * inv_fact[i - j - 1];
                    const REAL gi = g[i];
                    dz[i - 1] += gi * st[i - 1];
                    REAL sd = gi * z[i - 1];
                    for (uint64_t j = i - 1; j-- > 0;) {
                        dz[j] += sd * st[j];
                        g[j + 1] += sd * inv_fact[i - j - 1];
                        sd *= z[j];
                    }
                }
                for (uint64_t i = 0; i < k; ++i) {
                    dx[s * p.d + word[i]] += dz[i];
                    dx[(s - 1) * p.d + word[i]] -= dz[i];
                }
            }
            word += k; crow += k; grow += k;
        }
        /* augmented-path gradient -> raw path gradient (adjoint of the augmentation) */
        REAL *o = out + b * d_raw * len_raw;
        for (uint64_t i = 0; i < len_raw; ++i)
            for (uint64_t j = 0; j < d_raw; ++j) {
                if (!lead_lag) { o[i * d_raw + j] = p.len ? dx[i * p.d + j] : (REAL)0; continue; }
                REAL v = dx[(2 * i) * p.d + j] + dx[(2 * i) * p.d + d_raw + j];
                if (i + 1 < len_raw) v += dx[(2 * i + 1) * p.d + j];
                if (i >= 1) v += dx[(2 * i - 1) * p.d + d_raw + j];
                o[i * d_raw + j] = v;
            }
    }
    free(c); free(dx);
    return 0;
}

/* Product without the identity terms: c_t = sum_{l=1..t-1} a_l (x) b_{t-l} for 2 <= t <= maxlevel (full layout). */
static void FN(tail_product)(const REAL *a, const REAL *b, REAL *c, uint64_t maxlevel, const uint64_t *lvl)
{
    for (uint64_t t = 2; t <= maxlevel; ++t) {
        REAL *res = c + lvl[t];
        for (uint64_t i = 0; i < lvl[t + 1] - lvl[t]; ++i) res[i] = (REAL)0;
        for (uint64_t left = 1; left < t; ++left) {
            const uint64_t right = t - left, nl = lvl[left + 1] - lvl[left], nr = lvl[right + 1] - lvl[right];
            for (uint64_t i = 0; i < nl; ++i)
                for (uint64_t j = 0; j < nr; ++j) res[i * nr + j] += a[lvl[left] + i] * b[lvl[right] + j];
        }
    }
}

/* siglib/cpsig/cp_tensor_log.h:40-113 tensor_log_: with x = sig - 1,
 *   log(1 + x) = P_1,  P_k = x / k - x (x) P_{k+1},  P_{N+1} = 0   (P_k needs levels <= N - k + 1).
 * `P` (optional) receives P_2 .. P_N, each in full layout, zero above its top level. */
static int FN(tensor_log)(const REAL *x /* full layout, x[0] ignored */, REAL *out, REAL *P, uint64_t d, uint64_t degree,
                          const uint64_t *lvl)
{
    const uint64_t full = lvl[degree + 1];
    REAL *cur = (REAL *)calloc(2 * full, sizeof(REAL));
    if (!cur) return 1;
    REAL *prod = cur + full;
    (void)d;
    for (uint64_t k = degree; k >= 1; --k) {
        const uint64_t top = degree - k + 1;
        FN(tail_product)(x, cur, prod, top, lvl);       /* x (x) P_{k+1}; empty for k = N */
        const REAL inv = (REAL)1 / (REAL)k;
        for (uint64_t i = 0; i < full; ++i) cur[i] = (REAL)0;
        for (uint64_t t = 1; t <= top; ++t)
            for (uint64_t i = lvl[t]; i < lvl[t + 1]; ++i) cur[i] = inv * x[i] - (t >= 2 ? prod[i] : (REAL)0);
        if (P && k >= 2) memcpy(P + (k - 2) * full, cur, full * sizeof(REAL));
    }
    memcpy(out, cur, full * sizeof(REAL));
    out[0] = (REAL)0;
    free(cur);
    return 0;
}

/* siglib/cpsig/cp_tensor_log.h:115-125 log_sig_expanded / sig_to_log_sig with method 0 */
int FN(sigref_sig_to_log_sig)(const REAL *sig, REAL *out, uint64_t batch, uint64_t d, uint64_t degree, int scalar_term)
{
    if (d == 0) return 2;
    const uint64_t full = sigref_sig_length(d, degree);
    if (full == 0) return 10;
    const uint64_t stride = scalar_term ? full : full - 1, off = scalar_term ? 0 : 1;
    uint64_t *lvl = (uint64_t *)malloc((degree + 2) * sizeof(uint64_t));
    REAL *x = (REAL *)malloc(2 * full * sizeof(REAL));
    if (!lvl || !x) { free(lvl); free(x); return 1; }
    REAL *o = x + full;
    sigref_level_index(lvl, d, degree + 2);
    int rc = 0;
    for (uint64_t i = 0; i < batch && !rc; ++i) {
        x[0] = (REAL)1;
        memcpy(x + off, sig + i * stride, stride * sizeof(REAL));
        rc = FN(tensor_log)(x, o, NULL, d, degree, lvl);
        memcpy(out + i * stride, o + off, stride * sizeof(REAL));
    }
    free(lvl); free(x);
    return rc;
}

/* siglib/cpsig/cp_tensor_log.h:164-221 tensor_log_backprop_: the adjoint of the recursion above, walked from P_1
 * (where the upstream gradient enters) to P_N:  dx += g_k / k - [adjoint of x (x) P_{k+1} w.r.t. x],
 * g_{k+1} = -[adjoint w.r.t. P_{k+1}]. */
int FN(sigref_sig_to_log_sig_backprop)(const REAL *sig, REAL *out, const REAL *derivs, uint64_t batch, uint64_t d,
                                       uint64_t degree, int scalar_term)
{
    if (d == 0) return 2;
    const uint64_t full = sigref_sig_length(d, degree);
    if (full == 0) return 10;
    const uint64_t stride = scalar_term ? full : full - 1, off = scalar_term ? 0 : 1;
    uint64_t *lvl = (uint64_t *)malloc((degree + 2) * sizeof(uint64_t));
    REAL *x = (REAL *)malloc((5 + (degree > 1 ? degree - 1 : 1)) * full * sizeof(REAL));
    if (!lvl || !x) { free(lvl); free(x); return 1; }
    REAL *o = x + full, *g = o + full, *gn = g + full, *dx = gn + full, *P = dx + full;
    sigref_level_index(lvl, d, degree + 2);
    int rc = 0;
    for (uint64_t b = 0; b < batch && !rc; ++b) {
        x[0] = (REAL)1;
        memcpy(x + off, sig + b * stride, stride * sizeof(REAL));
        g[0] = (REAL)0;
        memcpy(g + off, derivs + b * stride, stride * sizeof(REAL));
        g[0] = (REAL)0;
        for (uint64_t i = 0; i < full; ++i) dx[i] = (REAL)0;
        if (degree >= 1) {
            rc = FN(tensor_log)(x, o, P, d, degree, lvl);
            for (uint64_t k = 1; k <= degree && !rc; ++k) {
                const uint64_t top = degree - k + 1;
                const REAL inv = (REAL)1 / (REAL)k;
                for (uint64_t i = lvl[1]; i < lvl[top + 1]; ++i) dx[i] += inv * g[i];
                if (k == degree) break;
                const REAL *Pn = P + (k - 1) * full;        /* P_{k+1} */
                for (uint64_t i = 0; i < full; ++i) gn[i] = (REAL)0;
                for (uint64_t t = 2; t <= top; ++t)
                    for (uint64_t left = 1; left < t; ++left) {
                        const uint64_t right = t - left, nl = lvl[left + 1] - lvl[left], nr = lvl[right + 1] - lvl[right];
                        const REAL *gt = g + lvl[t];
                        for (uint64_t i = 0; i < nl; ++i)
                            for (uint64_t j = 0; j < nr; ++j) {
                                dx[lvl[left] + i] -= gt[i * nr + j] * Pn[lvl[right] + j];
                                gn[lvl[right] + j] -= gt[i * nr + j] * x[lvl[left] + i];
                            }
                    }
                memcpy(g, gn, full * sizeof(REAL));
            }
        }
        dx[0] = (REAL)0;
        memcpy(out + b * stride, dx + off, stride * sizeof(REAL));
    }
    free(lvl); free(x);
    return rc;
}

#undef FN
#undef CAT
#undef CAT_
