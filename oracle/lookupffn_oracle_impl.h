/*
 * TEST INFRASTRUCTURE ONLY -- body of the CPU restatement, compiled twice by
 * lookupffn_oracle.c: once with REAL = float (the arithmetic the reference
 * computes in, in the reference's own operation order) and once with
 * REAL = double (the "truth" tolerances are measured against).
 *
 * Reference paths are relative to the reference checkout;
 * PL/ = src/roberta/models/prenorm_lookup/.
 */

/* Unnormalised Sylvester-ordered Hadamard transform of every row,
 * out[b,:] = in[b,:] . H_D with H[i,j] = (-1)^popcount(i&j).
 * Butterfly order follows PL/bh4/fast_hadamard_transform/extension/cuda_kernel.cu:235-251:
 * strides D/2, D/4, ..., 1; at each stride the element whose stride bit is 0
 * becomes (a + b) and the one whose bit is 1 becomes (a - b) with a the low
 * partner (":241" computes sign*val1 + val2 with val2 the partner).  The divide
 * by sqrt(D) is commented out there (":255-256"), so none is applied. */
void FN(orc_fht)(const REAL *in, REAL *out, int64_t B, int64_t D)
{
#pragma omp parallel for schedule(static)
    for (int64_t b = 0; b < B; b++) {
        REAL *o = out + b * D;
        if (o != in + b * D) memcpy(o, in + b * D, (size_t)D * sizeof(REAL));
        for (int64_t stride = D / 2; stride >= 1; stride /= 2) {
            for (int64_t base = 0; base < D; base += 2 * stride) {
                for (int64_t j = base; j < base + stride; j++) {
                    REAL lo = o[j], hi = o[j + stride];
                    o[j] = lo + hi;
                    o[j + stride] = lo - hi;
                }
            }
        }
    }
}

/* BH4 mixing, GPU convention: PL/bh4/kernel.py:23-36.
 *   for r < R:  y = x;  for j < J:  y = FHT( blockdiag(w[r,j]) y )
 *   out[:, r*D:(r+1)*D] = y
 * blockdiag is the einsum "bni,noi->bno" (":32"): y[b,n,o] = sum_i y[b,n,i] * w[n,o,i].
 * w is [R, J, D/bs, bs, bs] row-major; bs == 1 degenerates to a diagonal scale.
 * x is [B, D] (already padded). */
void FN(orc_bh4)(const REAL *x, const REAL *w, REAL *out,
                 int64_t B, int64_t D, int64_t R, int64_t J, int64_t bs)
{
    const int64_t NB = D / bs;
#pragma omp parallel
    {
        REAL *y = (REAL *)malloc((size_t)D * sizeof(REAL));
        REAL *u = (REAL *)malloc((size_t)D * sizeof(REAL));
#pragma omp for schedule(static)
        for (int64_t b = 0; b < B; b++) {
            for (int64_t r = 0; r < R; r++) {
                memcpy(y, x + b * D, (size_t)D * sizeof(REAL));
                for (int64_t j = 0; j < J; j++) {
                    const REAL *wj = w + ((r * J + j) * NB) * bs * bs;
                    for (int64_t n = 0; n < NB; n++) {
                        for (int64_t o = 0; o < bs; o++) {
                            REAL acc = 0;
                            for (int64_t i = 0; i < bs; i++)
                                acc += y[n * bs + i] * wj[(n * bs + o) * bs + i];
                            u[n * bs + o] = acc;
                        }
                    }
                    /* in-place butterfly on u, result back into y */
                    for (int64_t stride = D / 2; stride >= 1; stride /= 2)
                        for (int64_t base = 0; base < D; base += 2 * stride)
                            for (int64_t q = base; q < base + stride; q++) {
                                REAL lo = u[q], hi = u[q + stride];
                                u[q] = lo + hi;
                                u[q + stride] = lo - hi;
                            }
                    memcpy(y, u, (size_t)D * sizeof(REAL));
                }
                memcpy(out + (b * R + r) * D, y, (size_t)D * sizeof(REAL));
            }
        }
        free(y);
        free(u);
    }
}

/* Projection of the Hashing module with projection_type == "bh4":
 * PL/lookup.py:29-39.  x is [B, H]; zero-pad to D (":32-34"); z = decay * bh4(x)
 * + (1 - decay) * tile(x, R) (":36"); keep the first out_dim columns and add
 * the bias (":37").  z is [B, out_dim]. */
void FN(orc_projection)(const REAL *x, const REAL *w, const REAL *bias, REAL *z,
                        int64_t B, int64_t H, int64_t D, int64_t R, int64_t J,
                        int64_t bs, int64_t out_dim, REAL decay)
{
    REAL *xp = (REAL *)calloc((size_t)(B * D), sizeof(REAL));
    REAL *y = (REAL *)malloc((size_t)(B * R * D) * sizeof(REAL));
    for (int64_t b = 0; b < B; b++)
        memcpy(xp + b * D, x + b * H, (size_t)H * sizeof(REAL));
    FN(orc_bh4)(xp, w, y, B, D, R, J, bs);
#pragma omp parallel for schedule(static)
    for (int64_t b = 0; b < B; b++)
        for (int64_t c = 0; c < out_dim; c++) {
            REAL v = decay * y[b * R * D + c] + ((REAL)1 - decay) * xp[b * D + (c % D)];
            z[b * out_dim + c] = v + (bias ? bias[c] : (REAL)0);
        }
    free(xp);
    free(y);
}

/* Code and score per (token, table): PL/compute_code_score/torch_extension.cc:28-41.
 *   code  = sum_d (z_d > 0) << (k-1-d)      (MSB first, strict >, ":35")
 *   score = sum_d |z_d| / prod_d (1 + exp(-2 |z_d|))   (":36-40", d ascending)
 * z is [N, k] with N = B*T. */
void FN(orc_code_score)(const REAL *z, int32_t *codes, REAL *scores, int64_t N, int64_t k)
{
#pragma omp parallel for schedule(static)
    for (int64_t n = 0; n < N; n++) {
        int32_t code = 0;
        REAL num = 0, den = 1;
        for (int64_t d = 0; d < k; d++) {
            REAL hs = z[n * k + d];
            REAL a = ABS(hs);
            code = code + (hs > 0) * (1 << (k - d - 1));
            num = num + a;
            den = den * ((REAL)1 + EXP(-(REAL)2 * a));
        }
        codes[n] = code;
        scores[n] = num / den;
    }
}

/* Gradient of the score w.r.t. z (the code has none: PL/compute_code_score/kernel.py:48
 * casts it to int).  Differentiating PL/compute_code_score/kernel.py:51-53 the way
 * torch autograd does (abs'(0) = 0):
 *   S = sum |z|, P = prod (1 + e_d), e_d = exp(-2|z_d|)
 *   d score / d z_j = sgn(z_j) * (1 + S * 2 e_j / (1 + e_j)) / P
 * g_z[n,j] = g_score[n] * that. */
void FN(orc_code_score_bwd)(const REAL *z, const REAL *g_score, REAL *g_z, int64_t N, int64_t k)
{
#pragma omp parallel for schedule(static)
    for (int64_t n = 0; n < N; n++) {
        REAL S = 0, P = 1;
        for (int64_t d = 0; d < k; d++) {
            REAL a = ABS(z[n * k + d]);
            S += a;
            P *= (REAL)1 + EXP(-(REAL)2 * a);
        }
        for (int64_t d = 0; d < k; d++) {
            REAL v = z[n * k + d];
            REAL a = ABS(v);
            REAL e = EXP(-(REAL)2 * a);
            REAL sg = (v > 0) ? (REAL)1 : ((v < 0) ? (REAL)-1 : (REAL)0);
            g_z[n * k + d] = g_score[n] * sg * ((REAL)1 + S * (REAL)2 * e / ((REAL)1 + e)) / P;
        }
    }
}

/* out[b,:] = sum_i w[b,i] * src[idx[b,i],:], i ascending, accumulated in REAL.
 * Follows the scalar x86 loop PL/gather/cpu/torch_extension.cpp:36-44 and the
 * GPU loop PL/gather/cuda/extension/gather_kernel_fp32.cu:41-43 (same order). */
void FN(orc_gather_add)(const int32_t *idx, const REAL *src, const REAL *w, REAL *out,
                        int64_t B, int64_t I, int64_t Dv)
{
#pragma omp parallel for schedule(static)
    for (int64_t b = 0; b < B; b++) {
        REAL *o = out + b * Dv;
        for (int64_t d = 0; d < Dv; d++) o[d] = 0;
        for (int64_t i = 0; i < I; i++) {
            const REAL *row = src + (int64_t)idx[b * I + i] * Dv;
            const REAL wt = w[b * I + i];
            for (int64_t d = 0; d < Dv; d++) o[d] += row[d] * wt;
        }
    }
}

/* Same with the rows stored as bfloat16 (upper 16 bits of an IEEE float32) and
 * REAL accumulation: the reduced-precision table format of this build (the
 * reference's own reduced format is fp16 storage with fp16 accumulation,
 * PL/gather/cuda/extension/gather_kernel_fp16.cu:56-57, whose rounding only
 * CUDA hardware can show). */
void FN(orc_gather_add_bf16)(const int32_t *idx, const uint16_t *src, const REAL *w, REAL *out,
                             int64_t B, int64_t I, int64_t Dv)
{
#pragma omp parallel for schedule(static)
    for (int64_t b = 0; b < B; b++) {
        REAL *o = out + b * Dv;
        for (int64_t d = 0; d < Dv; d++) o[d] = 0;
        for (int64_t i = 0; i < I; i++) {
            const uint16_t *row = src + (int64_t)idx[b * I + i] * Dv;
            const REAL wt = w[b * I + i];
            for (int64_t d = 0; d < Dv; d++) {
                union { uint32_t u; float f; } cv;
                cv.u = (uint32_t)row[d] << 16;
                o[d] += (REAL)cv.f * wt;
            }
        }
    }
}

/* out[b,i] = <g[b,:], src[idx[b,i],:]>: PL/gather/cuda/kernel.py:95-107 (the
 * reference's own slow formula) / gather_kernel_fp32.cu:129-145. */
void FN(orc_indexed_inner_product)(const int32_t *idx, const REAL *g, const REAL *src, REAL *out,
                                   int64_t B, int64_t I, int64_t Dv)
{
#pragma omp parallel for schedule(static)
    for (int64_t b = 0; b < B; b++)
        for (int64_t i = 0; i < I; i++) {
            const REAL *row = src + (int64_t)idx[b * I + i] * Dv;
            REAL acc = 0;
            for (int64_t d = 0; d < Dv; d++) acc += g[b * Dv + d] * row[d];
            out[b * I + i] = acc;
        }
}

/* out[idx[b,i],:] += w[b,i] * g[b,:] into a zeroed [Sz, Dv] buffer, b then i
 * ascending: PL/gather/cuda/kernel.py:149-156 / gather_kernel_fp32.cu:83-91
 * (the GPU order is whatever the atomics give; this is one valid order).
 * Serial on purpose: the accumulation order is part of the definition. */
void FN(orc_scatter_add)(const int32_t *idx, const REAL *g, const REAL *w, REAL *out,
                         int64_t B, int64_t I, int64_t Sz, int64_t Dv)
{
    memset(out, 0, (size_t)(Sz * Dv) * sizeof(REAL));
    for (int64_t b = 0; b < B; b++)
        for (int64_t i = 0; i < I; i++) {
            REAL *row = out + (int64_t)idx[b * I + i] * Dv;
            const REAL wt = w[b * I + i];
            for (int64_t d = 0; d < Dv; d++) row[d] += wt * g[b * Dv + d];
        }
}

/* torch.nn.LayerNorm over the last dim (biased variance, eps inside the sqrt):
 * PL/lookup.py:84,99. */
void FN(orc_layernorm)(const REAL *x, const REAL *gamma, const REAL *beta, REAL eps, REAL *out,
                       int64_t B, int64_t H)
{
#pragma omp parallel for schedule(static)
    for (int64_t b = 0; b < B; b++) {
        const REAL *r = x + b * H;
        REAL mean = 0, var = 0;
        for (int64_t h = 0; h < H; h++) mean += r[h];
        mean /= (REAL)H;
        for (int64_t h = 0; h < H; h++) var += (r[h] - mean) * (r[h] - mean);
        var /= (REAL)H;
        const REAL rstd = (REAL)1 / SQRT(var + eps);
        for (int64_t h = 0; h < H; h++)
            out[b * H + h] = (r[h] - mean) * rstd * gamma[h] + beta[h];
    }
}

/* Whole layer forward: PL/lookup.py:98-130.
 *   h = LayerNorm(x); z = projection(h).view(B,T,k); (code, score) = code_score(z)
 *   idx = code + arange(T)*S (":126"); out = gather_add(idx, tables.view(T*S,Do), score) + bias (":108")
 * Optional outputs (NULL to skip): z_out [B,T*k], codes_out [B,T], scores_out [B,T]. */
void FN(orc_lookup_ffn)(const REAL *x, const REAL *ln_w, const REAL *ln_b, REAL eps,
                        const REAL *proj_w, const REAL *proj_b, REAL decay,
                        const REAL *tables, const REAL *bias, REAL *out,
                        REAL *z_out, int32_t *codes_out, REAL *scores_out,
                        int64_t B, int64_t H, int64_t D, int64_t R, int64_t J, int64_t bs,
                        int64_t T, int64_t k, int64_t Do)
{
    const int64_t S = (int64_t)1 << k;
    REAL *h = (REAL *)malloc((size_t)(B * H) * sizeof(REAL));
    REAL *z = (REAL *)malloc((size_t)(B * T * k) * sizeof(REAL));
    int32_t *code = (int32_t *)malloc((size_t)(B * T) * sizeof(int32_t));
    REAL *score = (REAL *)malloc((size_t)(B * T) * sizeof(REAL));
    FN(orc_layernorm)(x, ln_w, ln_b, eps, h, B, H);
    FN(orc_projection)(h, proj_w, proj_b, z, B, H, D, R, J, bs, T * k, decay);
    FN(orc_code_score)(z, code, score, B * T, k);
    if (z_out) memcpy(z_out, z, (size_t)(B * T * k) * sizeof(REAL));
    if (codes_out) memcpy(codes_out, code, (size_t)(B * T) * sizeof(int32_t));
    if (scores_out) memcpy(scores_out, score, (size_t)(B * T) * sizeof(REAL));
    for (int64_t b = 0; b < B; b++)
        for (int64_t t = 0; t < T; t++) code[b * T + t] += (int32_t)(t * S);
    FN(orc_gather_add)(code, tables, score, out, B, T, Do);
    if (bias)
        for (int64_t b = 0; b < B; b++)
            for (int64_t d = 0; d < Do; d++) out[b * Do + d] += bias[d];
    free(h);
    free(z);
    free(code);
    free(score);
}
