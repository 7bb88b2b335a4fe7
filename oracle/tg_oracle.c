/* TEST INFRASTRUCTURE, NOT PRODUCT CODE.  See tg_oracle.h for what this is and how it is pinned.
 *
 * Scalar C restatement of the reference's arithmetic, written so that every output element
 * sees the same sequence of fp32 operations (same operands, same order, same fused/unfused
 * choice) as the reference's AVX2 code.  Build with -ffp-contract=off and WITHOUT -ffast-math:
 * every fused multiply-add below is an explicit fmaf().
 */
#include "tg_oracle.h"

#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

/* ------------------------------------------------------------------------------------------ */
/* shapes                                                                                     */
/* ------------------------------------------------------------------------------------------ */

int tgo_config_named(const char *name, tgo_config *out) {
	/* config.hpp:46-48 */
	tgo_config c = {0, 0, 0, 262144, 32768, 512, 256, 4, 1, 1000000.0f, 10000.0f, 6};
	if (strcmp(name, "270m") == 0) {
		c.hidden = 640; c.ffn = 2048; c.n_layers = 18;
	} else if (strcmp(name, "1B") == 0) {
		c.hidden = 1152; c.ffn = 6912; c.n_layers = 26;
	} else {
		return -1;
	}
	*out = c;
	return 0;
}

int tgo_legal_in(int d) { /* ROW_SWITCH, static_switch.hpp:7-30 */
	return d == 640 || d == 2048 || d == 1024 || d == 256 || d == 1152 || d == 6912;
}
int tgo_legal_out(int d) { /* COL_SWITCH, static_switch.hpp:32-58 */
	return d == 640 || d == 262144 || d == 2048 || d == 256 || d == 1024 || d == 1152 || d == 6912;
}

/* ------------------------------------------------------------------------------------------ */
/* GEMV / GEMM (linalg.hpp)                                                                   */
/* ------------------------------------------------------------------------------------------ */

static void scale_cols(float *y, const float *s, int out) { /* linalg.hpp:83-107, 151-173 */
	for (int c = 0; c < out; c++) y[c] = y[c] * s[c];
}

/* gemv::qgemv, linalg.hpp:46-81: per input row, product rounded to fp32, then added to y */
static void gemv_rows(float *y, const float *x, const int8_t *W, int in, int out) {
	for (int r = 0; r < in; r++) {
		const float xr = x[r];
		const int8_t *w = W + (size_t)r * out;
		for (int c = 0; c < out; c++) {
			float p = xr * (float)w[c];
			y[c] = y[c] + p;
		}
	}
}

/* gemv::qgemv_row_tile<.,.,T>, linalg.hpp:119-149: fused chain over T rows from 0, then one add into y */
#define GEMV_TILE(NAME, T)                                                                  \
	static void NAME(float *y, const float *x, const int8_t *W, int in, int out) {          \
		for (int r = 0; r < in; r += T) {                                                   \
			const int8_t *w = W + (size_t)r * out;                                          \
			for (int c = 0; c < out; c++) {                                                 \
				float acc = 0.0f;                                                           \
				for (int t = 0; t < T; t++) acc = fmaf(x[r + t], (float)w[(size_t)t * out + c], acc); \
				y[c] = y[c] + acc;                                                          \
			}                                                                               \
		}                                                                                   \
	}
GEMV_TILE(gemv_tile4, 4)
GEMV_TILE(gemv_tile8, 8)

int tgo_qgemv(float *y, const float *x, const int8_t *W, const float *s, int in, int out) {
	if (!tgo_legal_in(in) || !tgo_legal_out(out)) return -1;
	if (out == 6912) /* linalg.hpp:177-185 */
		gemv_tile8(y, x, W, in, out);
	else
		gemv_rows(y, x, W, in, out);
	scale_cols(y, s, out);
	return 0;
}

int tgo_qgemv_logits(float *y, const float *x, const int8_t *W, const float *s, int in, int out) {
	if (!tgo_legal_in(in) || !tgo_legal_out(out)) return -1;
	gemv_tile4(y, x, W, in, out); /* linalg.hpp:197-204 */
	scale_cols(y, s, out);
	return 0;
}

/* gemm::qgemmnn + microkernel, linalg.hpp:215-248: one fused chain over k = 0..K-1 per element,
 * scale applied once, C overwritten */
int tgo_qgemm(float *C, const float *A, const int8_t *B, const float *s, int m, int in, int out) {
	if (!tgo_legal_in(in) || !tgo_legal_out(out)) return -1;
	float *acc = (float *)malloc(sizeof(float) * (size_t)out);
	for (int i = 0; i < m; i++) {
		const float *a = A + (size_t)i * in;
		for (int c = 0; c < out; c++) acc[c] = 0.0f;
		for (int k = 0; k < in; k++) {
			const float ak = a[k];
			const int8_t *b = B + (size_t)k * out;
			for (int c = 0; c < out; c++) acc[c] = fmaf(ak, (float)b[c], acc[c]);
		}
		float *crow = C + (size_t)i * out;
		for (int c = 0; c < out; c++) crow[c] = acc[c] * s[c];
	}
	free(acc);
	return 0;
}

/* ------------------------------------------------------------------------------------------ */
/* reductions in the reference's lane order (simd.hpp:16-34)                                  */
/* ------------------------------------------------------------------------------------------ */

/* 32 interleaved partials p[i] (element d goes to partial d % 32) -> scalar:
 * reduce_horizontalx4: (a+b)+(c+d) per lane, then v_hsum's hadd tree */
static float reduce32(const float p[32]) {
	float a[8];
	for (int l = 0; l < 8; l++) a[l] = (p[l] + p[8 + l]) + (p[16 + l] + p[24 + l]);
	return ((a[0] + a[1]) + (a[2] + a[3])) + ((a[4] + a[5]) + (a[6] + a[7]));
}

/* dot product as in ops.hpp:305-314 / 451-461: fused partials, then reduce32 */
static float dot_lanes(const float *q, const float *k, int dim) {
	float p[32];
	for (int i = 0; i < 32; i++) p[i] = 0.0f;
	for (int d = 0; d < dim; d += 32)
		for (int i = 0; i < 32; i++) p[i] = fmaf(q[d + i], k[d + i], p[i]);
	return reduce32(p);
}

/* ------------------------------------------------------------------------------------------ */
/* ops                                                                                        */
/* ------------------------------------------------------------------------------------------ */

/* ops.hpp:126-180.  The reference writes ms = ms + x*x with plain vector operators, which its
 * build flags contract to a fused multiply-add. */
void tgo_rmsnorm(float *x, const float *w, int rows, int dim) {
	const float eps = 1e-06f;
	for (int r = 0; r < rows; r++) {
		float *a = x + (size_t)r * dim;
		float p[32];
		for (int i = 0; i < 32; i++) p[i] = 0.0f;
		for (int d = 0; d < dim; d += 32)
			for (int i = 0; i < 32; i++) p[i] = fmaf(a[d + i], a[d + i], p[i]);
		const float ms = reduce32(p) / (float)dim;
		const float irms = 1.0f / sqrtf(ms + eps);
		for (int d = 0; d < dim; d++) a[d] = (a[d] * irms) * (w[d] + 1.0f);
	}
}

/* decode.hpp:176-201 */
void tgo_rope_tables(float theta, int n_pos, int dhead, float *cos_out, float *sin_out) {
	const int dhalf = dhead / 2;
	float *freqs = (float *)malloc(sizeof(float) * (size_t)dhalf);
	for (int i = 0; i < dhalf; i++) {
		float denom = powf(theta, (float)(2 * i) / (float)dhead);
		freqs[i] = 1.0f / denom;
	}
	for (int p = 0; p < n_pos; p++) {
		for (int d = 0; d < dhalf; d++) {
			float outer = (float)p * freqs[d];
			float c = cosf(outer), s = sinf(outer);
			size_t i = (size_t)p * dhead + d;
			cos_out[i] = c; cos_out[i + dhalf] = c;
			sin_out[i] = s; sin_out[i + dhalf] = s;
		}
	}
	free(freqs);
}

/* decode.hpp:136-174, 203-211: x = cos*x + rotate_half(x)*sin, x is [heads][seq][dhead] */
void tgo_rope_apply(float *x, int heads, int seq, int dhead, const float *cos_t, const float *sin_t, int offset) {
	const int h2 = dhead / 2;
	float rot[1024];
	for (int h = 0; h < heads; h++) {
		for (int s = 0; s < seq; s++) {
			float *v = x + ((size_t)h * seq + s) * dhead;
			const float *c = cos_t + (size_t)(s + offset) * dhead;
			const float *sn = sin_t + (size_t)(s + offset) * dhead;
			for (int i = 0; i < h2; i++) { rot[i] = -v[i + h2]; rot[i + h2] = v[i]; }
			for (int d = 0; d < dhead; d++) v[d] = fmaf(c[d], v[d], rot[d] * sn[d]);
		}
	}
}

/* ops.hpp:16-39: tanh-GeLU evaluated in double at x = min + i*eps, stored fp32 */
void tgo_gelu_table(float gmin, float gmax, int size, float *table) {
	const float eps = (float)(gmax - gmin) / (float)size;
	const float c0 = 0.7978845608f, c1 = 0.044715f;
	for (int i = 0; i < size; i++) {
		float x = gmin + (float)i * eps;
		double a = (double)x;
		table[i] = (float)((0.5 * a) * (1.0 + tanh((double)c0 * (a + (double)c1 * (a * a * a)))));
	}
}

/* ops.hpp:41-51: truncating index; below range -> 0, above range -> x */
void tgo_gelu(float *x, size_t n, const float *table, float gmin, float gmax, int size) {
	const float eps = (float)(gmax - gmin) / (float)size;
	for (size_t i = 0; i < n; i++) {
		int idx = (int)((x[i] - gmin) / eps);
		if (idx < 0) x[i] = 0.0f;
		else if (idx < size) x[i] = table[idx];
	}
}

/* ops.hpp:537-568: s[d] * (sqrt(hidden) * q) */
void tgo_embedding(float *out, const int32_t *ids, int n, const int8_t *wte, const float *scales, int hidden) {
	const float scale = (float)sqrt((double)hidden);
	for (int t = 0; t < n; t++) {
		const int8_t *row = wte + (size_t)ids[t] * hidden;
		float *o = out + (size_t)t * hidden;
		for (int d = 0; d < hidden; d++) o[d] = scales[d] * (scale * (float)row[d]);
	}
}

/* ops.hpp:410-524. q,o [heads][S][dim]; k,v [S][dim] (one KV head).
 * Local layers start at qs - sw_context: sw_context + 1 keys (ops.hpp:437-443). */
void tgo_attention_prefill(float *o, const float *q, const float *k, const float *v, int heads, int S, int dim, int is_sw, int sw_context) {
	const float scale = (float)(1.0 / (double)sqrtf((float)dim));
	float *acc = (float *)malloc(sizeof(float) * (size_t)dim);
	for (int h = 0; h < heads; h++) {
		for (int qs = 0; qs < S; qs++) {
			const float *qv = q + ((size_t)h * S + qs) * dim;
			for (int d = 0; d < dim; d++) acc[d] = 0.0f;
			float s_star = 0.0f, m_star = -INFINITY;
			int ks0 = 0;
			if (is_sw) ks0 = (qs >= sw_context) ? qs - sw_context : 0;
			for (int ks = ks0; ks <= qs; ks++) {
				const float *kv = k + (size_t)ks * dim;
				const float *vv = v + (size_t)ks * dim;
				float s = dot_lanes(qv, kv, dim) * scale;
				float m = fmaxf(m_star, s);
				float corr, update;
				if (s > m_star) { corr = expf(m_star - s); update = 1.0f; }
				else { corr = 1.0f; update = expf(s - m_star); }
				for (int d = 0; d < dim; d++) acc[d] = fmaf(vv[d], update, acc[d] * corr);
				s_star = fmaf(s_star, corr, update);
				m_star = m;
			}
			const float inv = 1.0f / s_star;
			float *ov = o + ((size_t)h * S + qs) * dim;
			for (int d = 0; d < dim; d++) ov[d] = acc[d] * inv;
		}
	}
	free(acc);
}

/* ops.hpp:257-367. q,o [heads][dim]; kc,vc [valid..][dim] walked in slot order 0..valid-1;
 * renormalised after every key: o = ((l*o)*corr + e*v) * (1/l') */
void tgo_attention_decode(float *o, const float *q, const float *kc, const float *vc, int heads, int dim, int valid) {
	const float scale = (float)(1.0 / (double)sqrtf((float)dim));
	float *qs = (float *)malloc(sizeof(float) * (size_t)heads * dim);
	float *ms = (float *)malloc(sizeof(float) * (size_t)heads);
	float *ls = (float *)malloc(sizeof(float) * (size_t)heads);
	for (int h = 0; h < heads; h++) {
		ms[h] = -INFINITY; ls[h] = 0.0f;
		for (int d = 0; d < dim; d++) { o[(size_t)h * dim + d] = 0.0f; qs[(size_t)h * dim + d] = q[(size_t)h * dim + d] * scale; }
	}
	for (int j = 0; j < valid; j++) {
		const float *kv = kc + (size_t)j * dim;
		const float *vv = vc + (size_t)j * dim;
		for (int h = 0; h < heads; h++) {
			float s = dot_lanes(qs + (size_t)h * dim, kv, dim);
			float m = fmaxf(ms[h], s);
			float corr = expf(ms[h] - m);
			float update = expf(s - m);
			float l_new = fmaf(corr, ls[h], update);
			float il = 1.0f / l_new;
			float *ov = o + (size_t)h * dim;
			for (int d = 0; d < dim; d++) {
				float t = ls[h] * ov[d];
				t = corr * t;
				t = fmaf(update, vv[d], t);
				ov[d] = t * il;
			}
			ms[h] = m; ls[h] = l_new;
		}
	}
	free(qs); free(ms); free(ls);
}

/* ops.hpp:749-757: strict '>' scan from index 0, so the lowest index wins ties */
int tgo_argmax(const float *logits, int n) {
	float best = -INFINITY;
	int arg = -1;
	for (int i = 0; i < n; i++)
		if (logits[i] > best) { arg = i; best = logits[i]; }
	return arg;
}

/* ops.hpp:762-859.  The reference keeps 4 AVX2 accumulators (32 lanes) for the masked denominator and
 * folds them as (v0+v1)+(v2+v3), then pairs of lanes (two hadd), then the two 128-bit halves
 * (simd.hpp:16-32); that order is followed here.  The mask (p < minp * maxp -> 0) is applied inside
 * the denominator loop only and never stored (ops.hpp:808-826 blend into a local), so every token,
 * also those below the cut, is scaled by 1/denom and takes part in the draw (ops.hpp:836-857). */
int tgo_minp_logits(float *l, int n, float minp, float temp, float randf) {
	for (int i = 0; i < n; i++) l[i] /= temp;              /* :767-769 */
	float rowmax = -INFINITY;
	for (int i = 0; i < n; i++) rowmax = fmaxf(rowmax, l[i]); /* :773-787, max is order independent */
	float maxp = -INFINITY;
	for (int i = 0; i < n; i++) {                          /* :790-797 */
		l[i] = expf(l[i] - rowmax);
		if (l[i] > maxp) maxp = l[i];
	}
	const float cut = minp * maxp;                          /* :800 */
	float lanes[32];
	for (int j = 0; j < 32; j++) lanes[j] = 0.0f;
	for (int i = 0; i < n; i += 32)                         /* :807-827 */
		for (int j = 0; j < 32; j++) lanes[j] += (l[i + j] < cut) ? 0.0f : l[i + j];
	float a[8];
	for (int j = 0; j < 8; j++) a[j] = (lanes[j] + lanes[8 + j]) + (lanes[16 + j] + lanes[24 + j]); /* simd.hpp:27-29 */
	const float denom = ((a[0] + a[1]) + (a[2] + a[3])) + ((a[4] + a[5]) + (a[6] + a[7]));            /* simd.hpp:17-22 */
	const float inv = (float)(1.0 / (double)denom);         /* :836 */
	for (int i = 0; i < n; i++) l[i] *= inv;                /* :838-846 */
	float cum = 0.0f;                                       /* :849-857 */
	int index = 0;
	for (int i = 0; i < n; i++) {
		cum += l[i];
		if (cum >= randf) { index = i; break; }
	}
	return index;
}

/* ------------------------------------------------------------------------------------------ */
/* quantizer + generator                                                                      */
/* ------------------------------------------------------------------------------------------ */

/* py/weight_handlers.py:10-20: scales = max|w| over axis 0 / 127 (fp32); q = rint(w / scales) */
int tgo_quantize(const float *w, size_t rows, size_t cols, int8_t *q, float *scales) {
	for (size_t c = 0; c < cols; c++) scales[c] = 0.0f;
	for (size_t r = 0; r < rows; r++) {
		const float *wr = w + r * cols;
		for (size_t c = 0; c < cols; c++) {
			float a = fabsf(wr[c]);
			if (a > scales[c]) scales[c] = a;
		}
	}
	int bad = 0;
	for (size_t c = 0; c < cols; c++) {
		if (scales[c] == 0.0f) bad = 1;
		scales[c] = scales[c] / 127.0f;
	}
	if (bad) return -1;
#pragma omp parallel for schedule(static)
	for (size_t r = 0; r < rows; r++) {
		const float *wr = w + r * cols;
		int8_t *qr = q + r * cols;
		for (size_t c = 0; c < cols; c++) qr[c] = (int8_t)rintf(wr[c] / scales[c]);
	}
	return 0;
}

static inline uint64_t mix64(uint64_t z) { /* splitmix64 finaliser */
	z = (z ^ (z >> 30)) * 0xbf58476d1ce4e5b9ULL;
	z = (z ^ (z >> 27)) * 0x94d049bb133111ebULL;
	return z ^ (z >> 31);
}

/* inverse normal CDF, P. Acklam's rational approximation (relative error < 1.2e-9) */
static double inv_norm_cdf(double p) {
	static const double a[] = {-3.969683028665376e+01, 2.209460984245205e+02, -2.759285104469687e+02,
	                           1.383577518672690e+02, -3.066479806614716e+01, 2.506628277459239e+00};
	static const double b[] = {-5.447609879822406e+01, 1.615858368580409e+02, -1.556989798598866e+02,
	                           6.680131188771972e+01, -1.328068155288572e+01};
	static const double c[] = {-7.784894002430293e-03, -3.223964580411365e-01, -2.400758277161838e+00,
	                           -2.549732539343734e+00, 4.374664141464968e+00, 2.938163982698783e+00};
	static const double d[] = {7.784695709041462e-03, 3.224671290700398e-01, 2.445134137142996e+00, 3.754408661907416e+00};
	const double plow = 0.02425;
	if (p < plow) {
		double q = sqrt(-2.0 * log(p));
		return (((((c[0] * q + c[1]) * q + c[2]) * q + c[3]) * q + c[4]) * q + c[5]) /
		       ((((d[0] * q + d[1]) * q + d[2]) * q + d[3]) * q + 1.0);
	}
	if (p > 1.0 - plow) {
		double q = sqrt(-2.0 * log(1.0 - p));
		return -(((((c[0] * q + c[1]) * q + c[2]) * q + c[3]) * q + c[4]) * q + c[5]) /
		       ((((d[0] * q + d[1]) * q + d[2]) * q + d[3]) * q + 1.0);
	}
	double q = p - 0.5, r = q * q;
	return (((((a[0] * r + a[1]) * r + a[2]) * r + a[3]) * r + a[4]) * r + a[5]) * q /
	       (((((b[0] * r + b[1]) * r + b[2]) * r + b[3]) * r + b[4]) * r + 1.0);
}

float tgo_normal(uint64_t seed, uint64_t tensor_id, uint64_t i, float std) {
	uint64_t h = mix64(mix64(seed * 0x9e3779b97f4a7c15ULL + tensor_id) + i * 0x9e3779b97f4a7c15ULL);
	double p = ((double)(h >> 11) + 0.5) * (1.0 / 9007199254740992.0);
	return (float)(inv_norm_cdf(p) * (double)std);
}

static void fill_normal(float *dst, size_t n, uint64_t seed, uint64_t tensor_id, float std) {
#pragma omp parallel for schedule(static)
	for (size_t i = 0; i < n; i++) dst[i] = tgo_normal(seed, tensor_id, (uint64_t)i, std);
}

/* byte offsets of every block of the flat file, transformer.hpp:122-160 / py/gemma.py:27-77 */
typedef struct {
	size_t q, qs, k, ks, v, vs, o, os, rmsq, rmsk, apre, apost, u, us, g, gs, d, ds, mpre, mpost;
} layer_off;
typedef struct {
	size_t wte, wte_s, rmsw, lm, lm_s, total;
	layer_off *L;
} file_layout;

static void layout_build(const tgo_config *c, file_layout *f) {
	size_t h = (size_t)c->hidden, ffn = (size_t)c->ffn, V = (size_t)c->vocab;
	size_t qo = (size_t)c->n_head * c->head_dim, kv = (size_t)c->n_kv * c->head_dim, hd = (size_t)c->head_dim;
	size_t p = 0;
	f->wte = p; p += V * h;
	f->wte_s = p; p += 4 * h;
	f->rmsw = p; p += 4 * h;
	f->L = (layer_off *)malloc(sizeof(layer_off) * (size_t)c->n_layers);
	for (int l = 0; l < c->n_layers; l++) {
		layer_off *o = &f->L[l];
		o->q = p; p += h * qo; o->qs = p; p += 4 * qo;
		o->k = p; p += h * kv; o->ks = p; p += 4 * kv;
		o->v = p; p += h * kv; o->vs = p; p += 4 * kv;
		o->o = p; p += qo * h; o->os = p; p += 4 * h;
		o->rmsq = p; p += 4 * hd; o->rmsk = p; p += 4 * hd;
		o->apre = p; p += 4 * h; o->apost = p; p += 4 * h;
		o->u = p; p += h * ffn; o->us = p; p += 4 * ffn;
		o->g = p; p += h * ffn; o->gs = p; p += 4 * ffn;
		o->d = p; p += ffn * h; o->ds = p; p += 4 * h;
		o->mpre = p; p += 4 * h; o->mpost = p; p += 4 * h;
	}
	f->lm = p; p += h * V;
	f->lm_s = p; p += 4 * V;
	f->total = p;
}

size_t tgo_weight_file_bytes(const tgo_config *cfg) {
	file_layout f;
	layout_build(cfg, &f);
	free(f.L);
	return f.total;
}

static int gen_quant(uint8_t *buf, size_t off_q, size_t off_s, size_t rows, size_t cols, uint64_t seed, uint64_t id, float *tmp) {
	fill_normal(tmp, rows * cols, seed, id, 0.02f);
	return tgo_quantize(tmp, rows, cols, (int8_t *)(buf + off_q), (float *)(buf + off_s));
}

int tgo_generate_weights_mem(const tgo_config *c, uint64_t seed, void *bufv) {
	uint8_t *buf = (uint8_t *)bufv;
	file_layout f;
	layout_build(c, &f);
	size_t h = (size_t)c->hidden, ffn = (size_t)c->ffn, V = (size_t)c->vocab;
	size_t qo = (size_t)c->n_head * c->head_dim, kv = (size_t)c->n_kv * c->head_dim, hd = (size_t)c->head_dim;
	size_t biggest = V * h;
	if (h * ffn > biggest) biggest = h * ffn;
	float *tmp = (float *)malloc(sizeof(float) * biggest);
	float *tmpT = (float *)malloc(sizeof(float) * V * h);
	int rc = 0;
	/* tensor ids: 0 wte, 1 final norm, 100*l + k for layer l */
	fill_normal(tmp, V * h, seed, 0, 0.02f);
	rc |= tgo_quantize(tmp, V, h, (int8_t *)(buf + f.wte), (float *)(buf + f.wte_s));
	/* tied head: lm_head = wte^T as fp32, quantized along its own axis 0 (py/gemma.py:75, 397-402) */
#pragma omp parallel for schedule(static)
	for (size_t r = 0; r < h; r++)
		for (size_t v = 0; v < V; v++) tmpT[r * V + v] = tmp[v * h + r];
	rc |= tgo_quantize(tmpT, h, V, (int8_t *)(buf + f.lm), (float *)(buf + f.lm_s));
	free(tmpT);
	fill_normal((float *)(buf + f.rmsw), h, seed, 1, 0.1f);
	for (int l = 0; l < c->n_layers; l++) {
		const layer_off *o = &f.L[l];
		uint64_t b = 100ULL * (uint64_t)(l + 1);
		rc |= gen_quant(buf, o->q, o->qs, h, qo, seed, b + 0, tmp);
		rc |= gen_quant(buf, o->k, o->ks, h, kv, seed, b + 1, tmp);
		rc |= gen_quant(buf, o->v, o->vs, h, kv, seed, b + 2, tmp);
		rc |= gen_quant(buf, o->o, o->os, qo, h, seed, b + 3, tmp);
		fill_normal((float *)(buf + o->rmsq), hd, seed, b + 4, 0.1f);
		fill_normal((float *)(buf + o->rmsk), hd, seed, b + 5, 0.1f);
		fill_normal((float *)(buf + o->apre), h, seed, b + 6, 0.1f);
		fill_normal((float *)(buf + o->apost), h, seed, b + 7, 0.1f);
		rc |= gen_quant(buf, o->u, o->us, h, ffn, seed, b + 8, tmp);
		rc |= gen_quant(buf, o->g, o->gs, h, ffn, seed, b + 9, tmp);
		rc |= gen_quant(buf, o->d, o->ds, ffn, h, seed, b + 10, tmp);
		fill_normal((float *)(buf + o->mpre), h, seed, b + 11, 0.1f);
		fill_normal((float *)(buf + o->mpost), h, seed, b + 12, 0.1f);
	}
	free(tmp);
	free(f.L);
	return rc;
}

int tgo_generate_weights_file(const tgo_config *c, uint64_t seed, const char *path) {
	size_t n = tgo_weight_file_bytes(c);
	void *buf = malloc(n);
	if (!buf) return -3;
	int rc = tgo_generate_weights_mem(c, seed, buf);
	if (rc == 0) {
		FILE *fp = fopen(path, "wb");
		if (!fp) rc = -1;
		else {
			if (fwrite(buf, 1, n, fp) != n) rc = -2;
			fclose(fp);
		}
	}
	free(buf);
	return rc;
}

/* ------------------------------------------------------------------------------------------ */
/* model                                                                                      */
/* ------------------------------------------------------------------------------------------ */

struct tgo_model {
	tgo_config cfg;
	file_layout f;
	uint8_t *img; /* the weight file, byte for byte */
};

typedef struct {
	float *k, *v;
	int position_ptr, buffer_ptr, max_pos, is_sw;
} kv_cache;

struct tgo_session {
	tgo_model *m;
	float *cos_g, *sin_g, *cos_l, *sin_l;
	float *table;
	float gmin, gmax;
	int gsize;
	kv_cache *kv;
	int n_layers;
	float *logits;
};

tgo_model *tgo_model_create(const tgo_config *cfg) {
	tgo_model *m = (tgo_model *)calloc(1, sizeof(tgo_model));
	m->cfg = *cfg;
	layout_build(cfg, &m->f);
	m->img = (uint8_t *)malloc(m->f.total);
	return m;
}

int tgo_model_load_file(tgo_model *m, const char *path) {
	FILE *fp = fopen(path, "rb");
	if (!fp) return -1; /* transformer.hpp:163 */
	size_t got = fread(m->img, 1, m->f.total, fp);
	fclose(fp);
	return got == m->f.total ? 0 : -2;
}

int tgo_model_load_mem(tgo_model *m, const void *buf, size_t n) {
	if (n != m->f.total) return -2;
	memcpy(m->img, buf, n);
	return 0;
}

void tgo_model_destroy(tgo_model *m) {
	if (!m) return;
	free(m->img); free(m->f.L); free(m);
}

static int layer_is_local(const tgo_config *c, int l) { return (l % c->pattern) != (c->pattern - 1); } /* transformer.hpp:43 */

tgo_session *tgo_session_create(tgo_model *m, float gmin, float gmax, int gsize) {
	const tgo_config *c = &m->cfg;
	tgo_session *s = (tgo_session *)calloc(1, sizeof(tgo_session));
	s->m = m;
	size_t tn = (size_t)c->n_pos * c->head_dim;
	s->cos_g = (float *)malloc(4 * tn); s->sin_g = (float *)malloc(4 * tn);
	s->cos_l = (float *)malloc(4 * tn); s->sin_l = (float *)malloc(4 * tn);
	tgo_rope_tables(c->theta, c->n_pos, c->head_dim, s->cos_g, s->sin_g);
	tgo_rope_tables(c->theta_local, c->n_pos, c->head_dim, s->cos_l, s->sin_l);
	s->gmin = gmin; s->gmax = gmax; s->gsize = gsize;
	s->table = (float *)malloc(4 * (size_t)gsize);
	tgo_gelu_table(gmin, gmax, gsize, s->table);
	s->n_layers = c->n_layers;
	s->kv = (kv_cache *)calloc((size_t)c->n_layers, sizeof(kv_cache));
	for (int l = 0; l < c->n_layers; l++) {
		kv_cache *kv = &s->kv[l];
		kv->is_sw = layer_is_local(c, l);
		kv->max_pos = kv->is_sw ? c->n_pos_local : c->n_pos; /* decode.hpp:30 */
		size_t n = (size_t)c->n_kv * kv->max_pos * c->head_dim;
		kv->k = (float *)calloc(n, 4); kv->v = (float *)calloc(n, 4);
	}
	s->logits = (float *)malloc(4 * (size_t)c->vocab);
	return s;
}

void tgo_session_destroy(tgo_session *s) {
	if (!s) return;
	for (int l = 0; l < s->n_layers; l++) { free(s->kv[l].k); free(s->kv[l].v); }
	free(s->kv); free(s->cos_g); free(s->sin_g); free(s->cos_l); free(s->sin_l); free(s->table); free(s->logits); free(s);
}

#define W8(off) ((const int8_t *)(m->img + (off)))
#define WF(off) ((const float *)(m->img + (off)))

static void vec_add(float *a, const float *b, size_t n) { for (size_t i = 0; i < n; i++) a[i] = a[i] + b[i]; }
static void vec_mul(float *a, const float *b, size_t n) { for (size_t i = 0; i < n; i++) a[i] = a[i] * b[i]; }

static void finish_logits(tgo_session *s, float *x_last, float *logits_out, int32_t *argmax_out) {
	tgo_model *m = s->m;
	const tgo_config *c = &m->cfg;
	/* modules.hpp:232-246: final norm, zeroed logits, row-tile-4 GEMV; no soft-capping */
	tgo_rmsnorm(x_last, WF(m->f.rmsw), 1, c->hidden);
	memset(s->logits, 0, 4 * (size_t)c->vocab);
	gemv_tile4(s->logits, x_last, W8(m->f.lm), c->hidden, c->vocab);
	scale_cols(s->logits, WF(m->f.lm_s), c->vocab);
	if (logits_out) memcpy(logits_out, s->logits, 4 * (size_t)c->vocab);
	if (argmax_out) *argmax_out = tgo_argmax(s->logits, c->vocab);
}

/* transformer.hpp:49-73 with modules.hpp:98-133, 179-201 */
int tgo_prefill(tgo_session *s, const int32_t *ids, int n, float *logits_out, int32_t *argmax_out, float *taps) {
	tgo_model *m = s->m;
	const tgo_config *c = &m->cfg;
	if (c->n_kv != 1) return -1; /* ops.hpp:394 */
	const int h = c->hidden, ffn = c->ffn, hd = c->head_dim, nh = c->n_head;
	const int qo = nh * hd, kvd = c->n_kv * hd;
	const size_t S = (size_t)n;
	float *x = (float *)malloc(4 * S * h), *xr = (float *)malloc(4 * S * h);
	float *q = (float *)malloc(4 * S * qo), *k = (float *)malloc(4 * S * kvd), *v = (float *)malloc(4 * S * kvd);
	float *qs = (float *)malloc(4 * S * qo), *os = (float *)malloc(4 * S * qo), *xo = (float *)malloc(4 * S * qo);
	float *up = (float *)malloc(4 * S * ffn), *gate = (float *)malloc(4 * S * ffn);

	tgo_embedding(x, ids, n, W8(m->f.wte), WF(m->f.wte_s), h);
	for (int l = 0; l < c->n_layers; l++) {
		const layer_off *o = &m->f.L[l];
		kv_cache *kv = &s->kv[l];
		const float *ct = kv->is_sw ? s->cos_l : s->cos_g, *st = kv->is_sw ? s->sin_l : s->sin_g;
		memcpy(xr, x, 4 * S * h);
		tgo_rmsnorm(x, WF(o->apre), n, h);
		tgo_qgemm(q, x, W8(o->q), WF(o->qs), n, h, qo);
		tgo_qgemm(k, x, W8(o->k), WF(o->ks), n, h, kvd);
		tgo_qgemm(v, x, W8(o->v), WF(o->vs), n, h, kvd);
		for (size_t t = 0; t < S; t++) /* split_rearrange, ops.hpp:670-705 */
			for (int hh = 0; hh < nh; hh++) memcpy(qs + ((size_t)hh * S + t) * hd, q + t * qo + (size_t)hh * hd, 4 * (size_t)hd);
		tgo_rmsnorm(qs, WF(o->rmsq), nh * n, hd);
		tgo_rmsnorm(k, WF(o->rmsk), n, hd);
		tgo_rope_apply(qs, nh, n, hd, ct, st, 0);
		tgo_rope_apply(k, 1, n, hd, ct, st, 0);
		{ /* KVCache::update_prefill, decode.hpp:72-105 */
			if (kv->position_ptr != 0 || kv->buffer_ptr != 0) return -2;
			int start = (n >= kv->max_pos) ? n - kv->max_pos : 0;
			memcpy(kv->k, k + (size_t)start * hd, 4 * (size_t)(n - start) * hd);
			memcpy(kv->v, v + (size_t)start * hd, 4 * (size_t)(n - start) * hd);
			kv->buffer_ptr += (start > 0) ? kv->max_pos : n;
			kv->position_ptr += n;
		}
		tgo_attention_prefill(os, qs, k, v, nh, n, hd, kv->is_sw, kv->max_pos);
		for (int hh = 0; hh < nh; hh++) /* fuse_rearrange, ops.hpp:708-742 */
			for (size_t t = 0; t < S; t++) memcpy(xo + t * qo + (size_t)hh * hd, os + ((size_t)hh * S + t) * hd, 4 * (size_t)hd);
		tgo_qgemm(x, xo, W8(o->o), WF(o->os), n, qo, h);
		tgo_rmsnorm(x, WF(o->apost), n, h);
		vec_add(x, xr, S * h);
		if (taps) memcpy(taps + (size_t)(2 * l) * S * h, x, 4 * S * h);

		memcpy(xr, x, 4 * S * h);
		tgo_rmsnorm(x, WF(o->mpre), n, h);
		tgo_qgemm(up, x, W8(o->u), WF(o->us), n, h, ffn);
		tgo_qgemm(gate, x, W8(o->g), WF(o->gs), n, h, ffn);
		tgo_gelu(gate, S * ffn, s->table, s->gmin, s->gmax, s->gsize);
		vec_mul(gate, up, S * ffn);
		tgo_qgemm(x, gate, W8(o->d), WF(o->ds), n, ffn, h);
		tgo_rmsnorm(x, WF(o->mpost), n, h);
		vec_add(x, xr, S * h);
		if (taps) memcpy(taps + (size_t)(2 * l + 1) * S * h, x, 4 * S * h);
	}
	finish_logits(s, x + (S - 1) * h, logits_out, argmax_out);
	free(x); free(xr); free(q); free(k); free(v); free(qs); free(os); free(xo); free(up); free(gate);
	return 0;
}

/* transformer.hpp:75-97 with modules.hpp:135-169, 203-220 */
int tgo_decode(tgo_session *s, int32_t id, float *logits_out, int32_t *argmax_out, float *taps) {
	tgo_model *m = s->m;
	const tgo_config *c = &m->cfg;
	const int h = c->hidden, ffn = c->ffn, hd = c->head_dim, nh = c->n_head;
	const int qo = nh * hd, kvd = c->n_kv * hd;
	float *x = (float *)malloc(4 * (size_t)h), *xr = (float *)malloc(4 * (size_t)h);
	float *q = (float *)malloc(4 * (size_t)qo), *k = (float *)malloc(4 * (size_t)kvd), *v = (float *)malloc(4 * (size_t)kvd);
	float *os = (float *)malloc(4 * (size_t)qo);
	float *up = (float *)malloc(4 * (size_t)ffn), *gate = (float *)malloc(4 * (size_t)ffn);

	tgo_embedding(x, &id, 1, W8(m->f.wte), WF(m->f.wte_s), h);
	for (int l = 0; l < c->n_layers; l++) {
		const layer_off *o = &m->f.L[l];
		kv_cache *kv = &s->kv[l];
		const float *ct = kv->is_sw ? s->cos_l : s->cos_g, *st = kv->is_sw ? s->sin_l : s->sin_g;
		memcpy(xr, x, 4 * (size_t)h);
		tgo_rmsnorm(x, WF(o->apre), 1, h);
		memset(q, 0, 4 * (size_t)qo); memset(k, 0, 4 * (size_t)kvd); memset(v, 0, 4 * (size_t)kvd);
		tgo_qgemv(q, x, W8(o->q), WF(o->qs), h, qo);
		tgo_qgemv(k, x, W8(o->k), WF(o->ks), h, kvd);
		tgo_qgemv(v, x, W8(o->v), WF(o->vs), h, kvd);
		tgo_rmsnorm(q, WF(o->rmsq), nh, hd); /* [heads][1][hd] has the same bytes as [1][heads*hd] */
		tgo_rmsnorm(k, WF(o->rmsk), c->n_kv, hd);
		tgo_rope_apply(q, nh, 1, hd, ct, st, kv->position_ptr);
		tgo_rope_apply(k, c->n_kv, 1, hd, ct, st, kv->position_ptr);
		{ /* KVCache::update_single, decode.hpp:49-70 */
			size_t slot = (size_t)(kv->buffer_ptr % kv->max_pos);
			memcpy(kv->k + slot * hd, k, 4 * (size_t)hd);
			memcpy(kv->v + slot * hd, v, 4 * (size_t)hd);
			kv->buffer_ptr += 1; kv->position_ptr += 1;
		}
		int valid = kv->max_pos > kv->position_ptr ? kv->position_ptr : kv->max_pos; /* decode.hpp:45-47 */
		tgo_attention_decode(os, q, kv->k, kv->v, nh, hd, valid);
		memset(x, 0, 4 * (size_t)h);
		tgo_qgemv(x, os, W8(o->o), WF(o->os), qo, h);
		tgo_rmsnorm(x, WF(o->apost), 1, h);
		vec_add(x, xr, (size_t)h);
		if (taps) memcpy(taps + (size_t)(2 * l) * h, x, 4 * (size_t)h);

		memcpy(xr, x, 4 * (size_t)h);
		tgo_rmsnorm(x, WF(o->mpre), 1, h);
		memset(up, 0, 4 * (size_t)ffn); memset(gate, 0, 4 * (size_t)ffn);
		tgo_qgemv(up, x, W8(o->u), WF(o->us), h, ffn);
		tgo_qgemv(gate, x, W8(o->g), WF(o->gs), h, ffn);
		tgo_gelu(gate, (size_t)ffn, s->table, s->gmin, s->gmax, s->gsize);
		vec_mul(gate, up, (size_t)ffn);
		memset(x, 0, 4 * (size_t)h);
		tgo_qgemv(x, gate, W8(o->d), WF(o->ds), ffn, h);
		tgo_rmsnorm(x, WF(o->mpost), 1, h);
		vec_add(x, xr, (size_t)h);
		if (taps) memcpy(taps + (size_t)(2 * l + 1) * h, x, 4 * (size_t)h);
	}
	finish_logits(s, x, logits_out, argmax_out);
	free(x); free(xr); free(q); free(k); free(v); free(os); free(up); free(gate);
	return 0;
}

int tgo_kv_read(tgo_session *s, int layer, float *keys, float *values, int *position_ptr, int *buffer_ptr, int *max_pos) {
	kv_cache *kv = &s->kv[layer];
	size_t n = (size_t)kv->max_pos * s->m->cfg.head_dim * s->m->cfg.n_kv;
	if (keys) memcpy(keys, kv->k, 4 * n);
	if (values) memcpy(values, kv->v, 4 * n);
	if (position_ptr) *position_ptr = kv->position_ptr;
	if (buffer_ptr) *buffer_ptr = kv->buffer_ptr;
	if (max_pos) *max_pos = kv->max_pos;
	return 0;
}
