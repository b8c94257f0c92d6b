// seq_kernels.h — device kernels of the layer-list engine (seq.hip).
//
// Everything outside the matrix products is f32: the residual stream, norms, attention
// scores and weights, routers, gates and states of the recurrences. Matrix products take
// their weights as WT (WBF16 or WF32, device_common.h) and accumulate in f32; portions of
// more than GEMV_MAX_M tokens run on the MFMA units with the activations rounded to bf16
// (WBF16) or as f32 FMA tiles (WF32), single tokens and short portions as weight-streaming
// GEMVs that keep the activations in f32. All sizes are runtime arguments.
#pragma once

#include <float.h>
#include <math.h>

#include "device_common.h"

#define SEQ_THREADS 256

// ------------------------------------------------------------------ scalar helpers
__device__ __forceinline__ float sq_sigmoid(float z) {
	return 1.0f / (1.0f + expf(-z));
}
__device__ __forceinline__ float sq_silu(float z) {
	return z / (1.0f + expf(-z));
}
__device__ __forceinline__ float sq_softplus(float z) {
	return z > 20.0f ? z : log1pf(expf(z));
}
__device__ __forceinline__ float sq_gelu_tanh(float z) {
	return 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
}
__device__ __forceinline__ uint16_t f2bf(float x) { // round to nearest even
	const uint32_t u = __builtin_bit_cast(uint32_t, x);
	return (uint16_t)((u + 0x7FFFu + ((u >> 16) & 1u)) >> 16);
}
__device__ __forceinline__ float bf2f(uint16_t b) {
	return __builtin_bit_cast(float, (uint32_t)b << 16);
}
template <class WT>
__device__ __forceinline__ float wload(const void *W, size_t i) {
	if constexpr (WT::BYTES == 4)
		return ((const float *)W)[i];
	else
		return bf2f(((const uint16_t *)W)[i]);
}

// Sum over the workgroup (SEQ_THREADS threads); red: SEQ_THREADS / 64 floats of LDS.
__device__ __forceinline__ float block_sum(float v, float *red) {
	v = wave_sum(v);
	__syncthreads();
	if ((threadIdx.x & 63) == 0)
		red[threadIdx.x >> 6] = v;
	__syncthreads();
	float t = 0.0f;
#pragma unroll
	for (int i = 0; i < SEQ_THREADS / 64; ++i)
		t += red[i];
	return t;
}

// The two norm kinds (YALM_NORM_*): an rms norm divides a row by sqrt(mean(x^2) + eps); a layer
// norm first takes the row's mean off, then divides by sqrt(mean(deviation^2) + eps). Both are
// followed by a weight and have no bias. Kernels take `ln` (1 = layer norm) and subtract the
// mean from the entries they hold before the sum of squares (two passes over values already
// in registers or LDS, so the variance is that of the deviations themselves).

// ------------------------------------------------------------------ embedding
// X[t] = embed[token] * scale (+ the interleaved (sin, cos) position vector of position
// st->pos + t if inv_freq), rms-normed with weight e_norm if e_norm (no mean taken off)
// (+ pre_add, a vector the first layer adds to the stream before its
// opening norm); tokens == nullptr: the single device-resident token of the greedy
// loop. w_next != nullptr: also Hn[t] = norm(X[t]) * w_next, the first layer's opening norm,
// and with w_next2 Hn2[t] = norm(X[t]) * w_next2 (the norm its feed-forward reads).
template <class WT>
__global__ __launch_bounds__(SEQ_THREADS) void seq_embed_kernel(const StepState *__restrict__ st,
                                                                const int *__restrict__ tokens,
                                                                const void *__restrict__ emb,
                                                                const float *__restrict__ inv_freq, int width,
                                                                int vocab, float scale, float *__restrict__ X,
                                                                const float *__restrict__ w_next, float eps,
                                                                float *__restrict__ Hn, int ln,
                                                                const float *__restrict__ pre_add = nullptr,
                                                                const float *__restrict__ e_norm = nullptr,
                                                                const float *__restrict__ w_next2 = nullptr,
                                                                float *__restrict__ Hn2 = nullptr) {
	__shared__ float red[SEQ_THREADS / 64];
	const int t = blockIdx.x;
	int tok = tokens ? tokens[t] : st->token;
	tok = min(max(tok, 0), vocab - 1);
	const float p = (float)(st->pos + t);
	float ss = 0.0f, sm = 0.0f;
	for (int i = threadIdx.x; i < width; i += SEQ_THREADS) {
		float pe = 0.0f;
		if (inv_freq) {
			const float ang = p * inv_freq[i >> 1];
			pe = (i & 1) ? cosf(ang) : sinf(ang);
		}
		float v = wload<WT>(emb, (size_t)tok * width + i) * scale + pe;
		if (pre_add && !e_norm)
			v += pre_add[i];
		X[(size_t)t * width + i] = v;
		ss = fmaf(v, v, ss);
		sm += v;
	}
	if (e_norm) { // the embedding's own norm (each thread re-reads its own entries)
		const float r0 = 1.0f / sqrtf(block_sum(ss, red) / (float)width + eps);
		ss = 0.0f;
		sm = 0.0f;
		for (int i = threadIdx.x; i < width; i += SEQ_THREADS) {
			float v = X[(size_t)t * width + i] * r0 * e_norm[i];
			if (pre_add)
				v += pre_add[i];
			X[(size_t)t * width + i] = v;
			ss = fmaf(v, v, ss);
			sm += v;
		}
	}
	if (!w_next)
		return;
	// the first layer's opening norm in the same launch (each thread re-reads its own entries)
	float mu = 0.0f;
	if (ln) {
		mu = block_sum(sm, red) / (float)width;
		ss = 0.0f;
		for (int i = threadIdx.x; i < width; i += SEQ_THREADS) {
			const float d = X[(size_t)t * width + i] - mu;
			ss = fmaf(d, d, ss);
		}
	}
	ss = block_sum(ss, red);
	const float r = 1.0f / sqrtf(ss / (float)width + eps);
	for (int i = threadIdx.x; i < width; i += SEQ_THREADS) {
		const float v = (X[(size_t)t * width + i] - mu) * r;
		Hn[(size_t)t * width + i] = v * w_next[i];
		if (w_next2)
			Hn2[(size_t)t * width + i] = v * w_next2[i];
	}
}

// ------------------------------------------------------------------ norms
// out[row(t)] = norm(in[t]) * w * post, one workgroup per row. rows != null: the input row
// is rows[t] (gather). pos_rows: the output row is st->pos + t (a cache write).
template <class OT>
__global__ __launch_bounds__(SEQ_THREADS) void seq_norm_kernel(const float *__restrict__ in, int ld_in,
                                                               const float *__restrict__ w, float eps, int n,
                                                               OT *__restrict__ out, int ld_out,
                                                               const int *__restrict__ rows,
                                                               const StepState *__restrict__ st, int pos_rows,
                                                               int ln = 0, float post = 1.0f) {
	__shared__ float red[SEQ_THREADS / 64];
	const int t = blockIdx.x;
	const float *x = in + (size_t)(rows ? rows[t] : t) * ld_in;
	float mu = 0.0f;
	if (ln) {
		float sm = 0.0f;
		for (int i = threadIdx.x; i < n; i += SEQ_THREADS)
			sm += x[i];
		mu = block_sum(sm, red) / (float)n;
	}
	float ss = 0.0f;
	for (int i = threadIdx.x; i < n; i += SEQ_THREADS) {
		const float d = x[i] - mu;
		ss = fmaf(d, d, ss);
	}
	ss = block_sum(ss, red);
	const float r = post / sqrtf(ss / (float)n + eps);
	OT *o = out + (size_t)(pos_rows ? st->pos + t : t) * ld_out;
	for (int i = threadIdx.x; i < n; i += SEQ_THREADS) {
		const float v = (x[i] - mu) * r * w[i];
		if constexpr (sizeof(OT) == 2)
			o[i] = f2bf(v);
		else
			o[i] = v;
	}
}

// Two row norms of the same rows in one launch (blockIdx.y picks the segment): the query
// latent into a f32 buffer and the key/value latent into the cache at rows st->pos + t.
template <class OT>
__global__ __launch_bounds__(SEQ_THREADS) void seq_norm2_kernel(const float *__restrict__ in, int ld_in, int n0,
                                                                const float *__restrict__ w0, float *__restrict__ out0,
                                                                int n1, const float *__restrict__ w1,
                                                                OT *__restrict__ out1, float eps,
                                                                const StepState *__restrict__ st) {
	__shared__ float red[SEQ_THREADS / 64];
	const int t = blockIdx.x, seg = blockIdx.y;
	const int n = seg ? n1 : n0;
	const float *x = in + (size_t)t * ld_in + (seg ? n0 : 0);
	const float *w = seg ? w1 : w0;
	float ss = 0.0f;
	for (int i = threadIdx.x; i < n; i += SEQ_THREADS)
		ss = fmaf(x[i], x[i], ss);
	ss = block_sum(ss, red);
	const float r = 1.0f / sqrtf(ss / (float)n + eps);
	for (int i = threadIdx.x; i < n; i += SEQ_THREADS) {
		const float v = x[i] * r * w[i];
		if (!seg) {
			out0[(size_t)t * n0 + i] = v;
		} else {
			OT *o = out1 + (size_t)(st->pos + t) * n1;
			if constexpr (sizeof(OT) == 2)
				o[i] = f2bf(v);
			else
				o[i] = v;
		}
	}
}

// The seam between two sublayers in one launch: X[t] += norm(Y[t]) * wb (the closing norm
// of the sublayer that produced Y and the residual sum), then, if w_next, Hn[t] =
// norm(X[t]) * w_next (the opening norm of the next sublayer). Dynamic LDS: n floats.
// Rows of up to E * SEQ_THREADS entries without a combine: the row of Y, the row of X and both
// weight vectors are loaded at once (one memory round trip instead of one per pass) and the
// row lives in registers.
template <int E>
__global__ __launch_bounds__(SEQ_THREADS) void seq_add_norm_reg_kernel(float *__restrict__ X,
                                                                       const float *__restrict__ Y,
                                                                       const float *__restrict__ wb, float eps, int n,
                                                                       const float *__restrict__ w_next,
                                                                       float *__restrict__ Hn, int ln) {
	__shared__ float red[SEQ_THREADS / 64];
	const int t = blockIdx.x;
	float y[E], x[E], b[E], wn[E];
#pragma unroll
	for (int e = 0; e < E; ++e) {
		const int i = threadIdx.x + e * SEQ_THREADS;
		const bool in = i < n;
		y[e] = in ? Y[(size_t)t * n + i] : 0.0f;
		x[e] = in ? X[(size_t)t * n + i] : 0.0f;
		b[e] = in ? wb[i] : 0.0f;
		wn[e] = (in && w_next) ? w_next[i] : 0.0f;
	}
	if (ln) { // entries past the row's end stay 0
		float sm = 0.0f;
#pragma unroll
		for (int e = 0; e < E; ++e)
			sm += y[e];
		const float mu = block_sum(sm, red) / (float)n;
#pragma unroll
		for (int e = 0; e < E; ++e)
			if (threadIdx.x + e * SEQ_THREADS < n)
				y[e] -= mu;
	}
	float ss = 0.0f;
#pragma unroll
	for (int e = 0; e < E; ++e)
		ss = fmaf(y[e], y[e], ss);
	ss = block_sum(ss, red);
	const float r = 1.0f / sqrtf(ss / (float)n + eps);
	float s2 = 0.0f, sm2 = 0.0f;
#pragma unroll
	for (int e = 0; e < E; ++e) {
		const int i = threadIdx.x + e * SEQ_THREADS;
		x[e] = x[e] + y[e] * r * b[e];
		if (i < n) {
			X[(size_t)t * n + i] = x[e];
			s2 = fmaf(x[e], x[e], s2);
			sm2 += x[e];
		}
	}
	if (!w_next)
		return;
	if (ln) {
		const float mu = block_sum(sm2, red) / (float)n;
		s2 = 0.0f;
#pragma unroll
		for (int e = 0; e < E; ++e)
			if (threadIdx.x + e * SEQ_THREADS < n) {
				x[e] -= mu;
				s2 = fmaf(x[e], x[e], s2);
			}
	}
	s2 = block_sum(s2, red);
	const float r2 = 1.0f / sqrtf(s2 / (float)n + eps);
#pragma unroll
	for (int e = 0; e < E; ++e) {
		const int i = threadIdx.x + e * SEQ_THREADS;
		if (i < n)
			Hn[(size_t)t * n + i] = x[e] * r2 * wn[e];
	}
}

// Yx != null: Y is not read; its row is the routed experts' combine sum_k wt[t][k] Yx[t top + k]
// (+ sgate[t] Ys[t], the shared expert), summed in slot order.
__global__ __launch_bounds__(SEQ_THREADS) void seq_add_norm_kernel(float *__restrict__ X, const float *__restrict__ Y,
                                                                   const float *__restrict__ wb, float eps, int n,
                                                                   const float *__restrict__ w_next,
                                                                   float *__restrict__ Hn,
                                                                   const float *__restrict__ Yx,
                                                                   const float *__restrict__ wt, int top,
                                                                   const float *__restrict__ Ys,
                                                                   const float *__restrict__ sgate, int ln) {
	extern __shared__ float row[];
	__shared__ float red[SEQ_THREADS / 64];
	const int t = blockIdx.x;
	float *x = X + (size_t)t * n;
	float ss = 0.0f, sm = 0.0f;
	for (int i = threadIdx.x; i < n; i += SEQ_THREADS) {
		float v;
		if (Yx) {
			v = 0.0f;
			for (int k = 0; k < top; ++k)
				v = fmaf(wt[(size_t)t * top + k], Yx[((size_t)t * top + k) * n + i], v);
			if (Ys)
				v = fmaf(sgate[t], Ys[(size_t)t * n + i], v);
		} else {
			v = Y[(size_t)t * n + i];
		}
		row[i] = v;
		ss = fmaf(v, v, ss);
		sm += v;
	}
	float mu = 0.0f;
	if (ln) { // each thread re-reads the entries it wrote
		mu = block_sum(sm, red) / (float)n;
		ss = 0.0f;
		for (int i = threadIdx.x; i < n; i += SEQ_THREADS) {
			const float d = row[i] - mu;
			ss = fmaf(d, d, ss);
		}
	}
	ss = block_sum(ss, red);
	const float r = 1.0f / sqrtf(ss / (float)n + eps);
	float s2 = 0.0f, sm2 = 0.0f;
	for (int i = threadIdx.x; i < n; i += SEQ_THREADS) {
		const float v = x[i] + (row[i] - mu) * r * wb[i];
		x[i] = v;
		row[i] = v;
		s2 = fmaf(v, v, s2);
		sm2 += v;
	}
	if (!w_next)
		return;
	float mu2 = 0.0f;
	if (ln) {
		mu2 = block_sum(sm2, red) / (float)n;
		s2 = 0.0f;
		for (int i = threadIdx.x; i < n; i += SEQ_THREADS) {
			const float d = row[i] - mu2;
			s2 = fmaf(d, d, s2);
		}
	}
	s2 = block_sum(s2, red);
	const float r2 = 1.0f / sqrtf(s2 / (float)n + eps);
	for (int i = threadIdx.x; i < n; i += SEQ_THREADS)
		Hn[(size_t)t * n + i] = (row[i] - mu2) * r2 * w_next[i];
}

// The seam after a parallel block, one launch: X[t] += s1 * Y1[t] + s2 * Y2[t] (s1, s2 the
// block's elementwise scales; Y2 == nullptr and Yx == nullptr: no feed-forward). Yx != nullptr:
// the feed-forward's row is the routed experts' combine sum_k wt[t][k] Yx[t top + k] (+ sgate[t]
// Ys[t], the shared expert; sgate == nullptr: + Ys[t]), summed in slot order. dump != nullptr:
// the row after the sums is also written there (the stream as the block leaves it). Then
// X[t] += add (the vector the next layer adds before its opening norm) and, if w_next, Hn[t]
// = norm(X[t]) * w_next and, with w_next2, Hn2[t] = norm(X[t]) * w_next2 (the norm the next
// block's feed-forward reads). s1 / s2 == nullptr: scale 1. Yb != nullptr: the block has two
// mixers side by side and its mixer row is jscale (rms(Y1[t]) ja + rms(Yb[t]) jb), each row
// divided by its own root mean square over n (no mean taken off). Dynamic LDS: n floats.
__global__ __launch_bounds__(SEQ_THREADS) void seq_par_close_kernel(float *__restrict__ X, const float *__restrict__ Y1,
                                                                    const float *__restrict__ s1,
                                                                    const float *__restrict__ Y2,
                                                                    const float *__restrict__ s2,
                                                                    const float *__restrict__ Yx,
                                                                    const float *__restrict__ wt, int top,
                                                                    const float *__restrict__ Ys,
                                                                    const float *__restrict__ sgate,
                                                                    float *__restrict__ dump,
                                                                    const float *__restrict__ add, float eps, int n,
                                                                    const float *__restrict__ w_next,
                                                                    float *__restrict__ Hn, int ln,
                                                                    const float *__restrict__ w_next2 = nullptr,
                                                                    float *__restrict__ Hn2 = nullptr,
                                                                    const float *__restrict__ Yb = nullptr,
                                                                    const float *__restrict__ ja = nullptr,
                                                                    const float *__restrict__ jb = nullptr,
                                                                    float jscale = 1.0f) {
	extern __shared__ float row[];
	__shared__ float red[SEQ_THREADS / 64];
	const int t = blockIdx.x;
	float *x = X + (size_t)t * n;
	float ra = 1.0f, rb = 0.0f;
	if (Yb) {
		float sa = 0.0f, sb = 0.0f;
		for (int i = threadIdx.x; i < n; i += SEQ_THREADS) {
			const float a = Y1[(size_t)t * n + i], b = Yb[(size_t)t * n + i];
			sa = fmaf(a, a, sa);
			sb = fmaf(b, b, sb);
		}
		ra = jscale / sqrtf(block_sum(sa, red) / (float)n + eps);
		rb = jscale / sqrtf(block_sum(sb, red) / (float)n + eps);
	}
	float ss = 0.0f, sm = 0.0f;
	for (int i = threadIdx.x; i < n; i += SEQ_THREADS) {
		float y1 = Y1[(size_t)t * n + i];
		if (Yb)
			y1 = y1 * ra * ja[i] + Yb[(size_t)t * n + i] * rb * jb[i];
		float v = fmaf(s1 ? s1[i] : 1.0f, y1, x[i]);
		if (Yx) {
			float f = 0.0f;
			for (int k = 0; k < top; ++k)
				f = fmaf(wt[(size_t)t * top + k], Yx[((size_t)t * top + k) * n + i], f);
			if (Ys)
				f = fmaf(sgate ? sgate[t] : 1.0f, Ys[(size_t)t * n + i], f);
			v = fmaf(s2 ? s2[i] : 1.0f, f, v);
		} else if (Y2) {
			v = fmaf(s2 ? s2[i] : 1.0f, Y2[(size_t)t * n + i], v);
		}
		if (dump)
			dump[(size_t)t * n + i] = v;
		if (add)
			v += add[i];
		x[i] = v;
		row[i] = v;
		ss = fmaf(v, v, ss);
		sm += v;
	}
	if (!w_next)
		return;
	float mu = 0.0f;
	if (ln) { // each thread re-reads the entries it wrote
		mu = block_sum(sm, red) / (float)n;
		ss = 0.0f;
		for (int i = threadIdx.x; i < n; i += SEQ_THREADS) {
			const float d = row[i] - mu;
			ss = fmaf(d, d, ss);
		}
	}
	ss = block_sum(ss, red);
	const float r = 1.0f / sqrtf(ss / (float)n + eps);
	for (int i = threadIdx.x; i < n; i += SEQ_THREADS) {
		const float v = (row[i] - mu) * r;
		Hn[(size_t)t * n + i] = v * w_next[i];
		if (w_next2)
			Hn2[(size_t)t * n + i] = v * w_next2[i];
	}
}

// The same seam with the row in registers (rows of up to E * SEQ_THREADS entries): every
// operand row and vector is loaded at once, one memory round trip instead of one per pass.
template <int E>
__global__ __launch_bounds__(SEQ_THREADS) void seq_par_close_reg_kernel(float *__restrict__ X, const float *__restrict__ Y1,
                                                                        const float *__restrict__ s1,
                                                                        const float *__restrict__ Y2,
                                                                        const float *__restrict__ s2,
                                                                        const float *__restrict__ Yx,
                                                                        const float *__restrict__ wt, int top,
                                                                        const float *__restrict__ Ys,
                                                                        const float *__restrict__ sgate,
                                                                        float *__restrict__ dump,
                                                                        const float *__restrict__ add, float eps, int n,
                                                                        const float *__restrict__ w_next,
                                                                        float *__restrict__ Hn, int ln,
                                                                        const float *__restrict__ w_next2 = nullptr,
                                                                        float *__restrict__ Hn2 = nullptr,
                                                                        const float *__restrict__ Yb = nullptr,
                                                                        const float *__restrict__ ja = nullptr,
                                                                        const float *__restrict__ jb = nullptr,
                                                                        float jscale = 1.0f) {
	__shared__ float red[SEQ_THREADS / 64];
	const int t = blockIdx.x;
	float x[E], y1[E], a1[E], f[E], a2[E], ad[E], wn[E];
	const bool ff = Yx || Y2;
#pragma unroll
	for (int e = 0; e < E; ++e) {
		const int i = threadIdx.x + e * SEQ_THREADS;
		const bool in = i < n;
		x[e] = in ? X[(size_t)t * n + i] : 0.0f;
		y1[e] = in ? Y1[(size_t)t * n + i] : 0.0f;
		a1[e] = in ? (s1 ? s1[i] : 1.0f) : 0.0f;
		a2[e] = (in && ff) ? (s2 ? s2[i] : 1.0f) : 0.0f;
		ad[e] = (in && add) ? add[i] : 0.0f;
		wn[e] = (in && w_next) ? w_next[i] : 0.0f;
		f[e] = (in && Y2 && !Yx) ? Y2[(size_t)t * n + i] : 0.0f;
	}
	if (Yb) { // two mixers side by side: the normed rows joined before anything else reads y1
		float yb[E], sa = 0.0f, sb = 0.0f;
#pragma unroll
		for (int e = 0; e < E; ++e) {
			const int i = threadIdx.x + e * SEQ_THREADS;
			yb[e] = i < n ? Yb[(size_t)t * n + i] : 0.0f;
			sa = fmaf(y1[e], y1[e], sa);
			sb = fmaf(yb[e], yb[e], sb);
		}
		const float ra = jscale / sqrtf(block_sum(sa, red) / (float)n + eps);
		const float rb = jscale / sqrtf(block_sum(sb, red) / (float)n + eps);
#pragma unroll
		for (int e = 0; e < E; ++e) {
			const int i = threadIdx.x + e * SEQ_THREADS;
			if (i < n)
				y1[e] = y1[e] * ra * ja[i] + yb[e] * rb * jb[i];
		}
	}
	if (Yx) {
		for (int k = 0; k < top; ++k) {
			const float w = wt[(size_t)t * top + k];
#pragma unroll
			for (int e = 0; e < E; ++e) {
				const int i = threadIdx.x + e * SEQ_THREADS;
				f[e] = fmaf(w, i < n ? Yx[((size_t)t * top + k) * n + i] : 0.0f, f[e]);
			}
		}
		if (Ys) {
			const float w = sgate ? sgate[t] : 1.0f;
#pragma unroll
			for (int e = 0; e < E; ++e) {
				const int i = threadIdx.x + e * SEQ_THREADS;
				f[e] = fmaf(w, i < n ? Ys[(size_t)t * n + i] : 0.0f, f[e]);
			}
		}
	}
	float ss = 0.0f, sm = 0.0f;
#pragma unroll
	for (int e = 0; e < E; ++e) {
		const int i = threadIdx.x + e * SEQ_THREADS;
		float v = fmaf(a1[e], y1[e], x[e]);
		if (ff)
			v = fmaf(a2[e], f[e], v);
		if (dump && i < n)
			dump[(size_t)t * n + i] = v;
		v += ad[e];
		x[e] = v;
		if (i < n) {
			X[(size_t)t * n + i] = v;
			ss = fmaf(v, v, ss);
			sm += v;
		}
	}
	if (!w_next)
		return;
	if (ln) {
		const float mu = block_sum(sm, red) / (float)n;
		ss = 0.0f;
#pragma unroll
		for (int e = 0; e < E; ++e)
			if (threadIdx.x + e * SEQ_THREADS < n) {
				x[e] -= mu;
				ss = fmaf(x[e], x[e], ss);
			}
	}
	ss = block_sum(ss, red);
	const float r = 1.0f / sqrtf(ss / (float)n + eps);
#pragma unroll
	for (int e = 0; e < E; ++e) {
		const int i = threadIdx.x + e * SEQ_THREADS;
		if (i < n) {
			Hn[(size_t)t * n + i] = x[e] * r * wn[e];
			if (w_next2)
				Hn2[(size_t)t * n + i] = x[e] * r * w_next2[i];
		}
	}
}

// Two mixers side by side: Ya[t] <- scale (rms(Ya[t]) wa + rms(Yb[t]) wb), each row divided by
// its own root mean square over n (no mean taken off). One workgroup per token.
__global__ __launch_bounds__(SEQ_THREADS) void seq_pair_join_kernel(float *__restrict__ Ya, const float *__restrict__ Yb,
                                                                    const float *__restrict__ wa,
                                                                    const float *__restrict__ wb, float scale, float eps,
                                                                    int n) {
	__shared__ float red[SEQ_THREADS / 64];
	const int t = blockIdx.x;
	float *a = Ya + (size_t)t * n;
	const float *b = Yb + (size_t)t * n;
	float sa = 0.0f, sb = 0.0f;
	for (int i = threadIdx.x; i < n; i += SEQ_THREADS) {
		sa = fmaf(a[i], a[i], sa);
		sb = fmaf(b[i], b[i], sb);
	}
	const float ra = scale / sqrtf(block_sum(sa, red) / (float)n + eps);
	const float rb = scale / sqrtf(block_sum(sb, red) / (float)n + eps);
	for (int i = threadIdx.x; i < n; i += SEQ_THREADS)
		a[i] = a[i] * ra * wa[i] + b[i] * rb * wb[i];
}

// C[t][j] *= sigmoid(Z[t][col0 + j]), j < n: an elementwise output gate whose logits are
// columns of the input projection's result.
__global__ __launch_bounds__(SEQ_THREADS) void seq_gate_mul_kernel(float *__restrict__ C, int ldc,
                                                                   const float *__restrict__ Z, int ldz, int col0,
                                                                   int n) {
	const int t = blockIdx.y;
	const int j = blockIdx.x * SEQ_THREADS + threadIdx.x;
	if (j < n)
		C[(size_t)t * ldc + j] *= sq_sigmoid(Z[(size_t)t * ldz + col0 + j]);
}

// ------------------------------------------------------------------ matrix products
enum { EPI_NONE = 0, EPI_GLU_GELU = 1, EPI_GLU_CLAMP = 2, EPI_SIGMOID = 3, EPI_GELU = 4, EPI_GLU_SILU = 5, EPI_RELU2 = 6 };

// C[c_row(m)][n] = epi(sum_k A[a_row(m)][k] W[n][k]) for every batch z = blockIdx.z.
struct GemmArgs {
	const float *A = nullptr;
	int lda = 0;
	long a_bs = 0;  // A offset per batch (elements)
	int a_zdiv = 0; // > 0: the A batch offset is (z / a_zdiv) * a_bs
	const void *W = nullptr, *W2 = nullptr; // W2: the second matrix of a GLU pair (same geometry)
	int ldw = 0;
	long w_bs = 0;
	const int *w_sel = nullptr; // != null: batch z reads matrix w_sel[z]
	float *C = nullptr;
	int ldc = 0;
	long c_bs = 0;
	const float *bias = nullptr;
	long bias_bs = 0;
	int M = 0, N = 0, K = 0;
	const int *rows = nullptr; // != null: row list of batch z at rows + z * rows_bs, its length counts[z]
	long rows_bs = 0;
	const int *counts = nullptr;
	int a_div = 1;   // A row = list entry / a_div
	int c_dense = 0; // 1: C row = m, 0: C row = list entry
	int epi = EPI_NONE;
	float limit = 0.0f;
	// batches z >= z_split (z_split > 0) are a second product over the same A batches:
	// matrices W_b, results C_b, bias bias_b, batch index z - z_split
	int z_split = 0;
	const void *W_b = nullptr;
	float *C_b = nullptr;
	const float *bias_b = nullptr;
};

__device__ __forceinline__ float epi_apply(const GemmArgs &a, float v, float v2, float b) {
	switch (a.epi) {
	case EPI_GLU_GELU: return sq_gelu_tanh(v) * v2;
	case EPI_GLU_CLAMP: {
		const float g = fminf(v, a.limit);
		const float u = fminf(fmaxf(v2, -a.limit), a.limit);
		return g * sq_sigmoid(1.702f * g) * (u + 1.0f);
	}
	case EPI_GLU_SILU: return sq_silu(v) * v2;
	case EPI_SIGMOID: return sq_sigmoid(v + b);
	case EPI_GELU: return sq_gelu_tanh(v + b);
	case EPI_RELU2: {
		const float r = fmaxf(v + b, 0.0f);
		return r * r;
	}
	default: return v + b;
	}
}

struct GemmBatch {
	const float *A;
	const char *W, *W2;
	float *C;
	const float *bias;
	const int *rows;
	int M;
};
template <class WT>
__device__ __forceinline__ GemmBatch gemm_batch(const GemmArgs &a, int z) {
	GemmBatch b;
	const bool second = a.z_split > 0 && z >= a.z_split;
	if (second)
		z -= a.z_split;
	const long za = a.a_zdiv > 0 ? z / a.a_zdiv : z;
	b.A = a.A + za * a.a_bs;
	const long zw = a.w_sel ? a.w_sel[z] : z;
	b.W = (const char *)(second ? a.W_b : a.W) + zw * a.w_bs * WT::BYTES;
	b.W2 = a.W2 ? (const char *)a.W2 + zw * a.w_bs * WT::BYTES : nullptr;
	b.C = (second ? a.C_b : a.C) + (long)z * a.c_bs;
	const float *bias = second ? a.bias_b : a.bias;
	b.bias = bias ? bias + (long)z * a.bias_bs : nullptr;
	b.rows = a.rows ? a.rows + (long)z * a.rows_bs : nullptr;
	b.M = a.counts ? a.counts[z] : a.M;
	return b;
}

// ---- single tokens and short portions: one wave per output column streams its weight
// row(s) once with 16-byte loads and keeps up to GEMV_MAX_M activation rows' sums.
#define GEMV_MAX_M 8
template <class WT, bool GLU>
__global__ __launch_bounds__(SEQ_THREADS) void seq_gemv_kernel(GemmArgs a) {
	const GemmBatch b = gemm_batch<WT>(a, blockIdx.z);
	const int lane = threadIdx.x & 63;
	const int n = blockIdx.x * (SEQ_THREADS / 64) + (threadIdx.x >> 6);
	if (n >= a.N || b.M <= 0)
		return;
	const int M = min(b.M, GEMV_MAX_M);
	const float *ar[GEMV_MAX_M];
	int crow[GEMV_MAX_M];
#pragma unroll
	for (int m = 0; m < GEMV_MAX_M; ++m) {
		const int mm = min(m, M - 1);
		const int s = b.rows ? b.rows[mm] : mm;
		ar[m] = b.A + (size_t)(b.rows ? s / a.a_div : s) * a.lda;
		crow[m] = (b.rows && !a.c_dense) ? s : mm;
	}
	float acc[GEMV_MAX_M] = {}, acc2[GEMV_MAX_M] = {};
	const char *w = b.W + (size_t)n * a.ldw * WT::BYTES;
	const char *w2 = GLU ? b.W2 + (size_t)n * a.ldw * WT::BYTES : nullptr;
	constexpr int E = 8; // elements per lane and pass
	const bool vec = (a.ldw % E == 0) && (((size_t)b.W | (size_t)(GLU ? b.W2 : b.W)) % 16 == 0) && (a.lda % 4 == 0) &&
	                 ((size_t)b.A % 16 == 0);
	int kbeg = lane * E;
	if (M == 1 && vec && a.K % E == 0) {
		// one token, whole aligned rows: four 512-element steps of the weight row (non-temporal:
		// read once per token) and of the activation row in flight before the first FMA
		constexpr int U = 4;
		for (; kbeg + (U - 1) * 64 * E < a.K; kbeg += U * 64 * E) {
			u32x4_t wv[U][WT::BYTES == 2 ? 1 : 2], wv2[U][WT::BYTES == 2 ? 1 : 2];
			float4_t xv[U][2];
#pragma unroll
			for (int u = 0; u < U; ++u) {
				const int k = kbeg + u * 64 * E;
				if constexpr (WT::BYTES == 2) {
					wv[u][0] = load_nt16(w + (size_t)k * 2);
					if constexpr (GLU)
						wv2[u][0] = load_nt16(w2 + (size_t)k * 2);
				} else {
					wv[u][0] = load_nt16(w + (size_t)k * 4);
					wv[u][1] = load_nt16(w + (size_t)k * 4 + 16);
					if constexpr (GLU) {
						wv2[u][0] = load_nt16(w2 + (size_t)k * 4);
						wv2[u][1] = load_nt16(w2 + (size_t)k * 4 + 16);
					}
				}
				xv[u][0] = *(const float4_t *)(ar[0] + k);
				xv[u][1] = *(const float4_t *)(ar[0] + k + 4);
			}
#pragma unroll
			for (int u = 0; u < U; ++u) {
				float wf[E], wf2[E];
				if constexpr (WT::BYTES == 2) {
					WT::unpack(wv[u][0], wf);
					if constexpr (GLU)
						WT::unpack(wv2[u][0], wf2);
				} else {
					WT::unpack(wv[u][0], wf);
					WT::unpack(wv[u][1], wf + 4);
					if constexpr (GLU) {
						WT::unpack(wv2[u][0], wf2);
						WT::unpack(wv2[u][1], wf2 + 4);
					}
				}
#pragma unroll
				for (int e = 0; e < E; ++e) {
					const float x = xv[u][e >> 2][e & 3];
					acc[0] = fmaf(wf[e], x, acc[0]);
					if constexpr (GLU)
						acc2[0] = fmaf(wf2[e], x, acc2[0]);
				}
			}
		}
	}
	for (int k0 = kbeg; k0 < a.K; k0 += 64 * E) {
		float wf[E], wf2[E];
		const bool full = vec && k0 + E <= a.K;
		if (full) {
			if constexpr (WT::BYTES == 2) {
				WT::unpack(load16(w + (size_t)k0 * 2), wf);
				if constexpr (GLU)
					WT::unpack(load16(w2 + (size_t)k0 * 2), wf2);
			} else {
				WT::unpack(load16(w + (size_t)k0 * 4), wf);
				WT::unpack(load16(w + (size_t)k0 * 4 + 16), wf + 4);
				if constexpr (GLU) {
					WT::unpack(load16(w2 + (size_t)k0 * 4), wf2);
					WT::unpack(load16(w2 + (size_t)k0 * 4 + 16), wf2 + 4);
				}
			}
		} else {
#pragma unroll
			for (int e = 0; e < E; ++e) {
				wf[e] = k0 + e < a.K ? wload<WT>(w, k0 + e) : 0.0f;
				if constexpr (GLU)
					wf2[e] = k0 + e < a.K ? wload<WT>(w2, k0 + e) : 0.0f;
			}
		}
#pragma unroll
		for (int m = 0; m < GEMV_MAX_M; ++m) {
			if (m < M) {
				float x[E];
				if (full) {
					const float4_t x0 = *(const float4_t *)(ar[m] + k0), x1 = *(const float4_t *)(ar[m] + k0 + 4);
#pragma unroll
					for (int e = 0; e < 4; ++e) {
						x[e] = x0[e];
						x[4 + e] = x1[e];
					}
				} else {
#pragma unroll
					for (int e = 0; e < E; ++e)
						x[e] = k0 + e < a.K ? ar[m][k0 + e] : 0.0f;
				}
#pragma unroll
				for (int e = 0; e < E; ++e) {
					acc[m] = fmaf(wf[e], x[e], acc[m]);
					if constexpr (GLU)
						acc2[m] = fmaf(wf2[e], x[e], acc2[m]);
				}
			}
		}
	}
#pragma unroll
	for (int m = 0; m < GEMV_MAX_M; ++m) {
		if (m < M) {
			const float v = wave_sum(acc[m]);
			const float v2 = GLU ? wave_sum(acc2[m]) : 0.0f;
			if (lane == 0)
				b.C[(size_t)crow[m] * a.ldc + n] = epi_apply(a, v, v2, b.bias ? b.bias[n] : 0.0f);
		}
	}
}

// ---- one token, the previous sublayer's closing norm folded in: x' = x + norm(y) wb is what
// the product reads when sublayers read the stream itself. Every workgroup rebuilds x' once
// (a thread KI groups of 4 entries, the row's statistics over the workgroup) into LDS, while
// its waves' first weight rows are already in flight; then each wave multiplies RPW weight
// rows: C[n] = epi(W[n] . x' + bias[n]). Workgroup 0 also writes x' to Xout, a second buffer
// (the other workgroups still read X). K % 8 == 0, K <= 1024 KI, rows of W contiguous and
// 16-byte aligned. Dynamic LDS: K floats.
#define GAN_RPW 2
template <class WT, int KI>
__global__ __launch_bounds__(SEQ_THREADS) void seq_gemv_an_kernel(const float *__restrict__ X, const float *__restrict__ Y,
                                                                  const float *__restrict__ wb, float eps, int ln, int K,
                                                                  float *__restrict__ Xout, const void *__restrict__ W,
                                                                  int N, float *__restrict__ C,
                                                                  const float *__restrict__ bias, int epi) {
	extern __shared__ __attribute__((aligned(16))) float xs[];
	__shared__ float red[SEQ_THREADS / 64];
	constexpr int KE = 2 * KI;                 // steps of 512 entries over a weight row
	constexpr int NL = WT::BYTES == 2 ? 1 : 2; // 16-byte loads per 8 weights
	const int tid = threadIdx.x, lane = tid & 63;
	const int n0 = (blockIdx.x * (SEQ_THREADS / 64) + (tid >> 6)) * GAN_RPW;
	u32x4_t wv[KE][NL];
	auto fetch = [&](int n) {
		const char *w = (const char *)W + (size_t)n * K * WT::BYTES;
#pragma unroll
		for (int u = 0; u < KE; ++u) {
			const int k = u * 512 + lane * 8;
#pragma unroll
			for (int i = 0; i < NL; ++i)
				wv[u][i] = (n < N && k < K) ? load_nt16(w + (size_t)k * WT::BYTES + 16 * i) : u32x4_t{0, 0, 0, 0};
		}
	};
	fetch(n0);
	float4_t x[KI], y[KI], b[KI];
	float sm = 0.0f;
#pragma unroll
	for (int i = 0; i < KI; ++i) {
		const int k = 4 * (tid + SEQ_THREADS * i);
		const bool in = k < K;
		y[i] = in ? *(const float4_t *)(Y + k) : float4_t{0, 0, 0, 0};
		x[i] = in ? *(const float4_t *)(X + k) : float4_t{0, 0, 0, 0};
		b[i] = in ? *(const float4_t *)(wb + k) : float4_t{0, 0, 0, 0};
		sm += (y[i][0] + y[i][1]) + (y[i][2] + y[i][3]);
	}
	if (ln) { // entries past the row's end stay 0
		const float mu = block_sum(sm, red) / (float)K;
#pragma unroll
		for (int i = 0; i < KI; ++i)
			if (4 * (tid + SEQ_THREADS * i) < K)
#pragma unroll
				for (int e = 0; e < 4; ++e)
					y[i][e] -= mu;
	}
	float ss = 0.0f;
#pragma unroll
	for (int i = 0; i < KI; ++i)
#pragma unroll
		for (int e = 0; e < 4; ++e)
			ss = fmaf(y[i][e], y[i][e], ss);
	const float r = 1.0f / sqrtf(block_sum(ss, red) / (float)K + eps);
#pragma unroll
	for (int i = 0; i < KI; ++i) {
		const int k = 4 * (tid + SEQ_THREADS * i);
		if (k >= K)
			continue;
#pragma unroll
		for (int e = 0; e < 4; ++e)
			x[i][e] = fmaf(y[i][e] * r, b[i][e], x[i][e]);
		*(float4_t *)(xs + k) = x[i];
		if (blockIdx.x == 0)
			*(float4_t *)(Xout + k) = x[i];
	}
	__syncthreads();
#pragma unroll
	for (int j = 0; j < GAN_RPW; ++j) {
		const int n = n0 + j;
		float acc = 0.0f;
#pragma unroll
		for (int u = 0; u < KE; ++u) {
			const int k = u * 512 + lane * 8;
			if (k >= K)
				continue;
			float wf[8];
			if constexpr (WT::BYTES == 2) {
				WT::unpack(wv[u][0], wf);
			} else {
				WT::unpack(wv[u][0], wf);
				WT::unpack(wv[u][NL - 1], wf + 4);
			}
			const float4_t x0 = *(const float4_t *)(xs + k), x1 = *(const float4_t *)(xs + k + 4);
#pragma unroll
			for (int e = 0; e < 4; ++e) {
				acc = fmaf(wf[e], x0[e], acc);
				acc = fmaf(wf[4 + e], x1[e], acc);
			}
		}
		if (j + 1 < GAN_RPW)
			fetch(n + 1); // the next row's loads run under this row's reduction
		acc = wave_sum(acc);
		if (lane == 0 && n < N) {
			const float v = acc + (bias ? bias[n] : 0.0f);
			C[n] = epi == EPI_GELU ? sq_gelu_tanh(v) : v;
		}
	}
}

// ---- portions: 64 x 64 output tiles, K in slabs of 32 through LDS.
#define GT_BM 64
#define GT_BN 64
#define GT_BK 32

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float float16_t __attribute__((ext_vector_type(16)));

// WBF16: activations rounded to bf16 on the way into LDS; each of the 4 waves owns a
// 32 x 32 quadrant as one v_mfma_f32_32x32x16_bf16 accumulator (A operand: lane l holds
// row l & 31, k = 8 (l >> 5) .. + 7; C/D: column = lane & 31, row = (reg & 3) + 8 (reg >> 2)
// + 4 (lane >> 5)). WF32: f32 FMA, each thread a 4 x 4 block.
template <class WT, bool GLU>
__global__ __launch_bounds__(SEQ_THREADS) void seq_gemm_kernel(GemmArgs a) {
	const GemmBatch b = gemm_batch<WT>(a, blockIdx.z);
	const int m0 = blockIdx.y * GT_BM, n0 = blockIdx.x * GT_BN;
	if (m0 >= b.M)
		return;
	const int tid = threadIdx.x;
	__shared__ int arow[GT_BM], crow[GT_BM];
	if (tid < GT_BM) {
		const int m = m0 + tid;
		int ra = -1, rc = -1;
		if (m < b.M) {
			const int s = b.rows ? b.rows[m] : m;
			ra = b.rows ? s / a.a_div : s;
			rc = (b.rows && !a.c_dense) ? s : m;
		}
		arow[tid] = ra;
		crow[tid] = rc;
	}
	__syncthreads();

	if constexpr (WT::BYTES == 2) {
		constexpr int LD = GT_BK + 8; // bf16 elements per LDS row: 80 bytes, 16-byte aligned pieces
		__shared__ __attribute__((aligned(16))) uint16_t As[GT_BM * LD], Bs[GT_BN * LD], Bs2[GLU ? GT_BN * LD : 8];
		const int wave = tid >> 6, lane = tid & 63;
		const int wm = (wave & 1) * 32, wn = (wave >> 1) * 32;
		float16_t acc = {}, acc2 = {};
		const int lr = tid >> 2, lk = (tid & 3) * 8; // loader: row, first k of 8
		const int ra = arow[lr];
		const int nb = n0 + lr;
		const bool avec = a.lda % 4 == 0 && (size_t)b.A % 16 == 0;
		const bool wvec = a.ldw % 8 == 0 && ((size_t)b.W | (size_t)(GLU ? b.W2 : b.W)) % 16 == 0;
		for (int k0 = 0; k0 < a.K; k0 += GT_BK) {
			const int k = k0 + lk;
			u32x4_t pa = {0, 0, 0, 0}, pb = {0, 0, 0, 0}, pb2 = {0, 0, 0, 0};
			if (ra >= 0) {
				const float *src = b.A + (size_t)ra * a.lda + k;
				float x[8];
				if (avec && k + 8 <= a.K) {
					const float4_t x0 = *(const float4_t *)src, x1 = *(const float4_t *)(src + 4);
#pragma unroll
					for (int e = 0; e < 4; ++e) {
						x[e] = x0[e];
						x[4 + e] = x1[e];
					}
				} else {
#pragma unroll
					for (int e = 0; e < 8; ++e)
						x[e] = k + e < a.K ? src[e] : 0.0f;
				}
#pragma unroll
				for (int e = 0; e < 4; ++e)
					pa[e] = (uint32_t)f2bf(x[2 * e]) | ((uint32_t)f2bf(x[2 * e + 1]) << 16);
			}
			if (nb < a.N) {
				const uint16_t *src = (const uint16_t *)b.W + (size_t)nb * a.ldw + k;
				const uint16_t *src2 = GLU ? (const uint16_t *)b.W2 + (size_t)nb * a.ldw + k : nullptr;
				if (wvec && k + 8 <= a.K) {
					pb = load16(src);
					if constexpr (GLU)
						pb2 = load16(src2);
				} else {
#pragma unroll
					for (int e = 0; e < 4; ++e) {
						const uint32_t lo = k + 2 * e < a.K ? src[2 * e] : 0, hi = k + 2 * e + 1 < a.K ? src[2 * e + 1] : 0;
						pb[e] = lo | (hi << 16);
						if constexpr (GLU) {
							const uint32_t lo2 = k + 2 * e < a.K ? src2[2 * e] : 0,
							               hi2 = k + 2 * e + 1 < a.K ? src2[2 * e + 1] : 0;
							pb2[e] = lo2 | (hi2 << 16);
						}
					}
				}
			}
			__syncthreads(); // the previous slab's MFMAs have read LDS
			*(u32x4_t *)(As + lr * LD + lk) = pa;
			*(u32x4_t *)(Bs + lr * LD + lk) = pb;
			if constexpr (GLU)
				*(u32x4_t *)(Bs2 + lr * LD + lk) = pb2;
			__syncthreads();
#pragma unroll
			for (int ks = 0; ks < GT_BK; ks += 16) {
				const int kk = ks + 8 * (lane >> 5);
				const bf16x8_t fa = __builtin_bit_cast(bf16x8_t, *(const u32x4_t *)(As + (wm + (lane & 31)) * LD + kk));
				const bf16x8_t fb = __builtin_bit_cast(bf16x8_t, *(const u32x4_t *)(Bs + (wn + (lane & 31)) * LD + kk));
				acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa, fb, acc, 0, 0, 0);
				if constexpr (GLU) {
					const bf16x8_t fb2 =
					    __builtin_bit_cast(bf16x8_t, *(const u32x4_t *)(Bs2 + (wn + (lane & 31)) * LD + kk));
					acc2 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa, fb2, acc2, 0, 0, 0);
				}
			}
		}
		const int n = n0 + wn + (lane & 31);
		if (n < a.N) {
			const float bias = b.bias ? b.bias[n] : 0.0f;
#pragma unroll
			for (int r = 0; r < 16; ++r) {
				const int ml = wm + (r & 3) + 8 * (r >> 2) + 4 * (lane >> 5);
				const int rc = crow[ml];
				if (rc >= 0)
					b.C[(size_t)rc * a.ldc + n] = epi_apply(a, acc[r], GLU ? acc2[r] : 0.0f, bias);
			}
		}
	} else {
		constexpr int LDF = GT_BM + 4;
		__shared__ float As[GT_BK * LDF], Bs[GT_BK * LDF], Bs2[GLU ? GT_BK * LDF : 4];
		const int tx = tid & 15, ty = tid >> 4;
		float acc[4][4] = {}, acc2[4][4] = {};
		for (int k0 = 0; k0 < a.K; k0 += GT_BK) {
			__syncthreads();
			for (int idx = tid; idx < GT_BM * GT_BK; idx += SEQ_THREADS) {
				const int r = idx / GT_BK, kk = idx % GT_BK;
				const int k = k0 + kk;
				const int ra = arow[r];
				As[kk * LDF + r] = (ra >= 0 && k < a.K) ? b.A[(size_t)ra * a.lda + k] : 0.0f;
				const int nb = n0 + r;
				const bool ok = nb < a.N && k < a.K;
				Bs[kk * LDF + r] = ok ? ((const float *)b.W)[(size_t)nb * a.ldw + k] : 0.0f;
				if constexpr (GLU)
					Bs2[kk * LDF + r] = ok ? ((const float *)b.W2)[(size_t)nb * a.ldw + k] : 0.0f;
			}
			__syncthreads();
#pragma unroll 8
			for (int kk = 0; kk < GT_BK; ++kk) {
				const float4_t av = *(const float4_t *)(As + kk * LDF + ty * 4);
				const float4_t bv = *(const float4_t *)(Bs + kk * LDF + tx * 4);
				float4_t bv2 = {0, 0, 0, 0};
				if constexpr (GLU)
					bv2 = *(const float4_t *)(Bs2 + kk * LDF + tx * 4);
#pragma unroll
				for (int i = 0; i < 4; ++i)
#pragma unroll
					for (int j = 0; j < 4; ++j) {
						acc[i][j] = fmaf(av[i], bv[j], acc[i][j]);
						if constexpr (GLU)
							acc2[i][j] = fmaf(av[i], bv2[j], acc2[i][j]);
					}
			}
		}
#pragma unroll
		for (int i = 0; i < 4; ++i) {
			const int rc = crow[ty * 4 + i];
			if (rc < 0)
				continue;
#pragma unroll
			for (int j = 0; j < 4; ++j) {
				const int n = n0 + tx * 4 + j;
				if (n < a.N)
					b.C[(size_t)rc * a.ldc + n] =
					    epi_apply(a, acc[i][j], GLU ? acc2[i][j] : 0.0f, b.bias ? b.bias[n] : 0.0f);
			}
		}
	}
}

// A [M][lda] f32 -> out [M][K] bf16 (round to nearest even): the A operand of the large-tile
// GEMM (prefill_gemm.h), which takes 16-bit activations. K % 8 == 0.
__global__ __launch_bounds__(SEQ_THREADS) void seq_to_bf16_kernel(const float *__restrict__ A, int lda, int M, int K,
                                                                  uint16_t *__restrict__ out) {
	const int k8 = K >> 3;
	const size_t n = (size_t)M * k8;
	for (size_t i = (size_t)blockIdx.x * SEQ_THREADS + threadIdx.x; i < n; i += (size_t)gridDim.x * SEQ_THREADS) {
		const int m = (int)(i / k8), k = (int)(i % k8) * 8;
		const float *src = A + (size_t)m * lda + k;
		u32x4_t w;
#pragma unroll
		for (int e = 0; e < 4; ++e)
			w[e] = (uint32_t)f2bf(src[2 * e]) | ((uint32_t)f2bf(src[2 * e + 1]) << 16);
		*(u32x4_t *)(out + (size_t)m * K + k) = w;
	}
}

// ---- long portions, bf16: 128 x 128 output tiles, 4 waves of 64 x 64 (2 x 2 MFMA tiles of
// 32 x 32), K in slabs of 32 through two LDS buffers: the next slab's global loads (and the
// activations' f32 -> bf16 rounding) are issued before the current slab's 8 MFMAs per wave
// and stored to the other buffer after them, one barrier per slab.
#define GB_BM 128
#define GB_BN 128
template <bool GLU>
__global__ __launch_bounds__(SEQ_THREADS) void seq_gemm_bf16_kernel(GemmArgs a) {
	const GemmBatch b = gemm_batch<WBF16>(a, blockIdx.z);
	const int m0 = blockIdx.y * GB_BM, n0 = blockIdx.x * GB_BN;
	if (m0 >= b.M)
		return;
	constexpr int LD = GT_BK + 8;
	__shared__ int arow[GB_BM], crow[GB_BM];
	__shared__ __attribute__((aligned(16))) uint16_t As[2][GB_BM * LD], Bs[2][GB_BN * LD],
	    Bs2[GLU ? 2 : 1][GLU ? GB_BN * LD : 8];
	const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
	if (tid < GB_BM) {
		const int m = m0 + tid;
		int ra = -1, rc = -1;
		if (m < b.M) {
			const int s = b.rows ? b.rows[m] : m;
			ra = b.rows ? s / a.a_div : s;
			rc = (b.rows && !a.c_dense) ? s : m;
		}
		arow[tid] = ra;
		crow[tid] = rc;
	}
	__syncthreads();
	const int wm = (wave & 1) * 64, wn = (wave >> 1) * 64;
	const int lr = tid >> 2, lk = (tid & 3) * 8; // loader: rows lr and lr + 64, first k of 8
	const int ra0 = arow[lr], ra1 = arow[lr + 64];
	const bool avec = a.lda % 4 == 0 && (size_t)b.A % 16 == 0;
	const bool wvec = a.ldw % 8 == 0 && ((size_t)b.W | (size_t)(GLU ? b.W2 : b.W)) % 16 == 0;
	u32x4_t pa[2], pb[2], pb2[2];
	auto fetch = [&](int k0) {
		const int k = k0 + lk;
#pragma unroll
		for (int h = 0; h < 2; ++h) {
			const int ra = h ? ra1 : ra0;
			pa[h] = u32x4_t{0, 0, 0, 0};
			if (ra >= 0) {
				const float *src = b.A + (size_t)ra * a.lda + k;
				float x[8];
				if (avec && k + 8 <= a.K) {
					const float4_t x0 = *(const float4_t *)src, x1 = *(const float4_t *)(src + 4);
#pragma unroll
					for (int e = 0; e < 4; ++e) {
						x[e] = x0[e];
						x[4 + e] = x1[e];
					}
				} else {
#pragma unroll
					for (int e = 0; e < 8; ++e)
						x[e] = k + e < a.K ? src[e] : 0.0f;
				}
#pragma unroll
				for (int e = 0; e < 4; ++e)
					pa[h][e] = (uint32_t)f2bf(x[2 * e]) | ((uint32_t)f2bf(x[2 * e + 1]) << 16);
			}
			const int nb = n0 + lr + 64 * h;
			pb[h] = u32x4_t{0, 0, 0, 0};
			pb2[h] = u32x4_t{0, 0, 0, 0};
			if (nb < a.N) {
				const uint16_t *src = (const uint16_t *)b.W + (size_t)nb * a.ldw + k;
				const uint16_t *src2 = GLU ? (const uint16_t *)b.W2 + (size_t)nb * a.ldw + k : nullptr;
				if (wvec && k + 8 <= a.K) {
					pb[h] = load16(src);
					if constexpr (GLU)
						pb2[h] = load16(src2);
				} else {
#pragma unroll
					for (int e = 0; e < 4; ++e) {
						const uint32_t lo = k + 2 * e < a.K ? src[2 * e] : 0, hi = k + 2 * e + 1 < a.K ? src[2 * e + 1] : 0;
						pb[h][e] = lo | (hi << 16);
						if constexpr (GLU) {
							const uint32_t lo2 = k + 2 * e < a.K ? src2[2 * e] : 0,
							               hi2 = k + 2 * e + 1 < a.K ? src2[2 * e + 1] : 0;
							pb2[h][e] = lo2 | (hi2 << 16);
						}
					}
				}
			}
		}
	};
	auto stash = [&](int buf) {
#pragma unroll
		for (int h = 0; h < 2; ++h) {
			*(u32x4_t *)(As[buf] + (lr + 64 * h) * LD + lk) = pa[h];
			*(u32x4_t *)(Bs[buf] + (lr + 64 * h) * LD + lk) = pb[h];
			if constexpr (GLU)
				*(u32x4_t *)(Bs2[buf] + (lr + 64 * h) * LD + lk) = pb2[h];
		}
	};
	float16_t acc[2][2] = {}, acc2[GLU ? 2 : 1][GLU ? 2 : 1] = {};
	fetch(0);
	stash(0);
	__syncthreads();
	int buf = 0;
	for (int k0 = 0; k0 < a.K; k0 += GT_BK) {
		const bool more = k0 + GT_BK < a.K;
		if (more)
			fetch(k0 + GT_BK);
#pragma unroll
		for (int ks = 0; ks < GT_BK; ks += 16) {
			const int kk = ks + 8 * (lane >> 5);
			bf16x8_t fa[2], fb[2], fb2[2];
#pragma unroll
			for (int i = 0; i < 2; ++i) {
				fa[i] = __builtin_bit_cast(bf16x8_t, *(const u32x4_t *)(As[buf] + (wm + 32 * i + (lane & 31)) * LD + kk));
				fb[i] = __builtin_bit_cast(bf16x8_t, *(const u32x4_t *)(Bs[buf] + (wn + 32 * i + (lane & 31)) * LD + kk));
				if constexpr (GLU)
					fb2[i] = __builtin_bit_cast(bf16x8_t,
					                            *(const u32x4_t *)(Bs2[buf] + (wn + 32 * i + (lane & 31)) * LD + kk));
			}
#pragma unroll
			for (int i = 0; i < 2; ++i)
#pragma unroll
				for (int j = 0; j < 2; ++j) {
					acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[i], fb[j], acc[i][j], 0, 0, 0);
					if constexpr (GLU)
						acc2[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[i], fb2[j], acc2[i][j], 0, 0, 0);
				}
		}
		if (more)
			stash(buf ^ 1); // the other buffer: its last readers passed the previous barrier
		__syncthreads();
		buf ^= 1;
	}
#pragma unroll
	for (int j = 0; j < 2; ++j) {
		const int n = n0 + wn + 32 * j + (lane & 31);
		if (n >= a.N)
			continue;
		const float bias = b.bias ? b.bias[n] : 0.0f;
#pragma unroll
		for (int i = 0; i < 2; ++i)
#pragma unroll
			for (int r = 0; r < 16; ++r) {
				const int ml = wm + 32 * i + (r & 3) + 8 * (r >> 2) + 4 * (lane >> 5);
				const int rc = crow[ml];
				if (rc >= 0)
					b.C[(size_t)rc * a.ldc + n] = epi_apply(a, acc[i][j][r], GLU ? acc2[i][j][r] : 0.0f, bias);
			}
	}
}

// ------------------------------------------------------------------ short causal convolution
#define SEQ_MAX_TAPS 16
// out[t][c] = act(bias[c] + sum_j w[c][j] in(t - (taps - 1) + j)), in(tau) = Z[tau][col0 + c] for
// tau >= 0, else the sequence's stored last inputs state[(taps - 1) + tau][c] (zeros at the start).
__global__ __launch_bounds__(SEQ_THREADS) void seq_conv_kernel(const float *__restrict__ Z, int ldz, int col0, int C,
                                                               int taps, const float *__restrict__ w,
                                                               const float *__restrict__ bias, int silu,
                                                               const float *__restrict__ state,
                                                               float *__restrict__ out, int ldo, int T) {
	const int c = blockIdx.x * SEQ_THREADS + threadIdx.x;
	const int t = blockIdx.y;
	if (c >= C)
		return;
	float acc = bias ? bias[c] : 0.0f;
	for (int j = 0; j < taps; ++j) {
		const int tau = t - (taps - 1) + j;
		const float v = tau >= 0 ? Z[(size_t)tau * ldz + col0 + c] : state[(size_t)(taps - 1 + tau) * C + c];
		acc = fmaf(w[(size_t)c * taps + j], v, acc);
	}
	out[(size_t)t * ldo + c] = silu ? sq_silu(acc) : acc;
}
// Short portions (T <= SEQ_CONV_STEP_T): convolution and state shift in one launch, a thread
// per channel walking the tokens with the last taps - 1 inputs in registers.
#define SEQ_CONV_STEP_T 8
__global__ __launch_bounds__(SEQ_THREADS) void seq_conv_step_kernel(const float *__restrict__ Z, int ldz, int col0, int C,
                                                                    int taps, const float *__restrict__ w,
                                                                    const float *__restrict__ bias, int silu,
                                                                    float *__restrict__ state, float *__restrict__ out,
                                                                    int ldo, int T) {
	const int c = blockIdx.x * SEQ_THREADS + threadIdx.x;
	if (c >= C)
		return;
	float win[SEQ_MAX_TAPS], wv[SEQ_MAX_TAPS]; // win[j]: input at (current token) - (taps - 1) + j
#pragma unroll
	for (int j = 0; j < SEQ_MAX_TAPS; ++j) {
		win[j] = (j < taps - 1) ? state[(size_t)j * C + c] : 0.0f;
		wv[j] = j < taps ? w[(size_t)c * taps + j] : 0.0f;
	}
	const float b = bias ? bias[c] : 0.0f;
	for (int t = 0; t < T; ++t) {
		const float cur = Z[(size_t)t * ldz + col0 + c];
		float acc = b;
#pragma unroll
		for (int j = 0; j < SEQ_MAX_TAPS; ++j) {
			if (j < taps) {
				const float v = (j == taps - 1) ? cur : win[j];
				acc = fmaf(wv[j], v, acc);
			}
		}
		out[(size_t)t * ldo + c] = silu ? sq_silu(acc) : acc;
#pragma unroll
		for (int j = 0; j < SEQ_MAX_TAPS - 1; ++j) // shift the window by one token
			if (j < taps - 1)
				win[j] = (j + 1 < taps - 1) ? win[j + 1] : cur;
	}
#pragma unroll
	for (int j = 0; j < SEQ_MAX_TAPS; ++j)
		if (j < taps - 1)
			state[(size_t)j * C + c] = win[j];
}
// The stored inputs after a portion of T tokens: the last taps - 1 of (old state ++ Z rows).
__global__ __launch_bounds__(SEQ_THREADS) void seq_conv_state_kernel(const float *__restrict__ Z, int ldz, int col0,
                                                                     int C, int taps, float *__restrict__ state,
                                                                     int T) {
	const int c = blockIdx.x * SEQ_THREADS + threadIdx.x;
	if (c >= C)
		return;
	float keep[SEQ_MAX_TAPS];
#pragma unroll
	for (int i = 0; i < SEQ_MAX_TAPS; ++i) {
		if (i < taps - 1) {
			const int tau = T - (taps - 1) + i;
			keep[i] = tau >= 0 ? Z[(size_t)tau * ldz + col0 + c] : state[(size_t)(taps - 1 + tau) * C + c];
		}
	}
#pragma unroll
	for (int i = 0; i < SEQ_MAX_TAPS; ++i)
		if (i < taps - 1)
			state[(size_t)i * C + c] = keep[i];
}

// ------------------------------------------------------------------ real-gated linear recurrence
// Per channel, over the portion's tokens in order: log a = -8 r softplus(lam), a = exp(log a),
// S = a S + sqrt(1 - a^2) (i u); out = S * gelu_tanh(gate branch). 1 - a^2 is taken as
// -expm1(2 log a), which keeps its relative precision when a is close to 1.
__global__ __launch_bounds__(SEQ_THREADS) void seq_rglru_scan_kernel(const float *__restrict__ R,
                                                                     const float *__restrict__ I,
                                                                     const float *__restrict__ U, int W,
                                                                     const float *__restrict__ Z, int ldz,
                                                                     const float *__restrict__ lam,
                                                                     float *__restrict__ state, float *__restrict__ out,
                                                                     int T) {
	const int c = blockIdx.x * SEQ_THREADS + threadIdx.x;
	if (c >= W)
		return;
	const float sp = sq_softplus(lam[c]);
	float S = state[c];
#pragma unroll 4
	for (int t = 0; t < T; ++t) {
		const size_t o = (size_t)t * W + c;
		const float la = -8.0f * R[o] * sp;
		const float aa = expf(la);
		const float mult = sqrtf(-expm1f(2.0f * la));
		S = fmaf(aa, S, mult * (I[o] * U[o]));
		out[o] = S * sq_gelu_tanh(Z[(size_t)t * ldz + c]);
	}
	state[c] = S;
}

// Long portions: everything that does not depend on the carried state is evaluated for all
// tokens at once (R <- a, I <- sqrt(1 - a^2) i u, U <- gelu_tanh(gate branch)), so that the
// sequential walk below is one fused multiply-add per token and channel.
__global__ __launch_bounds__(SEQ_THREADS) void seq_rglru_coef_kernel(float *__restrict__ R, float *__restrict__ I,
                                                                     float *__restrict__ U, int W,
                                                                     const float *__restrict__ Z, int ldz,
                                                                     const float *__restrict__ lam, int T) {
	const int c = blockIdx.x * SEQ_THREADS + threadIdx.x;
	const int t = blockIdx.y;
	if (c >= W)
		return;
	const size_t o = (size_t)t * W + c;
	const float la = -8.0f * R[o] * sq_softplus(lam[c]);
	R[o] = expf(la);
	I[o] = sqrtf(-expm1f(2.0f * la)) * (I[o] * U[o]);
	U[o] = sq_gelu_tanh(Z[(size_t)t * ldz + c]);
}
__global__ __launch_bounds__(SEQ_THREADS) void seq_rglru_walk_kernel(const float *__restrict__ A,
                                                                     const float *__restrict__ B,
                                                                     const float *__restrict__ G, int W,
                                                                     float *__restrict__ state, float *__restrict__ out,
                                                                     int T) {
	const int c = blockIdx.x * SEQ_THREADS + threadIdx.x;
	if (c >= W)
		return;
	float S = state[c];
#pragma unroll 8
	for (int t = 0; t < T; ++t) {
		const size_t o = (size_t)t * W + c;
		S = fmaf(A[o], S, B[o]);
		out[o] = S * G[o];
	}
	state[c] = S;
}

// ------------------------------------------------------------------ gated delta rule
// After the convolutions: q and k to unit length per head (q also x dim^-1/2), beta =
// sigmoid, decay g = exp(-exp(a_log) softplus(a + dt_bias)). QKV: [T][ldq] = q | k | v
// (convolved, silu); Z columns bcol.. = beta logits, acol.. = decay inputs. BG [T][2 H]: beta,
// per-head decay. GV != nullptr: one decay per head and key channel instead, GV [T][H D] holds
// the decay inputs on entry (no bias yet; dt_bias is [H D]) and the decays on return, and the
// per-head decay of BG is 1. One workgroup per token.
__global__ __launch_bounds__(SEQ_THREADS) void seq_delta_prep_kernel(float *__restrict__ QKV, int ldq, int KH, int D,
                                                                     const float *__restrict__ Z, int ldz, int bcol,
                                                                     int acol, int H, const float *__restrict__ a_log,
                                                                     const float *__restrict__ dt_bias,
                                                                     float *__restrict__ BG,
                                                                     float *__restrict__ GV = nullptr) {
	const int t = blockIdx.x;
	const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
	float *row = QKV + (size_t)t * ldq;
	const float qs = 1.0f / sqrtf((float)D);
	for (int seg = wave; seg < 2 * KH; seg += SEQ_THREADS / 64) {
		float *x = row + (size_t)seg * D;
		float ss = 0.0f;
		for (int i = lane; i < D; i += 64)
			ss = fmaf(x[i], x[i], ss);
		ss = wave_sum(ss);
		const float r = (1.0f / sqrtf(ss + 1e-6f)) * (seg < KH ? qs : 1.0f);
		for (int i = lane; i < D; i += 64)
			x[i] *= r;
	}
	for (int h = threadIdx.x; h < H; h += SEQ_THREADS) {
		BG[(size_t)t * 2 * H + h] = sq_sigmoid(Z[(size_t)t * ldz + bcol + h]);
		BG[(size_t)t * 2 * H + H + h] =
		    GV ? 1.0f : expf(-expf(a_log[h]) * sq_softplus(Z[(size_t)t * ldz + acol + h] + dt_bias[h]));
	}
	if (GV)
		for (int i = threadIdx.x; i < H * D; i += SEQ_THREADS) {
			float *g = GV + (size_t)t * H * D + i;
			*g = expf(-expf(a_log[i / D]) * sq_softplus(*g + dt_bias[i]));
		}
}

// Selective state-space layer: per token and head dt = softplus(step + dt_bias[h]) and the
// state's decay exp(-exp(a_log[h]) dt) into BG [T][2 H] (dt, decay), the layout the recurrence
// kernel reads its per-head factors from. Z columns scol.. = the step inputs.
__global__ __launch_bounds__(SEQ_THREADS) void seq_ssm_prep_kernel(const float *__restrict__ Z, int ldz, int scol, int H,
                                                                   const float *__restrict__ a_log,
                                                                   const float *__restrict__ dt_bias,
                                                                   float *__restrict__ BG, int T) {
	const int i = blockIdx.x * SEQ_THREADS + threadIdx.x;
	if (i >= T * H)
		return;
	const int t = i / H, h = i - t * H;
	const float dt = sq_softplus(Z[(size_t)t * ldz + scol + h] + dt_bias[h]);
	BG[(size_t)t * 2 * H + h] = dt;
	BG[(size_t)t * 2 * H + H + h] = expf(-expf(a_log[h]) * dt);
}

__device__ __forceinline__ float sum8(float v) { // over aligned groups of 8 lanes
	v += dpp<0xB1>(v);
	v += dpp<0x4E>(v);
	v += dpp<0x141>(v);
	return v;
}
template <int LPC>
__device__ __forceinline__ float sum_lanes(float v) { // over aligned groups of LPC = 8 or 16 lanes
	v = sum8(v);
	if constexpr (LPC == 16)
		v += dpp<0x140>(v);
	return v;
}

// The recurrence itself. The columns of a head's [dim][vdim] state never mix, so one group
// of LPC (8 or 16) lanes owns one column (each lane a contiguous slice of R dim entries, in
// registers; LPC R >= dim) and walks the portion's tokens in order:
//   S *= g;  u = beta (v - S.k);  S += k u;  o = S.q
// (the read-out after the write). The workgroup's 256 / LPC columns share the head's k and q:
// chunks of TC tokens are staged through two LDS buffers, the next chunk's global loads in
// flight while the current chunk is applied. grid (ceil(vdim LPC / 256), heads). 16 lanes per
// column halve every lane's rows (a shorter dependent chain and half the LDS reads per token)
// and double the workgroups of a walk that fills a fraction of the chip.
// SSM: the state-space form of the same walk, S *= g; S += k (beta v); o = S.q + dskip[h] v
// (no prediction S.k is taken off the write; k, q, v, beta are the layer's B, C, x and dt).
// GVEC: g is a vector over the key channels, GV [T][H D], instead of one number per head.
// QKV [T][ldq]: key/query head kh's q at column qo + kh D, its k at ko + kh D, head h's v at vo + h V.
template <int R, int TC, bool SSM, bool GVEC, int LPC>
__global__ __launch_bounds__(SEQ_THREADS) void seq_delta_kernel(const float *__restrict__ QKV, int ldq, int qo_, int ko_,
                                                                int vo_, int KH, int D, int H, int V,
                                                                const float *__restrict__ BG,
                                                                const float *__restrict__ GV,
                                                                const float *__restrict__ dskip,
                                                                float *__restrict__ state, float *__restrict__ O,
                                                                int T) {
	constexpr int DP = LPC * R;                    // padded key dimension
	constexpr int NS = GVEC ? 3 : 2;               // staged rows per token: k | q (| g)
	constexpr int NKQ = TC * NS * DP / SEQ_THREADS; // staged values per thread and chunk
	constexpr int COLS = SEQ_THREADS / LPC, NV = (TC * COLS + SEQ_THREADS - 1) / SEQ_THREADS;
	static_assert((LPC == 8 || LPC == 16) && (TC * NS * DP) % SEQ_THREADS == 0, "staging assumes whole passes of the workgroup");
	__shared__ __attribute__((aligned(16))) float kq[2][TC][NS * DP];
	__shared__ float vs[2][TC][COLS], bgs[2][TC][2];
	const int tid = threadIdx.x;
	const int h = blockIdx.y, kh = h / (H / KH);
	const int c0 = blockIdx.x * COLS, col = c0 + tid / LPC, sub = tid % LPC;
	const bool live = col < V;
	const int d0 = sub * R; // this lane's slice of the key dimension: d0 .. d0 + R - 1
	float S[R];
	float *sp = state + (size_t)h * D * V;
#pragma unroll
	for (int i = 0; i < R; ++i)
		S[i] = (live && d0 + i < D) ? sp[(size_t)(d0 + i) * V + col] : 0.0f;
	const int qo = qo_ + kh * D, ko = ko_ + kh * D, vo = vo_ + h * V;
	const float dsk = (SSM && dskip) ? dskip[h] : 0.0f;
	// a chunk of TC tokens: global -> registers (in flight while the previous chunk is applied) -> LDS
	float rkq[NKQ], rv[NV], rbg = 0.0f;
	auto fetch = [&](int t0) {
#pragma unroll
		for (int i = 0; i < NKQ; ++i) {
			const int idx = tid + i * SEQ_THREADS;
			const int tt = idx / (NS * DP), e = idx % (NS * DP), d = e % DP, part = e / DP;
			const int t = t0 + tt;
			float x = 0.0f;
			if (t < T && d < D) {
				if (GVEC && part == 2)
					x = GV[((size_t)t * H + h) * D + d];
				else
					x = QKV[(size_t)t * ldq + (part == 0 ? ko : qo) + d];
			}
			rkq[i] = x;
		}
#pragma unroll
		for (int i = 0; i < NV; ++i) {
			const int idx = tid + i * SEQ_THREADS;
			const int tt = idx / COLS, cc = idx % COLS, t = t0 + tt;
			rv[i] = (tt < TC && t < T && c0 + cc < V) ? QKV[(size_t)t * ldq + vo + c0 + cc] : 0.0f;
		}
		if (tid < 2 * TC) {
			const int t = t0 + (tid >> 1);
			rbg = t < T ? BG[(size_t)t * 2 * H + (tid & 1) * H + h] : 0.0f;
		}
	};
	auto stash = [&](int buf) {
#pragma unroll
		for (int i = 0; i < NKQ; ++i) {
			const int idx = tid + i * SEQ_THREADS;
			kq[buf][idx / (NS * DP)][idx % (NS * DP)] = rkq[i];
		}
#pragma unroll
		for (int i = 0; i < NV; ++i) {
			const int idx = tid + i * SEQ_THREADS;
			if (idx < TC * COLS)
				vs[buf][idx / COLS][idx % COLS] = rv[i];
		}
		if (tid < 2 * TC)
			bgs[buf][tid >> 1][tid & 1] = rbg;
	};
	fetch(0);
	stash(0);
	__syncthreads();
	int buf = 0;
	for (int t0 = 0; t0 < T; t0 += TC) {
		const bool more = t0 + TC < T;
		if (more)
			fetch(t0 + TC);
		const int nt = min(TC, T - t0);
		// One token's operands out of LDS, one token ahead of the arithmetic (two register sets in
		// turn), so that the LDS round trip runs under the previous token's dependent chain.
		struct Tok {
			float k[R], q[R], gv[GVEC ? R : 1];
			float v, beta, g;
		};
		auto load = [&](int tt, Tok &x) {
			if constexpr (R % 4 == 0) {
#pragma unroll
				for (int i = 0; i < R / 4; ++i) {
					const float4_t k4 = *(const float4_t *)&kq[buf][tt][d0 + 4 * i];
					const float4_t q4 = *(const float4_t *)&kq[buf][tt][DP + d0 + 4 * i];
#pragma unroll
					for (int e = 0; e < 4; ++e) {
						x.k[4 * i + e] = k4[e];
						x.q[4 * i + e] = q4[e];
					}
					if constexpr (GVEC) {
						const float4_t g4 = *(const float4_t *)&kq[buf][tt][2 * DP + d0 + 4 * i];
#pragma unroll
						for (int e = 0; e < 4; ++e)
							x.gv[4 * i + e] = g4[e];
					}
				}
			} else {
#pragma unroll
				for (int i = 0; i < R; ++i) {
					x.k[i] = kq[buf][tt][d0 + i];
					x.q[i] = kq[buf][tt][DP + d0 + i];
					if constexpr (GVEC)
						x.gv[i] = kq[buf][tt][2 * DP + d0 + i];
				}
			}
			x.v = vs[buf][tt][tid / LPC];
			x.beta = bgs[buf][tt][0];
			x.g = bgs[buf][tt][1];
		};
		auto apply = [&](int tt, const Tok &x) {
			float dd0 = 0.0f, dd1 = 0.0f;
#pragma unroll
			for (int i = 0; i < R; ++i) {
				if constexpr (GVEC)
					S[i] *= x.gv[i];
				else
					S[i] *= x.g;
				if constexpr (!SSM) {
					if (i & 1)
						dd1 = fmaf(S[i], x.k[i], dd1);
					else
						dd0 = fmaf(S[i], x.k[i], dd0);
				}
			}
			float u;
			if constexpr (SSM)
				u = x.beta * x.v;
			else
				u = x.beta * (x.v - sum_lanes<LPC>(dd0 + dd1));
			float o0 = 0.0f, o1 = 0.0f;
#pragma unroll
			for (int i = 0; i < R; ++i) {
				S[i] = fmaf(x.k[i], u, S[i]);
				if (i & 1)
					o1 = fmaf(S[i], x.q[i], o1);
				else
					o0 = fmaf(S[i], x.q[i], o0);
			}
			float o = sum_lanes<LPC>(o0 + o1);
			if constexpr (SSM)
				o = fmaf(dsk, x.v, o);
			if (sub == 0 && live)
				O[(size_t)(t0 + tt) * H * V + h * V + col] = o;
		};
		Tok xa, xb;
		load(0, xa);
		for (int tt = 0; tt < nt; tt += 2) {
			if (tt + 1 < nt)
				load(tt + 1, xb);
			apply(tt, xa);
			if (tt + 1 < nt) {
				if (tt + 2 < nt)
					load(tt + 2, xa);
				apply(tt + 1, xb);
			}
		}
		if (more)
			stash(buf ^ 1); // last read while the chunk before this one was applied
		__syncthreads();
		buf ^= 1;
	}
	if (live) {
#pragma unroll
		for (int i = 0; i < R; ++i)
			if (d0 + i < D)
				sp[(size_t)(d0 + i) * V + col] = S[i];
	}
}

// Each head's read-out divided by its root mean square over vdim, times the shared weight,
// times the output gate: silu (sig == 0) or sigmoid (sig != 0) of the gate logits Gl [t][ldg],
// head h's at column gcol + h V (out may alias Gl when both rows have the same layout: every
// entry is read before the same entry is written). One workgroup per token, a wave per head.
__global__ __launch_bounds__(SEQ_THREADS) void seq_delta_out_kernel(const float *__restrict__ O, int H, int V,
                                                                    const float *__restrict__ w, float eps,
                                                                    const float *Gl, int ldg, int gcol,
                                                                    float *out, int sig = 0) {
	const int t = blockIdx.x;
	const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
	for (int h = wave; h < H; h += SEQ_THREADS / 64) {
		const float *o = O + (size_t)t * H * V + (size_t)h * V;
		float ss = 0.0f;
		for (int i = lane; i < V; i += 64)
			ss = fmaf(o[i], o[i], ss);
		ss = wave_sum(ss);
		const float r = 1.0f / sqrtf(ss / (float)V + eps);
		for (int i = lane; i < V; i += 64) {
			const float gl = Gl[(size_t)t * ldg + gcol + h * V + i];
			out[(size_t)t * H * V + (size_t)h * V + i] = o[i] * r * w[i] * (sig ? sq_sigmoid(gl) : sq_silu(gl));
		}
	}
}

// Y[t] silu(Z[t][zcol ..]) rms-normed in `parts` equal parts of n / parts entries, each by its own
// root mean square, times w [n]: out[t]. grid (tokens, parts).
__global__ __launch_bounds__(SEQ_THREADS) void seq_gated_part_norm_kernel(const float *__restrict__ Y, int n, int parts,
                                                                          const float *__restrict__ Z, int ldz, int zcol,
                                                                          const float *__restrict__ w, float eps,
                                                                          float *__restrict__ out) {
	__shared__ float red[SEQ_THREADS / 64];
	const int t = blockIdx.x, pn = n / parts, c0 = blockIdx.y * pn;
	const float *y = Y + (size_t)t * n + c0;
	const float *z = Z + (size_t)t * ldz + zcol + c0;
	float ss = 0.0f;
	for (int i = threadIdx.x; i < pn; i += SEQ_THREADS) {
		const float v = y[i] * sq_silu(z[i]);
		ss = fmaf(v, v, ss);
	}
	const float r = 1.0f / sqrtf(block_sum(ss, red) / (float)pn + eps);
	for (int i = threadIdx.x; i < pn; i += SEQ_THREADS)
		out[(size_t)t * n + c0 + i] = y[i] * sq_silu(z[i]) * r * w[c0 + i];
}

// ------------------------------------------------------------------ latent attention
// Attention over the cached latent itself: with q~ = W_uk[h]^T q (per head, a kv_rank
// vector) the score q . (W_uk[h] c_j) equals q~ . c_j, and sum_j p_j (W_uv[h] c_j) equals
// W_uv[h] (sum_j p_j c_j); so every head of a token reads the same cached rows, as in
// multi-query attention with key = value = c. Rows r = t * H + h of Qa / Ctx; row r sees
// cache rows j <= st->pos + r / H. Scores, softmax (running maximum and sum per row) and the
// weighted sums are f32. A workgroup owns ATT_BR rows and walks the keys in tiles of 64:
// each wave scores 4 rows x 64 keys (a lane per key), then every thread updates NA4 groups
// of 4 latent entries of one row. Dynamic LDS: att_lds_bytes(rank).
#define ATT_BR 16
#define ATT_KT 64
// LDS rows are padded to a multiple of 4 floats (zeros) so that both phases read 16 bytes
// at a time. Key splits (gridDim.y = S > 1, single tokens and short portions): split s walks
// its share of the visible keys and leaves (sums, running maximum, running sum) per row in
// `part` for seq_latent_merge_kernel; S == 1 writes the normalised sums to Ctx.
__host__ __device__ inline int att_rank4(int rank) {
	return (rank + 3) & ~3;
}
template <class CT, int NA4>
__global__ __launch_bounds__(SEQ_THREADS) void seq_latent_attn_kernel(const float *__restrict__ Qa,
                                                                      const CT *__restrict__ cache, int rank, int H,
                                                                      int NR, float scale,
                                                                      const StepState *__restrict__ st,
                                                                      float *__restrict__ Ctx,
                                                                      float *__restrict__ part) {
	extern __shared__ __attribute__((aligned(16))) float lds[];
	const int rank4 = att_rank4(rank), ldc = rank4 + 4, q4n = rank4 >> 2;
	float *qs = lds;                      // [ATT_BR][rank4]
	float *cs = qs + ATT_BR * rank4;      // [ATT_KT][rank4 + 4]
	float *ps = cs + ATT_KT * ldc;        // [ATT_BR][ATT_KT]
	float *alpha = ps + ATT_BR * ATT_KT;  // [ATT_BR]
	float *lsum = alpha + ATT_BR;         // [ATT_BR]
	float *mfin = lsum + ATT_BR;          // [ATT_BR]
	const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
	const int r0 = blockIdx.x * ATT_BR;
	const int S = gridDim.y, split = blockIdx.y;
	const int pos0 = st->pos;
	const int rlast = min(r0 + ATT_BR, NR) - 1;
	const int nkeys = pos0 + rlast / H + 1; // keys visible to the workgroup's last row
	int k_begin = 0, k_end = nkeys;
	if (S > 1) {
		const int chunk = (((nkeys + S - 1) / S) + ATT_KT - 1) & ~(ATT_KT - 1);
		k_begin = split * chunk;
		k_end = min(nkeys, k_begin + chunk);
	}
	for (int i = tid; i < ATT_BR * rank4; i += SEQ_THREADS) {
		const int r = r0 + i / rank4, d = i % rank4;
		qs[i] = (r < NR && d < rank) ? Qa[(size_t)r * rank + d] * scale : 0.0f;
	}
	float4_t acc[NA4];
#pragma unroll
	for (int a = 0; a < NA4; ++a)
		acc[a] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};
	float mrun[4], lrun[4];
	int lim[4];
#pragma unroll
	for (int i = 0; i < 4; ++i) {
		const int r = r0 + wave * 4 + i;
		mrun[i] = -FLT_MAX;
		lrun[i] = 0.0f;
		lim[i] = r < NR ? min(pos0 + r / H, k_end - 1) : -1;
	}
	for (int kt = k_begin; kt < k_end; kt += ATT_KT) {
		__syncthreads(); // the previous tile's sums have read cs / ps
		if (rank % 8 == 0 && (size_t)cache % 16 == 0) { // 8 latent entries per load
			const int v8n = rank >> 3;
			for (int i = tid; i < ATT_KT * v8n; i += SEQ_THREADS) {
				const int jj = i / v8n, d = (i % v8n) * 8, j = kt + jj;
				float4_t lo = {0.0f, 0.0f, 0.0f, 0.0f}, hi = {0.0f, 0.0f, 0.0f, 0.0f};
				if (j < k_end) {
					if constexpr (sizeof(CT) == 2) {
						float f[8];
						WBF16::unpack(load16(cache + (size_t)j * rank + d), f);
						lo = float4_t{f[0], f[1], f[2], f[3]};
						hi = float4_t{f[4], f[5], f[6], f[7]};
					} else {
						lo = *(const float4_t *)(cache + (size_t)j * rank + d);
						hi = *(const float4_t *)(cache + (size_t)j * rank + d + 4);
					}
				}
				*(float4_t *)(cs + jj * ldc + d) = lo;
				*(float4_t *)(cs + jj * ldc + d + 4) = hi;
			}
		} else {
			for (int i = tid; i < ATT_KT * rank4; i += SEQ_THREADS) {
				const int jj = i / rank4, d = i % rank4, j = kt + jj;
				float v = 0.0f;
				if (j < k_end && d < rank) {
					if constexpr (sizeof(CT) == 2)
						v = bf2f(cache[(size_t)j * rank + d]);
					else
						v = cache[(size_t)j * rank + d];
				}
				cs[jj * ldc + d] = v;
			}
		}
		__syncthreads();
		{
			float s[4] = {0.0f, 0.0f, 0.0f, 0.0f};
			const float4_t *cj = (const float4_t *)(cs + lane * ldc);
			const float4_t *q0 = (const float4_t *)(qs + (wave * 4) * rank4);
			for (int d = 0; d < q4n; ++d) {
				const float4_t c = cj[d];
#pragma unroll
				for (int i = 0; i < 4; ++i) {
					const float4_t qv = q0[i * q4n + d];
					s[i] = fmaf(qv[0], c[0], s[i]);
					s[i] = fmaf(qv[1], c[1], s[i]);
					s[i] = fmaf(qv[2], c[2], s[i]);
					s[i] = fmaf(qv[3], c[3], s[i]);
				}
			}
#pragma unroll
			for (int i = 0; i < 4; ++i) {
				const bool vis = kt + lane <= lim[i];
				const float sv = vis ? s[i] : -FLT_MAX;
				const float mx = wave_max(sv);
				const float mnew = fmaxf(mrun[i], mx);
				const float p = vis ? expf(sv - mnew) : 0.0f;
				const float al = expf(mrun[i] - mnew); // 1 while nothing is visible yet, 0 at the first key
				lrun[i] = lrun[i] * al + wave_sum(p);
				mrun[i] = mnew;
				ps[(wave * 4 + i) * ATT_KT + lane] = p;
				if (lane == 0)
					alpha[wave * 4 + i] = al;
			}
		}
		__syncthreads();
#pragma unroll
		for (int a = 0; a < NA4; ++a) {
			const int u = tid + a * SEQ_THREADS;
			if (u < ATT_BR * q4n) {
				const int r = u / q4n, d4 = u % q4n;
				const float al = alpha[r];
				float4_t v = acc[a];
				v[0] *= al;
				v[1] *= al;
				v[2] *= al;
				v[3] *= al;
				const float4_t *pr = (const float4_t *)(ps + r * ATT_KT);
#pragma unroll 4
				for (int j4 = 0; j4 < ATT_KT / 4; ++j4) {
					const float4_t p = pr[j4];
#pragma unroll
					for (int e = 0; e < 4; ++e) {
						const float4_t c = *(const float4_t *)(cs + (4 * j4 + e) * ldc + 4 * d4);
						v[0] = fmaf(p[e], c[0], v[0]);
						v[1] = fmaf(p[e], c[1], v[1]);
						v[2] = fmaf(p[e], c[2], v[2]);
						v[3] = fmaf(p[e], c[3], v[3]);
					}
				}
				acc[a] = v;
			}
		}
	}
	if (lane == 0) {
#pragma unroll
		for (int i = 0; i < 4; ++i) {
			lsum[wave * 4 + i] = lrun[i];
			mfin[wave * 4 + i] = mrun[i];
		}
	}
	__syncthreads();
#pragma unroll
	for (int a = 0; a < NA4; ++a) {
		const int u = tid + a * SEQ_THREADS;
		if (u < ATT_BR * q4n) {
			const int r = u / q4n, d4 = u % q4n;
			if (r0 + r >= NR)
				continue;
			if (S == 1) {
				const float inv = 1.0f / lsum[r];
#pragma unroll
				for (int e = 0; e < 4; ++e)
					if (4 * d4 + e < rank)
						Ctx[(size_t)(r0 + r) * rank + 4 * d4 + e] = acc[a][e] * inv;
			} else {
				float *pp = part + ((size_t)(r0 + r) * S + split) * (rank4 + 4);
				*(float4_t *)(pp + 4 * d4) = acc[a];
				if (d4 == 0) {
					pp[rank4] = mfin[r];
					pp[rank4 + 1] = lsum[r];
				}
			}
		}
	}
}
static inline size_t att_lds_bytes(int rank) {
	const int r4 = att_rank4(rank);
	return sizeof(float) * ((size_t)ATT_BR * r4 + (size_t)ATT_KT * (r4 + 4) + ATT_BR * ATT_KT + 3 * ATT_BR);
}
// Ctx[r] = sum_s e^(m_s - M) acc_s / sum_s e^(m_s - M) l_s over the key splits of row r
// (times gate[r] if given; gate_e: times sigmoid of the row's own gate logits, row r = token
// r / H, head r % H, logits at gate_e[token * ldg + head * rank + d]).
// One workgroup per row: every wave works the splits' weights out for itself (lane s holds
// split s, S <= 64), then the waves share the row's entries.
__global__ __launch_bounds__(SEQ_THREADS) void seq_latent_merge_kernel(const float *__restrict__ part, int S, int rank,
                                                              float *__restrict__ Ctx,
                                                              const float *__restrict__ gate = nullptr,
                                                              const float *__restrict__ gate_e = nullptr, int ldg = 0,
                                                              int H = 1) {
	__shared__ float wsm_all[SEQ_THREADS];
	const int r = blockIdx.x, rank4 = att_rank4(rank), stride = rank4 + 4, lane = threadIdx.x & 63;
	float *wsm = wsm_all + (threadIdx.x & ~63); // this wave's copy
	const float *pp = part + (size_t)r * S * stride;
	const float m = lane < S ? pp[(size_t)lane * stride + rank4] : -FLT_MAX;
	const float l = lane < S ? pp[(size_t)lane * stride + rank4 + 1] : 0.0f;
	const float M = wave_max(m);
	const float w = expf(m - M);
	const float inv = (gate ? gate[r] : 1.0f) / wave_sum(w * l);
	wsm[lane] = w * inv;
	__syncthreads();
	for (int d = threadIdx.x; d < rank; d += SEQ_THREADS) {
		float v = 0.0f;
#pragma unroll 8
		for (int s = 0; s < S; ++s)
			v = fmaf(wsm[s], pp[(size_t)s * stride + d], v);
		if (gate_e)
			v *= sq_sigmoid(gate_e[(size_t)(r / H) * ldg + (size_t)(r % H) * rank + d]);
		Ctx[(size_t)r * rank + d] = v;
	}
}

// ---- portions over a bf16 cache: the same attention on the matrix cores. A workgroup owns
// 64 rows (a wave 16) and walks the keys in tiles of 32; scores and weighted sums are
// v_mfma_f32_16x16x32_bf16 products with f32 accumulation whose f32 operands (q~ * scale, the
// softmax weights) enter as hi + lo bf16 pairs (hi = bf16(x), lo = bf16(x - hi): 16 significant
// bits), the cached latent being bf16 already. Maximum, exponentials, running sums and the
// rescaling of the sums stay f32, in the MFMA's C layout (row = 4 (lane >> 4) + reg, column =
// lane & 15), where a row's 16 columns are the 16 lanes of a DPP row. KS = ceil(rank / 32).
typedef float f32x4a_t __attribute__((ext_vector_type(4)));
#define ATM_BR 64
#define ATM_KT 32
template <int KS>
__global__ __launch_bounds__(SEQ_THREADS) void seq_latent_attn_mfma_kernel(const float *__restrict__ Qa,
                                                                           const uint16_t *__restrict__ cache, int rank,
                                                                           int H, int NR, float scale,
                                                                           const StepState *__restrict__ st,
                                                                           float *__restrict__ Ctx) {
	constexpr int R32 = 32 * KS, NT = 2 * KS; // padded rank, 16-wide output tiles
	constexpr int LDC = R32 + 8, LDT = ATM_KT + 8, LDP = ATM_KT + 8;
	__shared__ __attribute__((aligned(16))) uint16_t Cs[ATM_KT * LDC]; // [key][latent entry]
	__shared__ __attribute__((aligned(16))) uint16_t CsT[R32 * LDT];   // [latent entry][key]
	__shared__ __attribute__((aligned(16))) uint16_t Ps[4][2][16 * LDP]; // per wave: weights hi / lo [row][key]
	const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
	const int lr = lane & 15, lq = lane >> 4;
	const int r0 = blockIdx.x * ATM_BR;
	const int pos0 = st->pos;
	const int rlast = min(r0 + ATM_BR, NR) - 1;
	const int nkeys = pos0 + rlast / H + 1;
	// this lane's A-operand row of q~ (row lr of the wave), as hi / lo fragments per 32-deep step
	bf16x8_t qh[KS], ql[KS];
	{
		const int r = r0 + wave * 16 + lr;
#pragma unroll
		for (int sst = 0; sst < KS; ++sst) {
			u32x4_t hi = {0, 0, 0, 0}, lo = {0, 0, 0, 0};
#pragma unroll
			for (int e = 0; e < 8; ++e) {
				const int d = 32 * sst + 8 * lq + e;
				const float x = (r < NR && d < rank) ? Qa[(size_t)r * rank + d] * scale : 0.0f;
				const uint16_t hb = f2bf(x);
				const uint16_t lb = f2bf(x - bf2f(hb));
				hi[e >> 1] |= (uint32_t)hb << (16 * (e & 1));
				lo[e >> 1] |= (uint32_t)lb << (16 * (e & 1));
			}
			qh[sst] = __builtin_bit_cast(bf16x8_t, hi);
			ql[sst] = __builtin_bit_cast(bf16x8_t, lo);
		}
	}
	int lim[4];
	float mrun[4], lrun[4];
#pragma unroll
	for (int g = 0; g < 4; ++g) {
		const int r = r0 + wave * 16 + 4 * lq + g;
		lim[g] = r < NR ? pos0 + r / H : -1;
		mrun[g] = -FLT_MAX;
		lrun[g] = 0.0f;
	}
	f32x4a_t oacc[NT];
#pragma unroll
	for (int n = 0; n < NT; ++n)
		oacc[n] = f32x4a_t{0.0f, 0.0f, 0.0f, 0.0f};
	const bool cvec = rank % 8 == 0 && (size_t)cache % 16 == 0;
	for (int kt = 0; kt < nkeys; kt += ATM_KT) {
		__syncthreads(); // the previous tile's products have read Cs / CsT / Ps
		for (int v = tid; v < ATM_KT * (R32 / 8); v += SEQ_THREADS) {
			const int jj = v / (R32 / 8), d8 = (v % (R32 / 8)) * 8, j = kt + jj;
			u32x4_t w = {0, 0, 0, 0};
			if (j < nkeys) {
				const uint16_t *src = cache + (size_t)j * rank + d8;
				if (cvec && d8 + 8 <= rank) {
					w = load16(src);
				} else {
#pragma unroll
					for (int e = 0; e < 8; ++e)
						if (d8 + e < rank)
							w[e >> 1] |= (uint32_t)src[e] << (16 * (e & 1));
				}
			}
			*(u32x4_t *)(Cs + jj * LDC + d8) = w;
#pragma unroll
			for (int e = 0; e < 8; ++e)
				CsT[(d8 + e) * LDT + jj] = (uint16_t)(w[e >> 1] >> (16 * (e & 1)));
		}
		__syncthreads();
		f32x4a_t sacc[2] = {f32x4a_t{0.0f, 0.0f, 0.0f, 0.0f}, f32x4a_t{0.0f, 0.0f, 0.0f, 0.0f}};
#pragma unroll
		for (int jt = 0; jt < 2; ++jt)
#pragma unroll
			for (int sst = 0; sst < KS; ++sst) {
				const bf16x8_t kb =
				    __builtin_bit_cast(bf16x8_t, *(const u32x4_t *)(Cs + (16 * jt + lr) * LDC + 32 * sst + 8 * lq));
				sacc[jt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(qh[sst], kb, sacc[jt], 0, 0, 0);
				sacc[jt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ql[sst], kb, sacc[jt], 0, 0, 0);
			}
		float al[4];
#pragma unroll
		for (int g = 0; g < 4; ++g) {
			const bool v0 = kt + lr <= lim[g], v1 = kt + 16 + lr <= lim[g];
			const float s0 = v0 ? sacc[0][g] : -FLT_MAX, s1 = v1 ? sacc[1][g] : -FLT_MAX;
			const float mnew = fmaxf(mrun[g], row16_max(fmaxf(s0, s1)));
			const float p0 = v0 ? expf(s0 - mnew) : 0.0f, p1 = v1 ? expf(s1 - mnew) : 0.0f;
			al[g] = expf(mrun[g] - mnew);
			lrun[g] = lrun[g] * al[g] + row16_sum(p0 + p1);
			mrun[g] = mnew;
			const int row = 4 * lq + g;
			const uint16_t h0 = f2bf(p0), h1 = f2bf(p1);
			Ps[wave][0][row * LDP + lr] = h0;
			Ps[wave][0][row * LDP + 16 + lr] = h1;
			Ps[wave][1][row * LDP + lr] = f2bf(p0 - bf2f(h0));
			Ps[wave][1][row * LDP + 16 + lr] = f2bf(p1 - bf2f(h1));
		}
#pragma unroll
		for (int n = 0; n < NT; ++n)
#pragma unroll
			for (int g = 0; g < 4; ++g)
				oacc[n][g] *= al[g];
		__syncthreads(); // the wave's weights are in LDS
		const bf16x8_t ph = __builtin_bit_cast(bf16x8_t, *(const u32x4_t *)(&Ps[wave][0][lr * LDP + 8 * lq]));
		const bf16x8_t pl = __builtin_bit_cast(bf16x8_t, *(const u32x4_t *)(&Ps[wave][1][lr * LDP + 8 * lq]));
#pragma unroll
		for (int n = 0; n < NT; ++n) {
			const bf16x8_t cb = __builtin_bit_cast(bf16x8_t, *(const u32x4_t *)(CsT + (16 * n + lr) * LDT + 8 * lq));
			oacc[n] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ph, cb, oacc[n], 0, 0, 0);
			oacc[n] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(pl, cb, oacc[n], 0, 0, 0);
		}
	}
#pragma unroll
	for (int g = 0; g < 4; ++g) {
		const int r = r0 + wave * 16 + 4 * lq + g;
		if (r >= NR)
			continue;
		const float inv = 1.0f / lrun[g];
#pragma unroll
		for (int n = 0; n < NT; ++n) {
			const int d = 16 * n + lr;
			if (d < rank)
				Ctx[(size_t)r * rank + d] = oacc[n][g] * inv;
		}
	}
}

// ------------------------------------------------------------------ routed experts
// One workgroup per token: router logits (+ bias) in f32. kind 0: softmax over all experts, a
// group's score = its best expert's, only experts of the `keep` best groups can be chosen, the
// `top` largest scores among them win (ties: the lower index); weight = score * rscale, not
// renormalised. kind 1: the `top` largest logits win (ties: the lower index), weights =
// softmax over the chosen logits only. kind 2: scores sigmoid(logit); the choice ranks score +
// bias: a group by the sum of its two largest, the `top` largest within the `keep` best groups
// win (ties: the lower index); weight = score * rscale, without the bias, not renormalised.
// Also the shared expert's gate sigmoid(w_sg . h). Dynamic LDS: 2 E + G floats.
#define SEQ_MAX_GROUPS 64
__global__ __launch_bounds__(SEQ_THREADS) void seq_router_kernel(const float *__restrict__ Hn, int width,
                                                                 const float *__restrict__ Wr, int E, int top, int G,
                                                                 int keep, float rscale,
                                                                 const float *__restrict__ w_sg, int *__restrict__ idx,
                                                                 float *__restrict__ wt, float *__restrict__ sgate,
                                                                 int kind = 0, const float *__restrict__ bias = nullptr) {
	extern __shared__ float sc[];
	const int t = blockIdx.x;
	const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
	const float *h = Hn + (size_t)t * width;
	for (int e = wave; e < E + (w_sg ? 1 : 0); e += SEQ_THREADS / 64) {
		const float *w = e < E ? Wr + (size_t)e * width : w_sg;
		float a = 0.0f;
		if (width % 4 == 0 && ((size_t)w | (size_t)h) % 16 == 0) {
			float a1 = 0.0f, a2 = 0.0f, a3 = 0.0f;
#pragma unroll 4
			for (int i = lane * 4; i < width; i += 256) {
				const float4_t wv = *(const float4_t *)(w + i), hv = *(const float4_t *)(h + i);
				a = fmaf(wv[0], hv[0], a);
				a1 = fmaf(wv[1], hv[1], a1);
				a2 = fmaf(wv[2], hv[2], a2);
				a3 = fmaf(wv[3], hv[3], a3);
			}
			a = (a + a1) + (a2 + a3);
		} else {
			for (int i = lane; i < width; i += 64)
				a = fmaf(w[i], h[i], a);
		}
		a = wave_sum(a);
		if (lane == 0) {
			if (e < E)
				sc[e] = a + ((bias && kind != 2) ? bias[e] : 0.0f);
			else
				sgate[t] = sq_sigmoid(a);
		}
	}
	__syncthreads();
	if (kind == 1) {
		if (threadIdx.x != 0)
			return;
		float zmax = 0.0f, sum = 0.0f;
		for (int k = 0; k < top; ++k) {
			int best = 0;
			float bv = -INFINITY; // finite logits: a taken expert (-inf) never wins
			for (int e = 0; e < E; ++e)
				if (sc[e] > bv) {
					bv = sc[e];
					best = e;
				}
			if (k == 0)
				zmax = bv;
			const float w = expf(bv - zmax);
			idx[(size_t)t * top + k] = best;
			wt[(size_t)t * top + k] = w;
			sum += w;
			sc[best] = -INFINITY;
		}
		for (int k = 0; k < top; ++k)
			wt[(size_t)t * top + k] /= sum;
		return;
	}
	float *gsc = sc + E; // [G]
	__shared__ float red[SEQ_THREADS / 64];
	if (kind == 2) { // sc holds the logits (no bias added above)
		if (threadIdx.x != 0)
			return;
		const int gs = E / G;
		float *sv = gsc + G; // [E] the scores themselves (the weights); sc becomes the choice scores
		for (int e = 0; e < E; ++e) {
			sv[e] = sq_sigmoid(sc[e]);
			sc[e] = sv[e] + (bias ? bias[e] : 0.0f);
		}
		for (int g = 0; g < G; ++g) { // sum of the group's two largest choice scores
			float m1 = -INFINITY, m2 = -INFINITY;
			for (int e = g * gs; e < (g + 1) * gs; ++e) {
				const float v = sc[e];
				if (v > m1) {
					m2 = m1;
					m1 = v;
				} else if (v > m2) {
					m2 = v;
				}
			}
			gsc[g] = gs > 1 ? m1 + m2 : m1;
		}
		unsigned long long allowed = 0ull;
		for (int k = 0; k < keep; ++k) {
			int best = -1;
			float bv = -INFINITY;
			for (int g = 0; g < G; ++g)
				if (!((allowed >> g) & 1ull) && (best < 0 || gsc[g] > bv)) {
					bv = gsc[g];
					best = g;
				}
			allowed |= 1ull << best;
		}
		for (int k = 0; k < top; ++k) {
			int best = -1;
			float bv = -INFINITY;
			for (int e = 0; e < E; ++e)
				if (((allowed >> (e / gs)) & 1ull) && sc[e] != -INFINITY && (best < 0 || sc[e] > bv)) {
					bv = sc[e];
					best = e;
				}
			idx[(size_t)t * top + k] = best;
			wt[(size_t)t * top + k] = sv[best] * rscale;
			sc[best] = -INFINITY; // taken
		}
		return;
	}
	float mx = -FLT_MAX;
	for (int e = threadIdx.x; e < E; e += SEQ_THREADS)
		mx = fmaxf(mx, sc[e]);
	mx = wave_max(mx);
	if (lane == 0)
		red[wave] = mx;
	__syncthreads();
	mx = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
	float sum = 0.0f;
	for (int e = threadIdx.x; e < E; e += SEQ_THREADS) {
		const float v = expf(sc[e] - mx);
		sc[e] = v;
		sum += v;
	}
	sum = block_sum(sum, red);
	const float inv = 1.0f / sum;
	const int gs = E / G;
	for (int g = threadIdx.x; g < G; g += SEQ_THREADS) {
		float m = -1.0f;
		for (int e = g * gs; e < (g + 1) * gs; ++e)
			m = fmaxf(m, sc[e]);
		gsc[g] = m;
	}
	__syncthreads();
	if (threadIdx.x != 0)
		return;
	unsigned long long allowed = 0ull; // groups that may be chosen from (G <= 64)
	for (int k = 0; k < keep; ++k) {
		int best = -1;
		float bv = -2.0f;
		for (int g = 0; g < G; ++g)
			if (!((allowed >> g) & 1ull) && gsc[g] > bv) {
				bv = gsc[g];
				best = g;
			}
		allowed |= 1ull << best;
	}
	for (int k = 0; k < top; ++k) {
		int best = 0;
		float bv = -1.0f;
		for (int e = 0; e < E; ++e)
			if (((allowed >> (e / gs)) & 1ull) && sc[e] > bv) {
				bv = sc[e];
				best = e;
			}
		idx[(size_t)t * top + k] = best;
		wt[(size_t)t * top + k] = bv * inv * rscale;
		sc[best] = -1.0f; // taken
	}
}

// Slot s = t * top + k goes onto its expert's list (any order: every slot's rows are
// computed independently of their neighbours in the list).
__global__ __launch_bounds__(SEQ_THREADS) void seq_moe_lists_kernel(const int *__restrict__ idx, int n_slots,
                                                                    int *__restrict__ counts, int *__restrict__ lists,
                                                                    int cap) {
	const int s = blockIdx.x * SEQ_THREADS + threadIdx.x;
	if (s >= n_slots)
		return;
	const int e = idx[s];
	const int p = atomicAdd(&counts[e], 1);
	lists[(size_t)e * cap + p] = s;
}
__global__ void seq_fill_int_kernel(int *p, int n, int v) {
	const int i = blockIdx.x * blockDim.x + threadIdx.x;
	if (i < n)
		p[i] = v;
}
__global__ void seq_fill_float_kernel(float *p, size_t n, float v) {
	for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x)
		p[i] = v;
}
