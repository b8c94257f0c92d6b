// seq_attn.h — softmax attention over cached keys and values for the layer-list engine
// (YALM_MIX_ATTN in include/yalm_hip.h): grouped key/value heads, rotary positions on the
// first rot_dims entries of a head (interleaved pairs, rescaled frequencies), query / key /
// value norms, a per-head score temperature, scores mixed across heads, causal / sliding
// window / chunked masks, a softmax with an optional zero-score sink, a per-head output gate.
// Every option is a runtime argument, so another design can combine them differently.
//
// Scores mixed across heads, s'_h = sum_g talk[h][g] (q_g . k_kv(g)), are linear in the queries:
// with q'_h = [sum_{g in c} talk[h][g] q_g for every key/value head c] (H D products per head,
// once per token) they are s'_h = q'_h . (the whole key row of kv_heads x dim entries). The
// mixed queries are built once per token (by the projection kernel for portions, by the
// attention kernel as it loads the queries for a few tokens, whose projection is spread over
// several workgroups), and the attention kernels then see ordinary independent heads whose
// keys are whole cache rows (DK = kv_heads x dim) while head h's values stay those of its own
// key/value head.
//
// Positions and angles, the norms, scores, softmax weights and their weighted sums are f32
// (the angle itself is evaluated and reduced to [-pi, pi] in double: position * frequency
// loses bits in f32 at large positions). The caches hold bf16 (WBF16 models) or f32 (WF32 models).
#pragma once

#include "seq_kernels.h"

struct AttnArgs {
	int H, G, D, V;           // query heads, key/value heads, key size, value size
	int mask_kind, mask_size; // YALM_MASK_*
	int qk_norm, v_norm, sink, out_gate;
	int rot_dims;
	float rot_mag;            // factor on cos and sin
	const double *rot_freq;   // [rot_dims / 2] angle per position
	float scale;              // score = q . k * scale (* temp[h])
	const float *q_w, *k_w;   // YALM_QK_WHOLE: [H D], [G D]
	const float *temp;        // [H] or null
	const float *talk;        // [H][H] or null
	float eps;
	int q_mixed;              // talk: the projection kernel has already written the mixed queries [t][H][G D]
	int KL = 0, VL = 0;       // entries per key / value cache row (head g's keys at column g D, values at g V)
	const float *sink_w = nullptr; // sink: [H] scores of the valueless key, unscaled; null: 0
	// a learned bias per head and distance, added to the scaled score: rel_dist[min(i - j, rel_far)][h]
	// (the bucketed table of the layer expanded per distance at creation), or null
	const float *rel_dist = nullptr;
	int rel_far = 0;
	// q_temp_every > 0: the query at position p times 1 + q_temp_coef ln(floor((p + 1) / q_temp_every) + 1)
	float q_temp_coef = 0.0f;
	int q_temp_every = 0;
};

// The bias of head h's score between a query and a key `dist` positions before it.
__device__ __forceinline__ float attn_rel_bias(const AttnArgs &a, int h, int dist) {
	return a.rel_dist ? a.rel_dist[(size_t)min(max(dist, 0), a.rel_far) * a.H + h] : 0.0f;
}

// The softmax's starting state for head h: with a sink, a valueless key of score sink_w[h] (or 0)
// has already been seen (running maximum = its score, running sum 1).
__device__ __forceinline__ float attn_sink_score(const AttnArgs &a, int h) {
	return a.sink_w ? a.sink_w[h] : 0.0f;
}

// First key position that position p sees.
__host__ __device__ __forceinline__ int attn_first_key(int mask_kind, int mask_size, int p) {
	if (mask_kind == YALM_MASK_WINDOW)
		return p - mask_size + 1 > 0 ? p - mask_size + 1 : 0;
	if (mask_kind == YALM_MASK_CHUNK)
		return (p / mask_size) * mask_size;
	return 0;
}

// Entry d of head h's query as the attention kernels use it: the query itself, or with score
// mixing (talk != null) entry d of the mixed query over the whole key row. Q: the projection
// kernel's output, [t][H][D] queries or (mixed) [t][H][G D] mixed queries.
__device__ __forceinline__ float attn_query(const float *__restrict__ Q, int t, const float *__restrict__ talk,
                                            bool mixed, int H, int G, int D, int h, int d) {
	if (!talk)
		return Q[((size_t)t * H + h) * D + d];
	if (mixed)
		return Q[((size_t)t * H + h) * G * D + d];
	const float *qt = Q + (size_t)t * H * D;
	const int rep = H / G;
	const int c = d / D, dd = d - c * D;
	float m = 0.0f;
	for (int x = 0; x < rep; ++x)
		m = fmaf(talk[h * H + c * rep + x], qt[(c * rep + x) * D + dd], m);
	return m;
}

template <class CT>
__device__ __forceinline__ void cache_store(CT *p, float v) {
	if constexpr (sizeof(CT) == 2)
		*p = f2bf(v);
	else
		*p = v;
}

// ------------------------------------------------------------------ projections -> queries, cache rows, gates
// Token t (blockIdx.x) at position p = st->pos + t; a wave per head job: the H query heads, G
// key heads, G value heads and, with an output gate, H gate heads; the workgroups of a token
// (gridDim.y) take the jobs in turn, so a single decoded token spreads over several workgroups
// while a long portion runs one workgroup per token. Z row: [q: H D | k: G D | v: G V] (biases
// already added). Queries leave scaled by scale * temp[h] in Q [t][H D], or (a.q_mixed, one
// workgroup per token) as the mixed queries [t][H][G D]; keys and values go to the cache rows p. A gate job is a short dot product taken here, from the sublayer's input
// row X[t] and the gate rows Wg [H][width] (stored as CT, the model's matrix type): gate[t][h]
// = sigmoid(Wg[h] . X[t] + gate_bias[h]). Dynamic LDS: rot_dims floats (cos | sin) (+ H D
// floats with a.q_mixed).
template <class CT>
__global__ __launch_bounds__(SEQ_THREADS) void seq_attn_prep_kernel(const float *__restrict__ Z, int ldz, AttnArgs a,
                                                                    const StepState *__restrict__ st,
                                                                    float *__restrict__ Q, CT *__restrict__ Kc,
                                                                    CT *__restrict__ Vc, float *__restrict__ gate,
                                                                    const float *__restrict__ X, int width,
                                                                    const CT *__restrict__ Wg,
                                                                    const float *__restrict__ gate_bias) {
	extern __shared__ float rot[];
	__shared__ float red[SEQ_THREADS / 64];
	constexpr int NW = SEQ_THREADS / 64;
	const int t = blockIdx.x, tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
	const int p = st->pos + t;
	const int half = a.rot_dims >> 1;
	float *qsh = rot + (a.rot_dims > 2 ? a.rot_dims : 2); // a.q_mixed: the token's queries [H][D]
	for (int i = tid; i < half; i += SEQ_THREADS) {
		// position x frequency and its reduction to [-pi, pi] in double, cos / sin of that in f32
		const double two_pi = 6.283185307179586476925286766559;
		const double ang = (double)p * a.rot_freq[i];
		const float red_ang = (float)(ang - two_pi * rint(ang * (1.0 / two_pi)));
		rot[i] = cosf(red_ang) * a.rot_mag;
		rot[half + i] = sinf(red_ang) * a.rot_mag;
	}
	const float *z = Z + (size_t)t * ldz;
	const int QN = a.H * a.D, KN = a.G * a.D, VN = a.G * a.V;
	const bool whole = a.qk_norm == YALM_QK_WHOLE;
	float rq = 1.0f, rk = 1.0f;
	if (whole) {
		float s = 0.0f;
		for (int i = tid; i < QN; i += SEQ_THREADS)
			s = fmaf(z[i], z[i], s);
		rq = 1.0f / sqrtf(block_sum(s, red) / (float)QN + a.eps);
		s = 0.0f;
		for (int i = tid; i < KN; i += SEQ_THREADS)
			s = fmaf(z[QN + i], z[QN + i], s);
		rk = 1.0f / sqrtf(block_sum(s, red) / (float)KN + a.eps);
	}
	__syncthreads();
	const int jobs = a.H + 2 * a.G + (a.out_gate ? a.H : 0);
	for (int job = blockIdx.y * NW + wave; job < jobs; job += gridDim.y * NW) {
		if (job >= a.H + 2 * a.G) { // an output gate
			constexpr int EPL = sizeof(CT) == 2 ? 8 : 4;
			const int h = job - a.H - 2 * a.G;
			const float *x = X + (size_t)t * width;
			const CT *wr = Wg + (size_t)h * width;
			float s = 0.0f;
			if (width % EPL == 0 && (size_t)Wg % 16 == 0 && (size_t)X % 16 == 0) {
				for (int k = lane * EPL; k < width; k += 64 * EPL) {
					float wf[EPL];
					if constexpr (sizeof(CT) == 2)
						WBF16::unpack(load16(wr + k), wf);
					else
						WF32::unpack(load16(wr + k), wf);
#pragma unroll
					for (int e = 0; e < EPL; e += 4) {
						const float4_t xv = *(const float4_t *)(x + k + e);
						s = fmaf(wf[e], xv[0], s);
						s = fmaf(wf[e + 1], xv[1], s);
						s = fmaf(wf[e + 2], xv[2], s);
						s = fmaf(wf[e + 3], xv[3], s);
					}
				}
			} else {
				for (int k = lane; k < width; k += 64) {
					float wv;
					if constexpr (sizeof(CT) == 2)
						wv = bf2f(wr[k]);
					else
						wv = wr[k];
					s = fmaf(wv, x[k], s);
				}
			}
			s = wave_sum(s);
			if (lane == 0)
				gate[(size_t)t * a.H + h] = sq_sigmoid(s + (gate_bias ? gate_bias[h] : 0.0f));
			continue;
		}
		const int kind = job < a.H ? 0 : (job < a.H + a.G ? 1 : 2); // query, key, value head
		const int hh = kind == 0 ? job : (kind == 1 ? job - a.H : job - a.H - a.G);
		const int n = kind == 2 ? a.V : a.D;
		const float *src = z + (kind == 0 ? hh * a.D : (kind == 1 ? QN + hh * a.D : QN + KN + hh * a.V));
		const float *nw = whole && kind < 2 ? (kind == 0 ? a.q_w : a.k_w) + hh * a.D : nullptr;
		const float rw = kind == 0 ? rq : rk;
		float val[4]; // heads of up to 256 entries
		float ss = 0.0f;
#pragma unroll
		for (int e = 0; e < 4; ++e) {
			const int d = lane + 64 * e;
			float v = 0.0f;
			if (d < n) {
				if (kind == 2) {
					v = src[d];
				} else if (d < a.rot_dims) {
					const int d0 = d & ~1, d1 = d | 1;
					float u = src[d0], w = src[d1];
					if (nw) {
						u = u * rw * nw[d0];
						w = w * rw * nw[d1];
					}
					const float c = rot[d >> 1], sn = rot[half + (d >> 1)];
					v = (d & 1) ? w * c + u * sn : u * c - w * sn;
				} else {
					v = src[d];
					if (nw)
						v = v * rw * nw[d];
				}
			}
			val[e] = v;
			ss = fmaf(v, v, ss);
		}
		ss = wave_sum(ss);
		float mul = 1.0f;
		const bool head_w = kind < 2 && a.qk_norm == YALM_QK_HEAD_W;
		if (kind == 2 ? a.v_norm != 0 : (a.qk_norm == YALM_QK_HEAD_UNIT || head_w))
			mul = 1.0f / sqrtf(ss / (float)n + a.eps);
		if (kind == 0) {
			mul *= a.scale * (a.temp ? a.temp[hh] : 1.0f);
			if (a.q_temp_every > 0)
				mul *= 1.0f + a.q_temp_coef * logf((float)((p + 1) / a.q_temp_every) + 1.0f);
		}
		const float *hw = head_w ? (kind == 0 ? a.q_w : a.k_w) : nullptr;
#pragma unroll
		for (int e = 0; e < 4; ++e) {
			const int d = lane + 64 * e;
			if (d >= n)
				continue;
			const float v = val[e] * mul * (hw ? hw[d] : 1.0f);
			if (kind == 0) {
				if (a.q_mixed)
					qsh[hh * a.D + d] = v;
				else
					Q[(size_t)t * QN + hh * a.D + d] = v;
			} else if (kind == 1)
				cache_store<CT>(Kc + (size_t)p * KN + hh * a.D + d, v);
			else
				cache_store<CT>(Vc + (size_t)p * VN + hh * a.V + d, v);
		}
	}
	if (a.q_mixed) { // q'[h][c D + d] = sum_x talk[h][c rep + x] q[c rep + x][d]
		__syncthreads();
		const int rep = a.H / a.G, DK = a.G * a.D;
		float *qo = Q + (size_t)t * a.H * DK;
		for (int cd = tid; cd < DK; cd += SEQ_THREADS) {
			const int c = cd / a.D, d = cd - c * a.D;
			const float *qc = qsh + c * rep * a.D + d;
			for (int h = 0; h < a.H; ++h) {
				const float *tr = a.talk + h * a.H + c * rep;
				float m = 0.0f;
				for (int x = 0; x < rep; ++x)
					m = fmaf(tr[x], qc[x * a.D], m);
				qo[(size_t)h * DK + cd] = m;
			}
		}
	}
}

// ------------------------------------------------------------------ latent attention with a rotated key part
// Token t (blockIdx.x) at position p = st->pos + t. Z row: [q: H heads of (D plain | R rotated)
// | latent: rank | rotated key part: R] (the input projection's result). The latent is rms-
// normed with weight kv_w into columns [0, rank) of cache row p, the key part is rotated into
// columns [rank, rank + R) (not normed); every head's plain query part leaves scaled in
// Qp [t][H][D] (the operand of the per-head product with the transposed key up-projection,
// which fills columns [0, rank) of Qa) and its rotated part, rotated and scaled, in columns
// [rank, rank + R) of Qa [t][H][rank + R]: the attention kernels then see H independent heads
// over ONE key/value head whose key row is the cache row and whose value is its first rank
// entries. Rotation: the first rot_dims <= R entries in interleaved pairs, as in
// seq_attn_prep_kernel. expanded != 0 (the portion attends over expanded per-head keys and
// values, seq_latent_expand_kernel): Qp is not written and Qa is [t][H][D + R], head h's
// scaled plain part followed by its rotated part. The workgroups of a token (gridDim.y) share its
// outputs (each works the rotation table and the latent's rms out for itself). Dynamic LDS:
// max(rot_dims, 2) floats.
template <class CT>
__global__ __launch_bounds__(SEQ_THREADS) void seq_latent_prep_kernel(const float *__restrict__ Z, int ldz, int H, int D,
                                                                      int R, int rank, int rot_dims,
                                                                      const double *__restrict__ rot_freq,
                                                                      const float *__restrict__ kv_w, float eps,
                                                                      float scale, const StepState *__restrict__ st,
                                                                      float *__restrict__ Qp, float *__restrict__ Qa,
                                                                      CT *__restrict__ cache, int expanded) {
	extern __shared__ float rot[];
	__shared__ float red[SEQ_THREADS / 64];
	const int t = blockIdx.x, tid = threadIdx.x;
	const int p = st->pos + t;
	const int half = rot_dims >> 1;
	for (int i = tid; i < half; i += SEQ_THREADS) {
		const double two_pi = 6.283185307179586476925286766559;
		const double ang = (double)p * rot_freq[i];
		const float red_ang = (float)(ang - two_pi * rint(ang * (1.0 / two_pi)));
		rot[i] = cosf(red_ang);
		rot[half + i] = sinf(red_ang);
	}
	const int i0 = blockIdx.y * SEQ_THREADS + tid, istep = gridDim.y * SEQ_THREADS; // this workgroup's share of every loop
	const int QH = D + R, QN = H * QH, KR = rank + R;
	const float *z = Z + (size_t)t * ldz;
	const float *lat = z + QN;
	float ss = 0.0f;
	for (int i = tid; i < rank; i += SEQ_THREADS)
		ss = fmaf(lat[i], lat[i], ss);
	const float r = 1.0f / sqrtf(block_sum(ss, red) / (float)rank + eps); // also orders rot[] before its readers
	CT *crow = cache + (size_t)p * KR;
	for (int i = i0; i < rank; i += istep)
		cache_store<CT>(crow + i, lat[i] * r * kv_w[i]);
	// the rotated parts: job 0 is the shared key part, job 1 + h head h's query part
	for (int i = i0; i < (H + 1) * R; i += istep) {
		const int job = i / R, d = i - job * R;
		const float *src = job == 0 ? lat + rank : z + (size_t)(job - 1) * QH + D;
		float v;
		if (d < rot_dims) {
			const float u = src[d & ~1], w = src[d | 1];
			const float c = rot[d >> 1], sn = rot[half + (d >> 1)];
			v = (d & 1) ? w * c + u * sn : u * c - w * sn;
		} else {
			v = src[d];
		}
		if (job == 0)
			cache_store<CT>(crow + rank + d, v);
		else if (expanded)
			Qa[((size_t)t * H + job - 1) * QH + D + d] = v * scale;
		else
			Qa[((size_t)t * H + job - 1) * KR + rank + d] = v * scale;
	}
	for (int i = i0; i < H * D; i += istep) {
		const int h = i / D, d = i - h * D;
		const float v = z[(size_t)h * QH + d] * scale;
		if (expanded)
			Qa[((size_t)t * H + h) * QH + d] = v;
		else
			Qp[(size_t)t * H * D + i] = v;
	}
}

// out[r][c] = cache[row0 + r][c], c < ncols, as f32: cached latent rows as the A operand of the
// product that expands them.
__global__ __launch_bounds__(SEQ_THREADS) void seq_cache_rows_f32_kernel(const uint16_t *__restrict__ cache, int row_len,
                                                                         int row0, int ncols,
                                                                         float *__restrict__ out) {
	const int r = blockIdx.x;
	const uint16_t *src = cache + (size_t)(row0 + r) * row_len;
	for (int c = threadIdx.x; c < ncols; c += SEQ_THREADS)
		out[(size_t)r * ncols + c] = bf2f(src[c]);
}

// Per-head keys and values of the cached positions row0 .. row0 + gridDim.x - 1, from KV [r][H D
// | H V] (the latent rows times the stacked key and value up-projections) and the cache's
// rotated key part: Kx [r][H][D + R] = [plain key of head h | the shared rotated part], Vx
// [r][H][V], in the cache's type. The softmax-attention kernels then see H key/value heads.
template <class CT>
__global__ __launch_bounds__(SEQ_THREADS) void seq_latent_expand_kernel(const float *__restrict__ KV,
                                                                        const CT *__restrict__ cache, int row0, int H,
                                                                        int D, int R, int V, int rank,
                                                                        CT *__restrict__ Kx, CT *__restrict__ Vx) {
	const int r = blockIdx.x, QH = D + R;
	const float *kv = KV + (size_t)r * H * (D + V);
	const CT *kr = cache + (size_t)(row0 + r) * (rank + R) + rank;
	CT *kx = Kx + (size_t)r * H * QH, *vx = Vx + (size_t)r * H * V;
	for (int i = threadIdx.x; i < H * QH; i += SEQ_THREADS) {
		const int h = i / QH, d = i - h * QH;
		if (d < D)
			cache_store<CT>(kx + i, kv[h * D + d]);
		else
			kx[i] = kr[d - D];
	}
	for (int i = threadIdx.x; i < H * V; i += SEQ_THREADS)
		cache_store<CT>(vx + i, kv[H * D + i]);
}

// ------------------------------------------------------------------ attention, f32 FMA form
// A workgroup owns TQ tokens x the Hb = H / G heads of one key/value head (gridDim.z = G; rows
// r = tq Hb + hl) and walks its share of the keys they see in tiles of SA_KT. Without score
// mixing the keys are that head's columns of the cache rows; with it the (mixed) queries span
// the whole key row, taken in G column chunks of D that accumulate into the same scores. Per
// tile: scores of every row (a lane per key), mask and running softmax per row, then the
// weighted sums of the value tile, each thread NA4 groups of 4 value entries of one row.
// Key splits (gridDim.y = S > 1; single tokens and short portions): split s leaves (sums,
// running maximum, running sum) per row in `part` for seq_latent_merge_kernel; the sink (a key
// of score 0 without a value) is split 0's starting state. S == 1 writes the normalised,
// gated sums to Ctx [t][H V].
#define SA_KT 64
#define SA_MAX_NA4 16

__host__ __device__ inline int sa_ldk(int D, int V) {
	const int d4 = (D + 3) & ~3, v4 = (V + 3) & ~3;
	return (d4 > v4 ? d4 : v4) + 4;
}
// R rows, Gb key column chunks per row
static inline size_t sa_lds_bytes(int R, int Gb, int D, int V) {
	const int d4 = (D + 3) & ~3;
	return sizeof(float) * ((size_t)R * Gb * d4 + (size_t)SA_KT * sa_ldk(D, V) + (size_t)R * SA_KT + 5 * (size_t)R);
}

// cs[jj][0 .. n4) = cache row kt + jj, columns col0 .. col0 + n (zeros past n and past k_end)
template <class CT>
__device__ __forceinline__ void sa_fill_tile(float *cs, int ldk, const CT *cache, int row_len, int col0, int n, int kt,
                                             int k_end) {
	const int n4 = (n + 3) & ~3;
	if (n % 8 == 0 && col0 % 8 == 0 && row_len % 8 == 0 && (size_t)cache % 16 == 0) {
		const int v8n = n >> 3;
		for (int i = threadIdx.x; i < SA_KT * v8n; i += SEQ_THREADS) {
			const int jj = i / v8n, d = (i % v8n) * 8, j = kt + jj;
			float4_t lo = {0.0f, 0.0f, 0.0f, 0.0f}, hi = {0.0f, 0.0f, 0.0f, 0.0f};
			if (j < k_end) {
				const CT *src = cache + (size_t)j * row_len + col0 + d;
				if constexpr (sizeof(CT) == 2) {
					float f[8];
					WBF16::unpack(load16(src), f);
					lo = float4_t{f[0], f[1], f[2], f[3]};
					hi = float4_t{f[4], f[5], f[6], f[7]};
				} else {
					lo = *(const float4_t *)src;
					hi = *(const float4_t *)(src + 4);
				}
			}
			*(float4_t *)(cs + jj * ldk + d) = lo;
			*(float4_t *)(cs + jj * ldk + d + 4) = hi;
		}
	} else {
		for (int i = threadIdx.x; i < SA_KT * n4; i += SEQ_THREADS) {
			const int jj = i / n4, d = i % n4, j = kt + jj;
			float v = 0.0f;
			if (j < k_end && d < n) {
				if constexpr (sizeof(CT) == 2)
					v = bf2f(cache[(size_t)j * row_len + col0 + d]);
				else
					v = cache[(size_t)j * row_len + col0 + d];
			}
			cs[jj * ldk + d] = v;
		}
	}
}

// Q [t][H D]: the projection kernel's queries.
template <class CT, int NA4>
__global__ __launch_bounds__(SEQ_THREADS) void seq_attn_kernel(const float *__restrict__ Q,
                                                               const CT *__restrict__ Kc, const CT *__restrict__ Vc,
                                                               AttnArgs a, int n_tok, int TQ,
                                                               const StepState *__restrict__ st,
                                                               const float *__restrict__ gate, float *__restrict__ Ctx,
                                                               float *__restrict__ part) {
	extern __shared__ __attribute__((aligned(16))) float lds[];
	const int H = a.H, G = a.G, D = a.D, V = a.V, rep = H / G;
	const bool talk = a.talk != nullptr;
	const int Hb = rep, Gb = talk ? G : 1;
	const int h0 = blockIdx.z * rep, g0 = talk ? 0 : blockIdx.z, vg = blockIdx.z;
	const int R = TQ * Hb;
	const int D4 = (D + 3) & ~3, q4n = D4 >> 2, V4n = (V + 3) >> 2, ldk = sa_ldk(D, V), ldqs = Gb * D4;
	float *qs = lds;                  // [R][Gb][D4]
	float *cs = qs + R * ldqs;        // [SA_KT][ldk]: a key chunk, then a value tile
	float *ps = cs + SA_KT * ldk;     // [R][SA_KT] scores, then softmax weights
	float *mrun = ps + R * SA_KT;     // [R]
	float *lrun = mrun + R, *alpha = lrun + R;
	int *rlo = (int *)(alpha + R), *rhi = rlo + R;
	const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
	const int S = gridDim.y, split = blockIdx.y;
	const int t0 = blockIdx.x * TQ, pos0 = st->pos;
	const int t_last = min(t0 + TQ, n_tok) - 1;
	const int klo = attn_first_key(a.mask_kind, a.mask_size, pos0 + t0), khi = pos0 + t_last;
	int k_begin = klo, k_end = khi + 1;
	if (S > 1) {
		const int nkeys = khi - klo + 1;
		const int chunk = (((nkeys + S - 1) / S) + SA_KT - 1) & ~(SA_KT - 1);
		k_begin = klo + split * chunk;
		k_end = min(khi + 1, k_begin + chunk);
	}
	for (int i = tid; i < R * ldqs; i += SEQ_THREADS) {
		const int r = i / ldqs, c = (i % ldqs) / D4, d = i % D4;
		const int t = t0 + r / Hb, h = h0 + r % Hb;
		qs[i] = (t < n_tok && d < D) ? attn_query(Q, t, a.talk, a.q_mixed != 0, H, G, D, h, c * D + d) : 0.0f;
	}
	const bool sink0 = a.sink && split == 0;
	for (int r = tid; r < R; r += SEQ_THREADS) {
		const int t = t0 + r / Hb;
		mrun[r] = sink0 ? attn_sink_score(a, h0 + r % Hb) : -FLT_MAX;
		lrun[r] = sink0 ? 1.0f : 0.0f;
		alpha[r] = 1.0f;
		rlo[r] = t < n_tok ? attn_first_key(a.mask_kind, a.mask_size, pos0 + t) : 0x7fffffff;
		rhi[r] = t < n_tok ? pos0 + t : -1;
	}
	float4_t acc[NA4];
#pragma unroll
	for (int x = 0; x < NA4; ++x)
		acc[x] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};
	// few rows (single tokens): a row per wave and pass, so that every wave scores; else four
	const int rg = R >= 4 * (SEQ_THREADS / 64) ? 4 : 1;
	for (int kt = k_begin; kt < k_end; kt += SA_KT) {
		// ---- scores
		for (int c = 0; c < Gb; ++c) {
			__syncthreads(); // the previous readers of cs are done
			sa_fill_tile<CT>(cs, ldk, Kc, a.KL, (g0 + c) * D, D, kt, k_end);
			__syncthreads();
			const float4_t *cj = (const float4_t *)(cs + lane * ldk);
			for (int i0 = wave * rg; i0 < R; i0 += rg * (SEQ_THREADS / 64)) {
				int rr[4];
#pragma unroll
				for (int x = 0; x < 4; ++x)
					rr[x] = min(i0 + (x < rg ? x : 0), R - 1);
				float s[4] = {0.0f, 0.0f, 0.0f, 0.0f};
				if (rg == 4) {
					for (int d = 0; d < q4n; ++d) {
						const float4_t k4 = cj[d];
#pragma unroll
						for (int x = 0; x < 4; ++x) {
							const float4_t qv = *(const float4_t *)(qs + rr[x] * ldqs + c * D4 + 4 * d);
							s[x] = fmaf(qv[0], k4[0], s[x]);
							s[x] = fmaf(qv[1], k4[1], s[x]);
							s[x] = fmaf(qv[2], k4[2], s[x]);
							s[x] = fmaf(qv[3], k4[3], s[x]);
						}
					}
				} else {
					const float4_t *q0 = (const float4_t *)(qs + rr[0] * ldqs + c * D4);
					float s1 = 0.0f, s2 = 0.0f, s3 = 0.0f;
					for (int d = 0; d < q4n; ++d) {
						const float4_t k4 = cj[d], qv = q0[d];
						s[0] = fmaf(qv[0], k4[0], s[0]);
						s1 = fmaf(qv[1], k4[1], s1);
						s2 = fmaf(qv[2], k4[2], s2);
						s3 = fmaf(qv[3], k4[3], s3);
					}
					s[0] = (s[0] + s1) + (s2 + s3);
				}
#pragma unroll
				for (int x = 0; x < 4; ++x)
					if (x < rg && i0 + x < R) {
						float *dst = ps + rr[x] * SA_KT + lane;
						*dst = c == 0 ? s[x] : *dst + s[x];
					}
			}
		}
		__syncthreads();
		// ---- mask and running softmax, a wave per row
		for (int r = wave; r < R; r += SEQ_THREADS / 64) {
			const int j = kt + lane;
			const bool vis = j >= rlo[r] && j <= rhi[r] && j < k_end;
			const float sv = vis ? ps[r * SA_KT + lane] + attn_rel_bias(a, h0 + r % Hb, rhi[r] - j) : -FLT_MAX;
			const float mold = mrun[r], lold = lrun[r];
			const float mnew = fmaxf(mold, wave_max(sv));
			const float p = vis ? expf(sv - mnew) : 0.0f;
			const float al = expf(mold - mnew); // 1 while nothing is visible yet, 0 at the first key
			const float l = lold * al + wave_sum(p);
			ps[r * SA_KT + lane] = p;
			if (lane == 0) {
				mrun[r] = mnew;
				lrun[r] = l;
				alpha[r] = al;
			}
		}
		// ---- weighted sums of the values
		{
			__syncthreads(); // the weights are written / the previous readers of cs are done
			sa_fill_tile<CT>(cs, ldk, Vc, a.VL, vg * V, V, kt, k_end);
			__syncthreads();
#pragma unroll
			for (int x = 0; x < NA4; ++x) {
				const int u = tid + x * SEQ_THREADS;
				if (u >= R * V4n)
					continue;
				const int r = u / V4n, d4 = u % V4n;
				const float al = alpha[r];
				float4_t v = acc[x];
				v[0] *= al;
				v[1] *= al;
				v[2] *= al;
				v[3] *= al;
				const float4_t *pr = (const float4_t *)(ps + r * SA_KT);
#pragma unroll 4
				for (int j4 = 0; j4 < SA_KT / 4; ++j4) {
					const float4_t p = pr[j4];
#pragma unroll
					for (int e = 0; e < 4; ++e) {
						const float4_t c4 = *(const float4_t *)(cs + (4 * j4 + e) * ldk + 4 * d4);
						v[0] = fmaf(p[e], c4[0], v[0]);
						v[1] = fmaf(p[e], c4[1], v[1]);
						v[2] = fmaf(p[e], c4[2], v[2]);
						v[3] = fmaf(p[e], c4[3], v[3]);
					}
				}
				acc[x] = v;
			}
		}
	}
	__syncthreads();
	const int stride = 4 * V4n + 4;
#pragma unroll
	for (int x = 0; x < NA4; ++x) {
		const int u = tid + x * SEQ_THREADS;
		if (u >= R * V4n)
			continue;
		const int r = u / V4n, d4 = u % V4n;
		const int t = t0 + r / Hb, h = h0 + r % Hb;
		if (t >= n_tok)
			continue;
		const size_t row = (size_t)t * H + h;
		if (S == 1) {
			const float f = (gate ? gate[row] : 1.0f) / lrun[r];
#pragma unroll
			for (int e = 0; e < 4; ++e)
				if (4 * d4 + e < V)
					Ctx[row * V + 4 * d4 + e] = acc[x][e] * f;
		} else {
			float *pp = part + (row * S + split) * stride;
			*(float4_t *)(pp + 4 * d4) = acc[x];
			if (d4 == 0) {
				pp[4 * V4n] = mrun[r];
				pp[4 * V4n + 1] = lrun[r];
			}
		}
	}
}

// ------------------------------------------------------------------ attention, single token
// One decoded token: nothing is staged through LDS but the queries. A workgroup owns one key
// split (gridDim.x = S) of the heads of one key/value head (gridDim.y = G; with score mixing
// their mixed queries meet the whole key row), or of a block of hblk of them (hblk > 0, gridDim.z
// blocks: many heads over one key/value head, where key splits alone are too few workgroups to
// fill the chip); a lane owns a key and reads its cache row itself, 16 bytes at a time,
// eight loads in flight; wave w takes a quarter of the key entries against every head's
// queries (LDS broadcasts) and leaves partial scores in LDS; wave w then adds them up and
// normalises heads w, w + 4, ...; then every thread sums NA4 groups of 4 value entries of one
// head straight from the value rows. Partial results per split as in
// seq_attn_kernel (S == 1 writes Ctx).
template <class CT, int NA4>
__global__ __launch_bounds__(SEQ_THREADS) void seq_attn_decode_kernel(const float *__restrict__ Q,
                                                                      const CT *__restrict__ Kc,
                                                                      const CT *__restrict__ Vc, AttnArgs a,
                                                                      const StepState *__restrict__ st,
                                                                      const float *__restrict__ gate,
                                                                      float *__restrict__ Ctx, float *__restrict__ part,
                                                                      int hblk) {
	extern __shared__ __attribute__((aligned(16))) float lds[];
	constexpr int NW = SEQ_THREADS / 64;
	constexpr int EPL = sizeof(CT) == 2 ? 8 : 4; // cache entries per 16-byte load
	constexpr int HP = 16;                        // heads per pass over a key slice
	const int H = a.H, G = a.G, D = a.D, V = a.V, rep = H / G;
	const bool talk = a.talk != nullptr;
	// the heads of one key/value head (a block of them with gridDim.z > 1)
	const int hz = hblk > 0 ? blockIdx.z * hblk : 0;
	const int Hb = hblk > 0 ? min(hblk, rep - hz) : rep, h0 = blockIdx.y * rep + hz;
	const int DK = talk ? G * D : D, KL = a.KL, VL = a.VL, kcol = talk ? 0 : blockIdx.y * D;
	const int DK8 = (DK + 7) & ~7, V4n = (V + 3) >> 2;
	float *qs = lds;               // [Hb][DK8]
	float *ps = qs + Hb * DK8;     // [Hb][SA_KT] softmax weights
	float *pw = ps + Hb * SA_KT;   // [NW][Hb][SA_KT] the waves' partial scores
	float *mrun = pw + NW * Hb * SA_KT; // [Hb]
	float *lrun = mrun + Hb, *alpha = lrun + Hb;
	const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
	const int S = gridDim.x, split = blockIdx.x;
	const int pos = st->pos;
	const int klo = attn_first_key(a.mask_kind, a.mask_size, pos);
	int k_begin = klo, k_end = pos + 1;
	if (S > 1) {
		const int nkeys = pos - klo + 1;
		const int chunk = (((nkeys + S - 1) / S) + SA_KT - 1) & ~(SA_KT - 1);
		k_begin = klo + split * chunk;
		k_end = min(pos + 1, k_begin + chunk);
	}
	if (talk && !a.q_mixed) { // the token's queries and the mixing matrix through LDS, then the mixed queries
		float *qraw = alpha + Hb, *tk = qraw + H * D;
		for (int i = tid; i < H * D; i += SEQ_THREADS)
			qraw[i] = Q[i];
		for (int i = tid; i < H * H; i += SEQ_THREADS)
			tk[i] = a.talk[i];
		__syncthreads();
		for (int cd = tid; cd < DK8; cd += SEQ_THREADS) {
			const int c = cd / D, d = cd - c * D;
			for (int hl = 0; hl < Hb; ++hl) {
				float m = 0.0f;
				if (cd < DK)
					for (int x = 0; x < rep; ++x)
						m = fmaf(tk[(h0 + hl) * H + c * rep + x], qraw[(c * rep + x) * D + d], m);
				qs[hl * DK8 + cd] = m;
			}
		}
	} else {
		for (int i = tid; i < Hb * DK8; i += SEQ_THREADS) {
			const int hl = i / DK8, d = i % DK8;
			qs[i] = d < DK ? attn_query(Q, 0, a.talk, a.q_mixed != 0, H, G, D, h0 + hl, d) : 0.0f;
		}
	}
	const bool sink0 = a.sink && split == 0;
	for (int r = tid; r < Hb; r += SEQ_THREADS) {
		mrun[r] = sink0 ? attn_sink_score(a, h0 + r) : -FLT_MAX;
		lrun[r] = sink0 ? 1.0f : 0.0f;
		alpha[r] = 1.0f;
	}
	float4_t acc[NA4];
#pragma unroll
	for (int x = 0; x < NA4; ++x)
		acc[x] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};
	const bool kvec = DK % EPL == 0 && kcol % EPL == 0 && KL % EPL == 0 && (size_t)Kc % 16 == 0;
	const bool vvec = V % 4 == 0 && VL % 4 == 0 && (size_t)Vc % 16 == 0;
	const int DKw = (((DK + NW - 1) / NW) + EPL - 1) / EPL * EPL; // key entries per wave
	const int dlo = min(wave * DKw, DK), dhi = min(DK, dlo + DKw);
	__syncthreads();
	for (int kt = k_begin; kt < k_end; kt += SA_KT) {
		const int j = kt + lane;
		const bool live = j < k_end;
		const CT *krow = Kc + (size_t)(live ? j : k_end - 1) * KL + kcol;
		// ---- partial scores: wave w takes its slice of the key entries, every head (HP per pass)
		for (int hp0 = 0; hp0 < Hb; hp0 += HP) {
			const int nh = min(HP, Hb - hp0);
			float s[HP];
#pragma unroll
			for (int x = 0; x < HP; ++x)
				s[x] = 0.0f;
			if (kvec) {
				constexpr int U = 8; // loads in flight
				for (int d0 = dlo; d0 < dhi; d0 += U * EPL) {
					u32x4_t w[U];
#pragma unroll
					for (int u = 0; u < U; ++u)
						w[u] = d0 + u * EPL < dhi ? load16(krow + d0 + u * EPL) : u32x4_t{0, 0, 0, 0};
#pragma unroll
					for (int u = 0; u < U; ++u) {
						const int d = d0 + u * EPL;
						if (d >= dhi)
							break;
						float kf[EPL];
						if constexpr (sizeof(CT) == 2)
							WBF16::unpack(w[u], kf);
						else
							WF32::unpack(w[u], kf);
#pragma unroll
						for (int x = 0; x < HP; ++x) {
							if (x >= nh)
								break;
							const float *qp = qs + (hp0 + x) * DK8 + d;
#pragma unroll
							for (int e = 0; e < EPL; e += 4) {
								const float4_t qv = *(const float4_t *)(qp + e);
								s[x] = fmaf(qv[0], kf[e], s[x]);
								s[x] = fmaf(qv[1], kf[e + 1], s[x]);
								s[x] = fmaf(qv[2], kf[e + 2], s[x]);
								s[x] = fmaf(qv[3], kf[e + 3], s[x]);
							}
						}
					}
				}
			} else {
				for (int d = dlo; d < dhi; ++d) {
					float kv;
					if constexpr (sizeof(CT) == 2)
						kv = bf2f(krow[d]);
					else
						kv = krow[d];
#pragma unroll
					for (int x = 0; x < HP; ++x)
						if (x < nh)
							s[x] = fmaf(qs[(hp0 + x) * DK8 + d], kv, s[x]);
				}
			}
#pragma unroll
			for (int x = 0; x < HP; ++x)
				if (x < nh)
					pw[(wave * Hb + hp0 + x) * SA_KT + lane] = s[x];
		}
		__syncthreads();
		// ---- running softmax, a wave per head
		for (int r = wave; r < Hb; r += NW) {
			float sv = 0.0f;
#pragma unroll
			for (int w = 0; w < NW; ++w)
				sv += pw[(w * Hb + r) * SA_KT + lane];
			sv = live ? sv + attn_rel_bias(a, h0 + r, pos - j) : -FLT_MAX;
			const float mold = mrun[r], lold = lrun[r];
			const float mnew = fmaxf(mold, wave_max(sv));
			const float p = live ? expf(sv - mnew) : 0.0f;
			const float al = expf(mold - mnew);
			const float l = lold * al + wave_sum(p);
			ps[r * SA_KT + lane] = p;
			if (lane == 0) {
				mrun[r] = mnew;
				lrun[r] = l;
				alpha[r] = al;
			}
		}
		__syncthreads();
		// ---- weighted sums of the values
		const int nk = min(SA_KT, k_end - kt);
#pragma unroll
		for (int x = 0; x < NA4; ++x) {
			const int u = tid + x * SEQ_THREADS;
			if (u >= Hb * V4n)
				continue;
			const int r = u / V4n, d4 = u % V4n;
			const CT *vp = Vc + (size_t)kt * VL + ((h0 + r) / rep) * V + 4 * d4;
			const float al = alpha[r];
			float4_t v = acc[x];
			v[0] *= al;
			v[1] *= al;
			v[2] *= al;
			v[3] *= al;
			const float *pr = ps + r * SA_KT;
			if (vvec) {
#pragma unroll 16
				for (int jj = 0; jj < nk; ++jj) {
					float c4[4];
					if constexpr (sizeof(CT) == 2) {
						const uint2 raw = *(const uint2 *)(vp + (size_t)jj * VL);
						c4[0] = __builtin_bit_cast(float, raw.x << 16);
						c4[1] = __builtin_bit_cast(float, raw.x & 0xffff0000u);
						c4[2] = __builtin_bit_cast(float, raw.y << 16);
						c4[3] = __builtin_bit_cast(float, raw.y & 0xffff0000u);
					} else {
						const float4_t raw = *(const float4_t *)(vp + (size_t)jj * VL);
						c4[0] = raw[0];
						c4[1] = raw[1];
						c4[2] = raw[2];
						c4[3] = raw[3];
					}
					const float p = pr[jj];
					v[0] = fmaf(p, c4[0], v[0]);
					v[1] = fmaf(p, c4[1], v[1]);
					v[2] = fmaf(p, c4[2], v[2]);
					v[3] = fmaf(p, c4[3], v[3]);
				}
			} else {
				for (int jj = 0; jj < nk; ++jj) {
					const float p = pr[jj];
#pragma unroll
					for (int e = 0; e < 4; ++e) {
						if (4 * d4 + e >= V)
							break;
						float c;
						if constexpr (sizeof(CT) == 2)
							c = bf2f(vp[(size_t)jj * VL + e]);
						else
							c = vp[(size_t)jj * VL + e];
						v[e] = fmaf(p, c, v[e]);
					}
				}
			}
			acc[x] = v;
		}
		__syncthreads(); // ps and alpha are rewritten by the next tile
	}
	__syncthreads();
	const int stride = 4 * V4n + 4;
#pragma unroll
	for (int x = 0; x < NA4; ++x) {
		const int u = tid + x * SEQ_THREADS;
		if (u >= Hb * V4n)
			continue;
		const int r = u / V4n, d4 = u % V4n;
		const size_t row = h0 + r;
		if (S == 1) {
			const float f = (gate ? gate[row] : 1.0f) / lrun[r];
#pragma unroll
			for (int e = 0; e < 4; ++e)
				if (4 * d4 + e < V)
					Ctx[row * V + 4 * d4 + e] = acc[x][e] * f;
		} else {
			float *pp = part + (row * S + split) * stride;
			*(float4_t *)(pp + 4 * d4) = acc[x];
			if (d4 == 0) {
				pp[4 * V4n] = mrun[r];
				pp[4 * V4n + 1] = lrun[r];
			}
		}
	}
}
// HD = heads x dim with score mixing (the raw queries and the mixing matrix are staged), else 0
static inline size_t sa_decode_lds_bytes(int Hb, int DK, int HD, int H) {
	return sizeof(float) * ((size_t)Hb * ((DK + 7) & ~7) + (size_t)(1 + SEQ_THREADS / 64) * Hb * SA_KT + 3 * (size_t)Hb +
	                        (HD ? (size_t)HD + (size_t)H * H : 0));
}

// ------------------------------------------------------------------ attention, MFMA form (portions, bf16 cache)
// v_mfma_f32_16x16x32_bf16 products with f32 accumulation; the f32 operands (queries, softmax
// weights) enter as hi + lo bf16 pairs (hi = bf16(x), lo = bf16(x - hi): 16 significant bits),
// the cached keys and values being bf16 already. Maximum, exponentials, running sums and the
// rescaling of the sums stay f32, in the MFMA's C layout (row = 4 (lane >> 4) + reg, column =
// lane & 15). A workgroup serves one key/value head g: its 4 waves are 4 / HW blocks of 16
// tokens x HW query heads of g (blockIdx.z: which HW heads), so one key tile and one value tile
// in LDS feed every wave. Keys in tiles of 32 from the first key the workgroup's first token
// sees to its last token, the next tile's rows in flight (registers) during the current
// tile's products. KS = ceil(DK / 32), NT = ceil(V / 16).
#define SAM_KT 32
template <int KS, int NT>
__global__ __launch_bounds__(SEQ_THREADS) void seq_attn_mfma_kernel(const float *__restrict__ Q,
                                                                    const uint16_t *__restrict__ Kc,
                                                                    const uint16_t *__restrict__ Vc, AttnArgs a,
                                                                    int n_tok, int HW, const StepState *__restrict__ st,
                                                                    const float *__restrict__ gate,
                                                                    float *__restrict__ Ctx) {
	constexpr int DKP = 32 * KS, LDK = DKP + 8, LDT = SAM_KT + 8, LDP = SAM_KT + 8, VP = 16 * NT;
	__shared__ __attribute__((aligned(16))) uint16_t Ks[SAM_KT * LDK];    // [key][key entry]
	__shared__ __attribute__((aligned(16))) uint16_t VsT[VP * LDT];       // [value entry][key]
	__shared__ __attribute__((aligned(16))) uint16_t Ps[4][2][16 * LDP];  // per wave: weights hi / lo [row][key]
	const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
	const int lr = lane & 15, lq = lane >> 4;
	const int H = a.H, G = a.G, D = a.D, V = a.V, rep = H / G;
	const bool talk = a.talk != nullptr;
	const int DK = talk ? G * D : D, KL = a.KL, VL = a.VL;
	const int g = blockIdx.y;
	const int kcol = talk ? 0 : g * D;
	const int TB = 4 / HW, tb = wave / HW, hl = blockIdx.z * HW + wave % HW;
	const bool active = hl < rep;
	const int h = g * rep + min(hl, rep - 1);
	const int t0 = blockIdx.x * 16 * TB, tw0 = t0 + 16 * tb;
	const int pos0 = st->pos;
	const int t_last = min(t0 + 16 * TB, n_tok) - 1;
	const int klo = attn_first_key(a.mask_kind, a.mask_size, pos0 + t0), khi = pos0 + t_last;
	// the keys this wave's rows see: between the first row's first key and the last row's position
	const int wlo = attn_first_key(a.mask_kind, a.mask_size, pos0 + min(tw0, n_tok - 1));
	const int whi = pos0 + min(tw0 + 15, n_tok - 1);
	const bool wave_on = active && tw0 < n_tok;
	bf16x8_t qh[KS], ql[KS];
	{
		const int t = tw0 + lr;
		const int tq = min(t, n_tok - 1);
#pragma unroll
		for (int sst = 0; sst < KS; ++sst) {
			u32x4_t hi = {0, 0, 0, 0}, lo = {0, 0, 0, 0};
#pragma unroll
			for (int e = 0; e < 8; ++e) {
				const int d = 32 * sst + 8 * lq + e;
				const float x =
				    (wave_on && t < n_tok && d < DK) ? attn_query(Q, tq, a.talk, a.q_mixed != 0, H, G, D, h, d) : 0.0f;
				const uint16_t hb = f2bf(x);
				const uint16_t lb = f2bf(x - bf2f(hb));
				hi[e >> 1] |= (uint32_t)hb << (16 * (e & 1));
				lo[e >> 1] |= (uint32_t)lb << (16 * (e & 1));
			}
			qh[sst] = __builtin_bit_cast(bf16x8_t, hi);
			ql[sst] = __builtin_bit_cast(bf16x8_t, lo);
		}
	}
	int lo_[4], hi_[4];
	float mrun[4], lrun[4];
#pragma unroll
	for (int r = 0; r < 4; ++r) {
		const int t = tw0 + 4 * lq + r;
		const bool ok = wave_on && t < n_tok;
		lo_[r] = ok ? attn_first_key(a.mask_kind, a.mask_size, pos0 + t) : 0x7fffffff;
		hi_[r] = ok ? pos0 + t : -1;
		mrun[r] = a.sink ? attn_sink_score(a, h) : -FLT_MAX;
		lrun[r] = a.sink ? 1.0f : 0.0f;
	}
	f32x4a_t oacc[NT];
#pragma unroll
	for (int n = 0; n < NT; ++n)
		oacc[n] = f32x4a_t{0.0f, 0.0f, 0.0f, 0.0f};
	const bool kvec = DK % 8 == 0 && kcol % 8 == 0 && KL % 8 == 0 && (size_t)Kc % 16 == 0;
	const bool vvec = V % 8 == 0 && VL % 8 == 0 && (size_t)Vc % 16 == 0;
	// The next tile's cache rows are fetched into registers before the current tile's products
	// and stored to LDS after them: the global-load latency runs under the matrix work.
	constexpr int NKL = (SAM_KT * (DKP / 8) + SEQ_THREADS - 1) / SEQ_THREADS; // 16-byte pieces per thread
	constexpr int NVL = (SAM_KT * (VP / 8) + SEQ_THREADS - 1) / SEQ_THREADS;
	u32x4_t kreg[NKL], vreg[NVL];
	auto fetch = [&](int kt) {
#pragma unroll
		for (int i = 0; i < NKL; ++i) {
			const int v = tid + i * SEQ_THREADS;
			const int jj = v / (DKP / 8), d8 = (v % (DKP / 8)) * 8, j = kt + jj;
			u32x4_t w = {0, 0, 0, 0};
			if (v < SAM_KT * (DKP / 8) && j <= khi && d8 < DK) {
				const uint16_t *src = Kc + (size_t)j * KL + kcol + d8;
				if (kvec && d8 + 8 <= DK) {
					w = load16(src);
				} else {
#pragma unroll
					for (int e = 0; e < 8; ++e)
						if (d8 + e < DK)
							w[e >> 1] |= (uint32_t)src[e] << (16 * (e & 1));
				}
			}
			kreg[i] = w;
		}
#pragma unroll
		for (int i = 0; i < NVL; ++i) {
			const int v = tid + i * SEQ_THREADS;
			const int jj = v % SAM_KT, d8 = (v / SAM_KT) * 8, j = kt + jj;
			u32x4_t w = {0, 0, 0, 0};
			if (v < SAM_KT * (VP / 8) && j <= khi && d8 < V) {
				const uint16_t *src = Vc + (size_t)j * VL + g * V + d8;
				if (vvec && d8 + 8 <= V) {
					w = load16(src);
				} else {
#pragma unroll
					for (int e = 0; e < 8; ++e)
						if (d8 + e < V)
							w[e >> 1] |= (uint32_t)src[e] << (16 * (e & 1));
				}
			}
			vreg[i] = w;
		}
	};
	auto stash = [&]() {
#pragma unroll
		for (int i = 0; i < NKL; ++i) {
			const int v = tid + i * SEQ_THREADS;
			if (v < SAM_KT * (DKP / 8))
				*(u32x4_t *)(Ks + (v / (DKP / 8)) * LDK + (v % (DKP / 8)) * 8) = kreg[i];
		}
#pragma unroll
		for (int i = 0; i < NVL; ++i) {
			const int v = tid + i * SEQ_THREADS;
			if (v < SAM_KT * (VP / 8)) {
				const int jj = v % SAM_KT, d8 = (v / SAM_KT) * 8;
#pragma unroll
				for (int e = 0; e < 8; ++e)
					VsT[(d8 + e) * LDT + jj] = (uint16_t)(vreg[i][e >> 1] >> (16 * (e & 1)));
			}
		}
	};
	fetch(klo);
	for (int kt = klo; kt <= khi; kt += SAM_KT) {
		__syncthreads(); // the previous tile's products have read Ks / VsT / Ps
		stash();
		if (kt + SAM_KT <= khi)
			fetch(kt + SAM_KT);
		__syncthreads();
		const bool need = wave_on && kt <= whi && kt + SAM_KT - 1 >= wlo;
		if (need) {
			f32x4a_t sacc[2] = {f32x4a_t{0.0f, 0.0f, 0.0f, 0.0f}, f32x4a_t{0.0f, 0.0f, 0.0f, 0.0f}};
			// the distance biases of this lane's eight scores: loaded now, in flight under the products
			float rb0[4], rb1[4];
#pragma unroll
			for (int r = 0; r < 4; ++r) {
				rb0[r] = attn_rel_bias(a, h, hi_[r] - (kt + lr));
				rb1[r] = attn_rel_bias(a, h, hi_[r] - (kt + 16 + lr));
			}
#pragma unroll
			for (int jt = 0; jt < 2; ++jt)
#pragma unroll
				for (int sst = 0; sst < KS; ++sst) {
					const bf16x8_t kb =
					    __builtin_bit_cast(bf16x8_t, *(const u32x4_t *)(Ks + (16 * jt + lr) * LDK + 32 * sst + 8 * lq));
					sacc[jt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(qh[sst], kb, sacc[jt], 0, 0, 0);
					sacc[jt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ql[sst], kb, sacc[jt], 0, 0, 0);
				}
			float al[4];
#pragma unroll
			for (int r = 0; r < 4; ++r) {
				const int j0 = kt + lr, j1 = kt + 16 + lr;
				const bool v0 = j0 >= lo_[r] && j0 <= hi_[r], v1 = j1 >= lo_[r] && j1 <= hi_[r];
				const float s0 = v0 ? sacc[0][r] + rb0[r] : -FLT_MAX;
				const float s1 = v1 ? sacc[1][r] + rb1[r] : -FLT_MAX;
				const float mnew = fmaxf(mrun[r], row16_max(fmaxf(s0, s1)));
				const float p0 = v0 ? expf(s0 - mnew) : 0.0f, p1 = v1 ? expf(s1 - mnew) : 0.0f;
				al[r] = expf(mrun[r] - mnew);
				lrun[r] = lrun[r] * al[r] + row16_sum(p0 + p1);
				mrun[r] = mnew;
				const int row = 4 * lq + r;
				const uint16_t h0 = f2bf(p0), h1 = f2bf(p1);
				Ps[wave][0][row * LDP + lr] = h0;
				Ps[wave][0][row * LDP + 16 + lr] = h1;
				Ps[wave][1][row * LDP + lr] = f2bf(p0 - bf2f(h0));
				Ps[wave][1][row * LDP + 16 + lr] = f2bf(p1 - bf2f(h1));
			}
#pragma unroll
			for (int n = 0; n < NT; ++n)
#pragma unroll
				for (int r = 0; r < 4; ++r)
					oacc[n][r] *= al[r];
		}
		__syncthreads(); // the waves' weights are in LDS
		if (need) {
			const bf16x8_t ph = __builtin_bit_cast(bf16x8_t, *(const u32x4_t *)(&Ps[wave][0][lr * LDP + 8 * lq]));
			const bf16x8_t pl = __builtin_bit_cast(bf16x8_t, *(const u32x4_t *)(&Ps[wave][1][lr * LDP + 8 * lq]));
#pragma unroll
			for (int n = 0; n < NT; ++n) {
				const bf16x8_t vb = __builtin_bit_cast(bf16x8_t, *(const u32x4_t *)(VsT + (16 * n + lr) * LDT + 8 * lq));
				oacc[n] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ph, vb, oacc[n], 0, 0, 0);
				oacc[n] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(pl, vb, oacc[n], 0, 0, 0);
			}
		}
	}
#pragma unroll
	for (int r = 0; r < 4; ++r) {
		const int t = tw0 + 4 * lq + r;
		if (!wave_on || t >= n_tok)
			continue;
		const size_t row = (size_t)t * H + h;
		const float f = (gate ? gate[row] : 1.0f) / lrun[r];
#pragma unroll
		for (int n = 0; n < NT; ++n) {
			const int d = 16 * n + lr;
			if (d < V)
				Ctx[row * V + d] = oacc[n][r] * f;
		}
	}
}
