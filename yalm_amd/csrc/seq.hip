// seq.hip — the layer-list engine of the C ABI (include/yalm_hip.h, "layer-list models"):
// a decoder whose layers each name their token mixer (latent attention, real-gated linear
// recurrence, gated delta rule, softmax attention with a window or chunk mask, selective
// state-space layer, or two of them side by side) and
// feed-forward (dense GLU, routed experts, plain), holding one sequence's latent and
// key / value caches and recurrent / convolution states in HBM. One step function
// serves whole prompts, portions of prompts and single decoded tokens; the device greedy
// loop feeds the argmax back without a host round trip, as yalm_generate_greedy does.
#include "../../include/yalm_hip.h"

#include <hip/hip_runtime.h>

#include <algorithm>
#include <cmath>
#include <cstring>
#include <string>
#include <vector>

#include "decoder.h"
#include "device_common.h"
#include "misc_kernels.h"
#include "seq_kernels.h"
#include "seq_attn.h"

// The large-tile 8-phase GEMM of the prefill unit (prefill.hip), bf16 instantiation. Weak: the
// library built from the shim and this unit alone has no prefill unit, and every product then
// runs on this unit's general-shape kernels.
int pf_gemm_bf16(const uint16_t *A, int lda, int M, int K, const uint16_t *W, int N, float *C, int ldc,
                 const float *bias, int act, hipStream_t st) __attribute__((weak));

int pf_gemm_glu_bf16(const uint16_t *A, int lda, int M, int K, const uint16_t *Wg, const uint16_t *Wu, int hidden,
                     float *C, int ldc, int mode, float limit, hipStream_t st) __attribute__((weak));

struct yalm_seq_s {
	yalm_seq_config c{};
	std::vector<yalm_seq_layer> L;
	const void *embed = nullptr, *head = nullptr;
	const float *final_norm = nullptr;
	hipStream_t stream = nullptr;
	bool own_stream = false;
	StepState *st = nullptr;
	int host_pos = 0;
	int cap = 0;                 // tokens per internal portion
	size_t bw = 0;               // floats per row of the work buffers B0..B3
	int zw = 0;                  // floats per row of Z (the widest input projection)
	float *X = nullptr, *Hn = nullptr, *Y = nullptr, *Y2 = nullptr, *Z = nullptr, *B[4] = {};
	float *Hn2 = nullptr;        // parallel blocks whose feed-forward has a norm of its own: norm2(x)
	float *Y3 = nullptr;         // the result of a layer's second mixer (side) before the two are joined
	float *Yout = nullptr;       // where the mixer being enqueued leaves its result: Y, or Y3
	const float *embed_norm = nullptr;
	std::vector<int> side_of;    // per layer: index in L of its second mixer, or -1 (sides follow the n_layers entries)
	std::vector<float *> rel_dist; // attn with a distance bias: [rel_far + 1][heads], the bucketed table per distance
	std::vector<int> rel_far;
	const float *In = nullptr;   // what a sublayer reads: Hn (pre_norm) or X itself
	float *Xalt = nullptr, *Xbase = nullptr; // single tokens without opening norms: the stream alternates between two rows
	const float *pend_wb = nullptr; // a closing norm not yet applied: X += norm(Y) pend_wb, owed to the next product
	bool ln = false;             // the model's norms are layer norms
	float *inv_freq = nullptr;
	uint16_t *a16 = nullptr;     // [cap][bw] bf16 copy of a product's activations (large-tile GEMM operand)
	int *tok = nullptr, *want = nullptr;
	float *logits = nullptr;     // [LOGIT_ROWS][vocab]
	int *idx = nullptr, *counts = nullptr, *lists = nullptr;
	float *wt = nullptr, *sgate = nullptr;
	int cur_pos = 0;             // the position the portion being enqueued starts at (host copy of st->pos)
	// latent attention with directly projected queries, portions: the visible positions' latents
	// as f32, their expanded keys | values as f32, then per-head key and value rows in the cache's type
	float *ex_c = nullptr, *ex_kv = nullptr;
	void *ex_k = nullptr, *ex_v = nullptr;
	int ex_rows = 0;
	float *att_part = nullptr;   // latent attention: per (row, key split) partial sums, maximum, sum
	int att_splits = 1;          // key splits of single-token / short-portion attention
	float *arena = nullptr;      // every recurrent and convolution state of the sequence
	size_t arena_floats = 0;
	std::vector<void *> cache;   // per layer: [max_tokens][kv_rank (+ rot_dim)] latent rows (own latent only); attn: key rows
	std::vector<void *> vcache;  // attn: [max_tokens][kv_heads vdim] value rows; latent with a rotated key part: the latent rows again
	std::vector<double *> rot_freq; // attn: [rot_dims / 2] rotary angle per position
	std::vector<float> rot_mag;
	std::vector<int> attn_splits; // attn: key splits of single tokens and short portions
	std::vector<float *> S, conv;
	float *dump = nullptr;
	bool dump_on = false;
	int dump_n = 0;
	int *gen_tokens = nullptr;
	int gen_cap = 0;
	// one greedy token (step, logits, argmax) as a static hipGraph: every position-dependent
	// value is read from the device StepState, so the same graph serves every token; the host
	// then pays one launch per token instead of one per kernel (the greedy loop is otherwise
	// bound by the host's launch rate, not by the device)
	hipGraph_t greedy_graph = nullptr;
	hipGraphExec_t greedy_exec = nullptr;
	std::vector<void *> allocs;
};
typedef yalm_seq_s Seq;

enum { LOGIT_ROWS = 64, SEQ_PORTION_CAP = 4096 };

static int salloc(Seq *q, void **p, size_t bytes) {
	*p = nullptr;
	HIPCHK(hipMalloc(p, bytes ? bytes : 1));
	q->allocs.push_back(*p);
	HIPCHK(hipMemset(*p, 0, bytes ? bytes : 1));
	return YALM_OK;
}
template <class T>
static int sallocT(Seq *q, T **p, size_t count) {
	return salloc(q, (void **)p, count * sizeof(T));
}

static int cdiv(int a, int b) {
	return (a + b - 1) / b;
}

// ------------------------------------------------------------------ validation
static int in_rows(const yalm_seq_layer &l) {
	switch (l.mixer) {
	case YALM_MIX_LATENT:
		if (l.q_rank == 0)
			return l.heads * (l.dim + l.rot_dim) + l.kv_rank + l.rot_dim;
		return l.q_rank + (l.kv_from < 0 ? l.kv_rank : 0);
	case YALM_MIX_RGLRU: return 2 * l.rec_width;
	case YALM_MIX_ATTN:
		return l.heads * l.dim + l.kv_heads * (l.dim + l.vdim) +
		       (l.out_gate == 2 ? l.heads * l.vdim : (l.out_gate ? l.heads : 0));
	case YALM_MIX_SSM: return 2 * l.heads * l.vdim + 2 * l.ssm_groups * l.ssm_state + l.heads;
	default:
		return 2 * l.kv_heads * l.dim + l.heads * l.vdim + (l.gate_rank > 0 ? l.gate_rank : l.heads * l.vdim) + l.heads +
		       (l.decay_rank > 0 ? l.decay_rank : l.heads);
	}
}

// latent attention whose queries come from the input directly (q_rank = 0): served by the
// softmax-attention kernels as one key/value head whose key row is [latent | rotated key part]
static bool latent_direct(const yalm_seq_layer &l) {
	return l.mixer == YALM_MIX_LATENT && l.q_rank == 0;
}

static int validate(const yalm_seq_config &c, const std::vector<yalm_seq_layer> &L) {
	ARGCHK(c.width > 0 && c.vocab > 0 && c.n_layers > 0 && c.max_tokens > 0, "yalm_seq_create: bad model sizes");
	ARGCHK(c.weight_dtype == YALM_BF16 || c.weight_dtype == YALM_F32, "yalm_seq_create: weight_dtype must be bf16 or f32");
	ARGCHK(c.norm_kind == YALM_NORM_RMS || c.norm_kind == YALM_NORM_LAYER, "yalm_seq_create: unknown norm kind");
	ARGCHK(c.block_kind == YALM_BLOCK_SERIAL || (c.block_kind == YALM_BLOCK_PARALLEL && c.pre_norm),
	       "yalm_seq_create: blocks are serial, or parallel with pre_norm");
	const bool par = c.block_kind == YALM_BLOCK_PARALLEL;
	for (int i = 0; i < (int)L.size(); ++i) { // the n_layers entries, then their second mixers
		const yalm_seq_layer &l = L[i];
		const bool is_side = i >= c.n_layers;
		const std::string at = "yalm_seq_create: " + std::string(is_side ? "second mixer " : "layer ") +
		                       std::to_string(is_side ? i - c.n_layers : i) + ": ";
		ARGCHK(l.w_in && l.w_o, at + "missing tensors");
		if (is_side) {
			ARGCHK(l.ff_kind == YALM_FF_NONE && !l.side && !l.pre_add, at + "a second mixer has no feed-forward, no vector and no side of its own");
		} else {
			ARGCHK((l.norm1 || !c.pre_norm) && (l.norm1b || par), at + "missing tensors");
			ARGCHK(!l.side || (l.join_w && l.side_join_w), at + "two mixers side by side need the norm weights of their results");
		}
		ARGCHK(l.ff_act >= YALM_ACT_DEFAULT && l.ff_act <= YALM_ACT_RELU2 &&
		           (l.ff_act != YALM_ACT_RELU2 || l.ff_kind == YALM_FF_PLAIN || l.ff_kind == YALM_FF_NONE),
		       at + "unknown feed-forward activation (relu^2 belongs to the plain feed-forward)");
		ARGCHK(!l.pre_add || i == 0 || par, at + "a vector added before an entry after the first needs parallel blocks");
		if (latent_direct(l)) {
			ARGCHK(l.heads > 0 && l.dim > 0 && l.vdim > 0 && l.kv_rank > 0 && l.rot_dim >= 0 && l.kv_from < 0,
			       at + "bad latent attention sizes");
			if ((size_t)l.heads * ((l.kv_rank + 3) / 4) > (size_t)SA_MAX_NA4 * SEQ_THREADS) {
				set_err(at + "heads x kv_rank above 16384 is not implemented by the attention kernels");
				return YALM_ERR_UNSUPPORTED;
			}
			ARGCHK(l.kv_norm && l.w_ukt && (l.w_uv || l.w_ukv), at + "missing latent attention tensors");
			ARGCHK(l.mask_kind == YALM_MASK_CAUSAL || ((l.mask_kind == YALM_MASK_WINDOW || l.mask_kind == YALM_MASK_CHUNK) && l.mask_size > 0),
			       at + "bad attention mask");
			ARGCHK(l.rot_dims >= 0 && l.rot_dims <= l.rot_dim && l.rot_dims % 2 == 0 && (l.rot_dims == 0 || l.rot_base > 0.0f),
			       at + "rotary sizes must be even and at most rot_dim");
			ARGCHK(!(l.rot_factor > 0.0f) || (l.rot_orig > 0 && l.rot_fast > 0.0f && l.rot_slow > 0.0f && l.rot_base != 1.0f),
			       at + "bad rotary rescaling");
		} else if (l.mixer == YALM_MIX_LATENT) {
			ARGCHK(l.heads > 0 && l.dim > 0 && l.vdim > 0 && l.kv_rank > 0 && l.q_rank > 0, at + "bad latent attention sizes");
			ARGCHK(l.rot_dim == 0 && l.mask_kind == YALM_MASK_CAUSAL && !l.sink,
			       at + "a rotated key part, a mask or a sink need directly projected queries (q_rank = 0)");
			if (l.kv_rank > 256) {
				set_err(at + "kv_rank above 256 is not implemented by the latent attention kernel");
				return YALM_ERR_UNSUPPORTED;
			}
			ARGCHK(l.q_norm && l.w_uq && l.w_ukt && l.w_uv, at + "missing latent attention tensors");
			if (l.kv_from >= 0) {
				ARGCHK(l.kv_from < i && L[l.kv_from].mixer == YALM_MIX_LATENT && L[l.kv_from].kv_from < 0 &&
				           L[l.kv_from].kv_rank == l.kv_rank,
				       at + "kv_from must name an earlier latent attention layer with its own latent of the same rank");
			} else {
				ARGCHK(l.kv_norm, at + "missing latent norm");
			}
		} else if (l.mixer == YALM_MIX_RGLRU) {
			ARGCHK(l.rec_width > 0 && l.blocks > 0 && l.rec_width % l.blocks == 0, at + "bad recurrence sizes");
			ARGCHK(l.conv >= 1 && l.conv <= SEQ_MAX_TAPS, at + "convolution taps out of range");
			ARGCHK(l.in_bias && l.conv_w && l.conv_b && l.gate_a && l.gate_a_b && l.gate_i && l.gate_i_b && l.lam,
			       at + "missing recurrence tensors");
		} else if (l.mixer == YALM_MIX_DELTA) {
			ARGCHK(l.heads > 0 && l.kv_heads > 0 && l.heads % l.kv_heads == 0 && l.dim > 0 && l.vdim > 0,
			       at + "bad delta rule sizes");
			if (l.dim > 256) {
				set_err(at + "dim above 256 is not implemented by the delta rule kernel");
				return YALM_ERR_UNSUPPORTED;
			}
			ARGCHK(l.conv >= 1 && l.conv <= SEQ_MAX_TAPS, at + "convolution taps out of range");
			ARGCHK(l.conv_w && l.a_log && l.dt_bias && l.out_norm, at + "missing delta rule tensors");
			ARGCHK(l.decay_rank >= 0 && l.gate_rank >= 0 && (l.decay_rank == 0 || l.w_a2) && (l.gate_rank == 0 || l.w_g2) &&
			           (l.gate_act == YALM_GATE_SILU || l.gate_act == YALM_GATE_SIGMOID),
			       at + "bad low-rank decay / gate of the delta rule");
		} else if (l.mixer == YALM_MIX_SSM) {
			ARGCHK(l.heads > 0 && l.vdim > 0 && l.ssm_state > 0 && l.ssm_groups > 0 && l.heads % l.ssm_groups == 0 &&
			           l.norm_groups > 0 && (l.heads * l.vdim) % l.norm_groups == 0,
			       at + "bad state-space sizes");
			if (l.ssm_state > 256) {
				set_err(at + "a state of more than 256 rows is not implemented by the recurrence kernel");
				return YALM_ERR_UNSUPPORTED;
			}
			ARGCHK(l.conv >= 1 && l.conv <= SEQ_MAX_TAPS, at + "convolution taps out of range");
			ARGCHK(l.conv_w && l.a_log && l.dt_bias && l.d_skip && l.out_norm, at + "missing state-space tensors");
		} else if (l.mixer == YALM_MIX_ATTN) {
			ARGCHK(l.heads > 0 && l.kv_heads > 0 && l.heads % l.kv_heads == 0 && l.dim > 0 && l.vdim > 0,
			       at + "bad attention sizes");
			if (l.dim > 256 || l.vdim > 256 || (size_t)l.heads * ((l.vdim + 3) / 4) > (size_t)SA_MAX_NA4 * SEQ_THREADS) {
				set_err(at + "heads of more than 256 entries (or heads x vdim above 16384) are not implemented by the attention kernels");
				return YALM_ERR_UNSUPPORTED;
			}
			ARGCHK(l.mask_kind == YALM_MASK_CAUSAL || ((l.mask_kind == YALM_MASK_WINDOW || l.mask_kind == YALM_MASK_CHUNK) && l.mask_size > 0),
			       at + "bad attention mask");
			ARGCHK(l.qk_norm == YALM_QK_NONE || l.qk_norm == YALM_QK_HEAD_UNIT || (l.qk_norm == YALM_QK_WHOLE && l.q_norm && l.kv_norm) ||
			           (l.qk_norm == YALM_QK_HEAD_W && l.q_norm && l.kv_norm && l.rot_dims == 0),
			       at + "bad query / key norm");
			ARGCHK(l.rel_rows == 0 || (l.rel && l.rel_rows >= 2 && l.rel_max > (float)(l.rel_rows / 2)),
			       at + "a distance bias needs its table, at least two rows and rel_max above half of them");
			ARGCHK(l.q_temp_every >= 0, at + "bad query temperature");
			ARGCHK(l.out_gate >= 0 && l.out_gate <= 2, at + "unknown output gate");
			ARGCHK(l.rot_dims >= 0 && l.rot_dims <= l.dim && l.rot_dims % 2 == 0 && (l.rot_dims == 0 || l.rot_base > 0.0f),
			       at + "rotary sizes must be even and at most dim");
			ARGCHK(!(l.rot_factor > 0.0f) || (l.rot_orig > 0 && l.rot_fast > 0.0f && l.rot_slow > 0.0f && l.rot_base != 1.0f),
			       at + "bad rotary rescaling");
		} else {
			ARGCHK(false, at + "unknown mixer");
		}
		if (l.ff_kind == YALM_FF_DENSE) {
			ARGCHK(l.ff > 0 && l.w_gate && l.w_up && l.w_down && (par || ((l.norm2 || !c.pre_norm) && l.norm2b)), at + "bad dense feed-forward");
		} else if (l.ff_kind == YALM_FF_PLAIN) {
			ARGCHK(l.ff > 0 && l.w_up && l.w_down && (par || ((l.norm2 || !c.pre_norm) && l.norm2b)), at + "bad plain feed-forward");
		} else if (l.ff_kind == YALM_FF_MOE) {
			ARGCHK(l.ff > 0 && l.experts > 0 && l.top > 0 && l.top <= l.experts && l.groups > 0 &&
			           l.groups <= SEQ_MAX_GROUPS && l.experts % l.groups == 0 && l.groups_keep > 0 &&
			           l.groups_keep <= l.groups && l.top <= l.groups_keep * (l.experts / l.groups),
			       at + "bad router sizes");
			ARGCHK(l.router_kind == YALM_ROUTER_SOFTMAX_TOP || l.router_kind == YALM_ROUTER_SIGMOID_GROUPS ||
			           (l.router_kind == YALM_ROUTER_TOP_SOFTMAX && l.groups == 1),
			       at + "unknown router kind (the top-logits router has no groups)");
			ARGCHK(l.router && l.w_gate && l.w_up && l.w_down && (par || ((l.norm2 || !c.pre_norm) && l.norm2b)), at + "missing expert tensors");
			if (l.shared_ff > 0)
				ARGCHK(l.ws_gate && l.ws_up && l.ws_down, at + "missing shared expert tensors");
		} else {
			ARGCHK(l.ff_kind == YALM_FF_NONE, at + "unknown feed-forward kind");
		}
	}
	return YALM_OK;
}

// ------------------------------------------------------------------ create / destroy
static void destroy_seq(Seq *q) {
	if (q->greedy_exec)
		(void)hipGraphExecDestroy(q->greedy_exec);
	if (q->greedy_graph)
		(void)hipGraphDestroy(q->greedy_graph);
	for (void *p : q->allocs)
		(void)hipFree(p);
	if (q->own_stream && q->stream)
		(void)hipStreamDestroy(q->stream);
	delete q;
}

template <class CT, int NACC>
static int att_attr(int rank) {
	HIPCHK(hipFuncSetAttribute((const void *)seq_latent_attn_kernel<CT, NACC>, hipFuncAttributeMaxDynamicSharedMemorySize,
	                           (int)att_lds_bytes(rank)));
	return YALM_OK;
}
template <class CT>
static int att_attr_ct(int rank) {
	const int na = cdiv(att_rank4(rank), 64);
	if (na <= 1) return att_attr<CT, 1>(rank);
	if (na <= 2) return att_attr<CT, 2>(rank);
	return att_attr<CT, 4>(rank);
}

// attn: the rotary angle per position of every rotated pair, in double. Pair i turns
// base^(-2i / dims) radians per position; with a rescaling (rot_factor > 0) the pairs that
// turn fewer than rot_slow times within rot_orig positions turn rot_factor times slower, those
// that turn more than rot_fast times are left, a linear ramp over the pair index between, and
// cos / sin are scaled by 0.1 ln(rot_factor) + 1.
static int attn_setup(yalm_seq_s *q, int li) {
	const yalm_seq_layer &l = q->L[li];
	const int dims = l.rot_dims, half = dims / 2;
	std::vector<double> f(std::max(half, 1), 0.0);
	double mag = 1.0;
	for (int i = 0; i < half; ++i)
		f[i] = std::pow((double)l.rot_base, -2.0 * i / (double)dims);
	if (l.rot_factor > 0.0f && half > 0) {
		const double pi = 3.14159265358979323846;
		auto turn = [&](double t) { return dims * std::log((double)l.rot_orig / (2.0 * pi * t)) / (2.0 * std::log((double)l.rot_base)); };
		const double lo = std::max(std::floor(turn(l.rot_fast)), 0.0);
		const double hi = std::min(std::ceil(turn(l.rot_slow)), (double)(dims - 1));
		for (int i = 0; i < half; ++i) {
			const double ramp = std::min(std::max((i - lo) / std::max(hi - lo, 0.001), 0.0), 1.0);
			f[i] = f[i] / (double)l.rot_factor * ramp + f[i] * (1.0 - ramp);
		}
		mag = 0.1 * std::log((double)l.rot_factor) + 1.0;
	}
	q->rot_mag[li] = (float)mag;
	TRY(sallocT(q, &q->rot_freq[li], f.size()));
	HIPCHK(hipMemcpy(q->rot_freq[li], f.data(), f.size() * sizeof(double), hipMemcpyHostToDevice));
	return YALM_OK;
}

// attn with a distance bias: the layer's bucketed table rel [rel_rows][heads] expanded per
// distance, [rel_far + 1][heads], so that the kernels look a bias up by min(i - j, rel_far).
// bucket(n) = n below half = rel_rows / 2, else min(rel_rows - 1, half + floor(ln(n / half) /
// ln(rel_max / half) (rel_rows - half))), evaluated in double; from rel_max on every distance
// falls into the last row.
static int rel_setup(yalm_seq_s *q, int li) {
	const yalm_seq_layer &l = q->L[li];
	if (l.rel_rows <= 0)
		return YALM_OK;
	const int B = l.rel_rows, half = B / 2, H = l.heads;
	const int far = std::max(half, std::min(q->c.max_tokens - 1, (int)std::ceil((double)l.rel_max)));
	std::vector<float> rel((size_t)B * H), tab((size_t)(far + 1) * H);
	HIPCHK(hipMemcpy(rel.data(), l.rel, rel.size() * sizeof(float), hipMemcpyDeviceToHost));
	for (int n = 0; n <= far; ++n) {
		int b = n;
		if (n >= half) {
			const double x = std::log((double)n / half) / std::log((double)l.rel_max / half) * (double)(B - half);
			b = (int)std::min((double)(B - 1), (double)half + std::floor(x));
		}
		for (int h = 0; h < H; ++h)
			tab[(size_t)n * H + h] = rel[(size_t)b * H + h];
	}
	q->rel_far[li] = far;
	TRY(sallocT(q, &q->rel_dist[li], tab.size()));
	HIPCHK(hipMemcpy(q->rel_dist[li], tab.data(), tab.size() * sizeof(float), hipMemcpyHostToDevice));
	return YALM_OK;
}

static int create_seq(const yalm_seq_config *config, const yalm_seq_weights *w, yalm_stream s, Seq **out) {
	ARGCHK(config && w && w->layers && w->embed && w->final_norm && w->head && out, "yalm_seq_create: null argument");
	Seq *q = new Seq;
	q->c = *config;
	q->L.assign(w->layers, w->layers + config->n_layers);
	q->side_of.assign(config->n_layers, -1);
	for (int i = 0; i < config->n_layers; ++i) // second mixers follow the layers, with caches and states of their own
		if (q->L[i].side) {
			q->side_of[i] = (int)q->L.size();
			q->L.push_back(*q->L[i].side);
		}
	q->embed_norm = w->embed_norm;
	q->embed = w->embed;
	q->head = w->head;
	q->final_norm = w->final_norm;
	int rc = validate(q->c, q->L);
	if (rc != YALM_OK) {
		delete q;
		return rc;
	}
	auto fail = [&](int r) {
		destroy_seq(q);
		return r;
	};
#define STRY(expr)                                                                                                     \
	do {                                                                                                               \
		int r_ = (expr);                                                                                               \
		if (r_ != YALM_OK)                                                                                             \
			return fail(r_);                                                                                           \
	} while (0)
	if (s) {
		q->stream = reinterpret_cast<hipStream_t>(s);
	} else {
		if (hipStreamCreateWithFlags(&q->stream, hipStreamNonBlocking) != hipSuccess) {
			set_err("hipStreamCreateWithFlags failed");
			return fail(YALM_ERR_HIP);
		}
		q->own_stream = true;
	}
	const yalm_seq_config &c = q->c;
	const bool bf = c.weight_dtype == YALM_BF16;
	q->cap = std::min(c.max_tokens, (int)SEQ_PORTION_CAP);
	size_t bw = c.width, arena = 0;
	int zw = 1, max_e = 1, max_top = 1;
	for (const yalm_seq_layer &l : q->L) {
		zw = std::max(zw, in_rows(l));
		if (l.mixer == YALM_MIX_LATENT) {
			bw = std::max({bw, (size_t)l.heads * (l.dim + l.rot_dim), (size_t)l.heads * (l.kv_rank + l.rot_dim),
			               (size_t)l.heads * l.vdim, (size_t)l.q_rank});
		} else if (l.mixer == YALM_MIX_RGLRU) {
			bw = std::max(bw, (size_t)l.rec_width);
			arena += (size_t)l.rec_width + (size_t)(l.conv - 1) * l.rec_width;
		} else if (l.mixer == YALM_MIX_ATTN) {
			// with score mixing a portion's queries span the whole key row
			bw = std::max({bw, (size_t)l.heads * l.dim * (l.talk ? l.kv_heads : 1), (size_t)l.heads * l.vdim});
		} else if (l.mixer == YALM_MIX_SSM) {
			const size_t cc = (size_t)l.heads * l.vdim + 2 * (size_t)l.ssm_groups * l.ssm_state;
			bw = std::max({bw, cc, (size_t)2 * l.heads});
			arena += (size_t)l.heads * l.ssm_state * l.vdim + (size_t)(l.conv - 1) * cc;
		} else {
			const size_t cc = 2 * (size_t)l.kv_heads * l.dim + (size_t)l.heads * l.vdim;
			// beta and per-head decay, then (decay_rank) one decay per head and key channel
			bw = std::max({bw, cc, (size_t)l.heads * l.vdim, (size_t)2 * l.heads + (l.decay_rank > 0 ? (size_t)l.heads * l.dim : 0)});
			arena += (size_t)l.heads * l.dim * l.vdim + (size_t)(l.conv - 1) * cc;
		}
		if (l.ff_kind == YALM_FF_DENSE || l.ff_kind == YALM_FF_PLAIN)
			bw = std::max(bw, (size_t)l.ff);
		if (l.ff_kind == YALM_FF_MOE) {
			bw = std::max({bw, (size_t)l.top * l.ff, (size_t)l.top * c.width, (size_t)l.shared_ff});
			max_e = std::max(max_e, l.experts);
			max_top = std::max(max_top, l.top);
		}
	}
	q->bw = bw;
	q->zw = zw;
	const size_t cap = q->cap;
	STRY(sallocT(q, &q->st, 1));
	STRY(sallocT(q, &q->X, cap * c.width));
	STRY(sallocT(q, &q->Hn, cap * c.width));
	STRY(sallocT(q, &q->Y, cap * c.width));
	if (c.block_kind == YALM_BLOCK_PARALLEL)
		STRY(sallocT(q, &q->Y2, cap * c.width));
	q->Yout = q->Y;
	{
		bool own_ff_norm = false, sides = false;
		for (int i = 0; i < c.n_layers; ++i) {
			own_ff_norm |= c.block_kind == YALM_BLOCK_PARALLEL && q->L[i].norm2 && q->L[i].ff_kind != YALM_FF_NONE;
			sides |= q->side_of[i] >= 0;
		}
		if (own_ff_norm)
			STRY(sallocT(q, &q->Hn2, cap * c.width));
		if (sides)
			STRY(sallocT(q, &q->Y3, cap * c.width));
	}
	STRY(sallocT(q, &q->Z, cap * zw));
	for (int i = 0; i < 4; ++i)
		STRY(sallocT(q, &q->B[i], cap * bw));
	if (bf && pf_gemm_bf16)
		STRY(sallocT(q, &q->a16, cap * bw));
	STRY(sallocT(q, &q->tok, cap));
	STRY(sallocT(q, &q->want, cap));
	STRY(sallocT(q, &q->logits, (size_t)LOGIT_ROWS * c.vocab));
	STRY(sallocT(q, &q->idx, cap * max_top));
	STRY(sallocT(q, &q->wt, cap * max_top));
	STRY(sallocT(q, &q->sgate, cap));
	STRY(sallocT(q, &q->counts, max_e));
	STRY(sallocT(q, &q->lists, (size_t)max_e * cap));
	{
		int max_h = 1, max_rank = 4;
		for (const yalm_seq_layer &l : q->L)
			if (l.mixer == YALM_MIX_LATENT) {
				max_h = std::max(max_h, l.heads);
				max_rank = std::max(max_rank, l.kv_rank);
			}
		q->att_splits = std::max(1, std::min(32, cdiv(c.max_tokens, 2 * ATT_KT)));
		size_t part = (size_t)(4 * ATT_BR + GEMV_MAX_M * max_h) * q->att_splits * (att_rank4(max_rank) + 4);
		// attn: the keys a single token can see, split so that a workgroup walks one tile (up to 64 splits)
		q->attn_splits.assign(q->L.size(), 1);
		for (int i = 0; i < (int)q->L.size(); ++i) {
			const yalm_seq_layer &l = q->L[i];
			if (l.mixer != YALM_MIX_ATTN && !latent_direct(l))
				continue;
			const int span = l.mask_kind == YALM_MASK_CAUSAL ? c.max_tokens : std::min(c.max_tokens, l.mask_size + GEMV_MAX_M);
			q->attn_splits[i] = std::max(1, std::min(64, cdiv(span, SA_KT)));
			const int vd = l.mixer == YALM_MIX_ATTN ? l.vdim : std::max(l.kv_rank, l.vdim); // the attention's value size
			part = std::max(part, (size_t)GEMV_MAX_M * l.heads * q->attn_splits[i] * (att_rank4(vd) + 4));
		}
		STRY(sallocT(q, &q->att_part, part));
	}
	q->gen_cap = 1 << 16;
	STRY(sallocT(q, &q->gen_tokens, q->gen_cap));
	q->ln = c.norm_kind == YALM_NORM_LAYER;
	q->In = c.pre_norm ? q->Hn : q->X;
	q->Xbase = q->X;
	if (!c.pre_norm)
		STRY(sallocT(q, &q->Xalt, (size_t)c.width));
	// position frequencies 10000^(-2 i / width), evaluated in double
	if (c.pos_embed) {
		std::vector<float> f((c.width + 1) / 2);
		for (int i = 0; i < (c.width + 1) / 2; ++i)
			f[i] = (float)std::pow(10000.0, -2.0 * i / (double)c.width);
		STRY(sallocT(q, &q->inv_freq, f.size()));
		if (hipMemcpy(q->inv_freq, f.data(), f.size() * sizeof(float), hipMemcpyHostToDevice) != hipSuccess) {
			set_err("hipMemcpy of the position frequencies failed");
			return fail(YALM_ERR_HIP);
		}
	}
	q->arena_floats = arena;
	STRY(sallocT(q, &q->arena, arena));
	const int NL = (int)q->L.size();
	q->cache.assign(NL, nullptr);
	q->S.assign(NL, nullptr);
	q->conv.assign(NL, nullptr);
	q->vcache.assign(NL, nullptr);
	q->rot_freq.assign(NL, nullptr);
	q->rot_mag.assign(NL, 1.0f);
	q->rel_dist.assign(NL, nullptr);
	q->rel_far.assign(NL, 0);
	size_t off = 0;
	for (int i = 0; i < NL; ++i) {
		const yalm_seq_layer &l = q->L[i];
		if (latent_direct(l)) {
			STRY(salloc(q, &q->cache[i], (size_t)c.max_tokens * (l.kv_rank + l.rot_dim) * (bf ? 2 : 4)));
			q->vcache[i] = q->cache[i];
			STRY(attn_setup(q, i));
		} else if (l.mixer == YALM_MIX_LATENT) {
			if (l.kv_from < 0)
				STRY(salloc(q, &q->cache[i], (size_t)c.max_tokens * l.kv_rank * (bf ? 2 : 4)));
			STRY(bf ? att_attr_ct<uint16_t>(l.kv_rank) : att_attr_ct<float>(l.kv_rank));
		} else if (l.mixer == YALM_MIX_ATTN) {
			STRY(salloc(q, &q->cache[i], (size_t)c.max_tokens * l.kv_heads * l.dim * (bf ? 2 : 4)));
			STRY(salloc(q, &q->vcache[i], (size_t)c.max_tokens * l.kv_heads * l.vdim * (bf ? 2 : 4)));
			STRY(attn_setup(q, i));
			STRY(rel_setup(q, i));
		} else if (l.mixer == YALM_MIX_RGLRU) {
			q->S[i] = q->arena + off;
			off += l.rec_width;
			q->conv[i] = q->arena + off;
			off += (size_t)(l.conv - 1) * l.rec_width;
		} else if (l.mixer == YALM_MIX_SSM) {
			const size_t cc = (size_t)l.heads * l.vdim + 2 * (size_t)l.ssm_groups * l.ssm_state;
			q->S[i] = q->arena + off;
			off += (size_t)l.heads * l.ssm_state * l.vdim;
			q->conv[i] = q->arena + off;
			off += (size_t)(l.conv - 1) * cc;
		} else {
			const size_t cc = 2 * (size_t)l.kv_heads * l.dim + (size_t)l.heads * l.vdim;
			q->S[i] = q->arena + off;
			off += (size_t)l.heads * l.dim * l.vdim;
			q->conv[i] = q->arena + off;
			off += (size_t)(l.conv - 1) * cc;
		}
	}
	{ // expansion buffers: the most positions a portion's rows see, over the layers that expand
		size_t rows = 0, nc = 0, nkv = 0, nk = 0, nv = 0;
		for (const yalm_seq_layer &l : q->L)
			if (latent_direct(l) && l.w_ukv) {
				const size_t span = l.mask_kind == YALM_MASK_CAUSAL ? (size_t)c.max_tokens : (size_t)l.mask_size + q->cap;
				rows = std::max(rows, std::min((size_t)c.max_tokens, span));
				nc = std::max(nc, (size_t)l.kv_rank);
				nkv = std::max(nkv, (size_t)l.heads * (l.dim + l.vdim));
				nk = std::max(nk, (size_t)l.heads * (l.dim + l.rot_dim));
				nv = std::max(nv, (size_t)l.heads * l.vdim);
			}
		if (rows) {
			q->ex_rows = (int)rows;
			if (bf)
				STRY(sallocT(q, &q->ex_c, rows * nc));
			STRY(sallocT(q, &q->ex_kv, rows * nkv));
			STRY(salloc(q, &q->ex_k, rows * nk * (bf ? 2 : 4)));
			STRY(salloc(q, &q->ex_v, rows * nv * (bf ? 2 : 4)));
		}
	}
	for (int i = 0; i < c.n_layers; ++i)
		if (q->L[i].mixer == YALM_MIX_LATENT && q->L[i].q_rank > 0 && q->L[i].kv_from >= 0)
			q->cache[i] = q->cache[q->L[i].kv_from];
#undef STRY
	*out = q;
	return YALM_OK;
}

extern "C" int yalm_seq_create(const yalm_seq_config *config, const yalm_seq_weights *weights, yalm_stream s,
                               yalm_seq *out) {
	Seq *q = nullptr;
	TRY(create_seq(config, weights, s, &q));
	*out = q;
	return YALM_OK;
}

extern "C" int yalm_seq_destroy(yalm_seq q) {
	if (!q)
		return YALM_OK;
	(void)hipStreamSynchronize(q->stream);
	destroy_seq(q);
	return YALM_OK;
}

extern "C" int yalm_seq_reset(yalm_seq q) {
	ARGCHK(q, "yalm_seq_reset: null decoder");
	if (q->arena_floats) {
		seq_fill_float_kernel<<<256, 256, 0, q->stream>>>(q->arena, q->arena_floats, 0.0f);
		HIPCHK(hipGetLastError());
	}
	q->host_pos = 0;
	return YALM_OK;
}

extern "C" int yalm_seq_pos(yalm_seq q, int *pos) {
	ARGCHK(q && pos, "yalm_seq_pos: null argument");
	*pos = q->host_pos;
	return YALM_OK;
}

// ------------------------------------------------------------------ launches
template <class WT>
static int gemm_t(Seq *q, const GemmArgs &a, int batches, int max_m) {
	const bool glu = a.W2 != nullptr;
	if (max_m <= GEMV_MAX_M) {
		const dim3 g(cdiv(a.N, SEQ_THREADS / 64), 1, batches);
		if (glu)
			seq_gemv_kernel<WT, true><<<g, SEQ_THREADS, 0, q->stream>>>(a);
		else
			seq_gemv_kernel<WT, false><<<g, SEQ_THREADS, 0, q->stream>>>(a);
	} else if (WT::BYTES == 2 && max_m > GT_BM) {
		const dim3 g(cdiv(a.N, GB_BN), cdiv(max_m, GB_BM), batches);
		if (glu)
			seq_gemm_bf16_kernel<true><<<g, SEQ_THREADS, 0, q->stream>>>(a);
		else
			seq_gemm_bf16_kernel<false><<<g, SEQ_THREADS, 0, q->stream>>>(a);
	} else {
		const dim3 g(cdiv(a.N, GT_BN), cdiv(max_m, GT_BM), batches);
		if (glu)
			seq_gemm_kernel<WT, true><<<g, SEQ_THREADS, 0, q->stream>>>(a);
		else
			seq_gemm_kernel<WT, false><<<g, SEQ_THREADS, 0, q->stream>>>(a);
	}
	HIPCHK(hipGetLastError());
	return YALM_OK;
}
// f32w: the matrices are f32 whatever the model's weight type (the recurrence's gates)
static int gemm(Seq *q, const GemmArgs &a, int batches = 1, int max_m = -1, bool f32w = false) {
	if (max_m < 0)
		max_m = a.M;
	if (f32w || q->c.weight_dtype == YALM_F32)
		return gemm_t<WF32>(q, a, batches, max_m);
	// plain products of long portions whose shape fits the large-tile GEMM of the prefill unit;
	// output columns past the last multiple of 128 (a few gate rows closing an input projection)
	// run on the general kernel as a second, narrow product
	const bool pair = a.W2 != nullptr && (a.epi == EPI_GLU_GELU || a.epi == EPI_GLU_CLAMP || a.epi == EPI_GLU_SILU) && !a.bias;
	const bool single = !a.W2 && (a.epi == EPI_NONE || a.epi == EPI_GELU || a.epi == EPI_RELU2);
	const int act1 = a.epi == EPI_GELU ? 1 : (a.epi == EPI_RELU2 ? 2 : 0); // the large-tile door's activation
	const int n_big = pair ? (a.N % 64 == 0 ? a.N : 0) : (single ? a.N & ~127 : 0);
	if (q->a16 && batches == 1 && max_m >= 2 * GB_BM && !a.rows && !a.w_sel && a.z_split == 0 && a.ldw == a.K &&
	    a.K % 64 == 0 && n_big > 0 && (a.N - n_big <= 64 || (!pair && a.N - n_big < 128))) {
		const size_t n8 = (size_t)a.M * (a.K / 8);
		seq_to_bf16_kernel<<<(unsigned)std::min<size_t>((n8 + SEQ_THREADS - 1) / SEQ_THREADS, 4096), SEQ_THREADS, 0,
		                     q->stream>>>(a.A, a.lda, a.M, a.K, q->a16);
		HIPCHK(hipGetLastError());
		const int rc =
		    pair ? pf_gemm_glu_bf16(q->a16, a.K, a.M, a.K, (const uint16_t *)a.W, (const uint16_t *)a.W2, a.N, a.C, a.ldc,
		                            a.epi == EPI_GLU_GELU ? 1 : (a.epi == EPI_GLU_CLAMP ? 2 : 3), a.limit, q->stream)
		         : pf_gemm_bf16(q->a16, a.K, a.M, a.K, (const uint16_t *)a.W, n_big, a.C, a.ldc, a.bias,
		                        act1, q->stream);
		if (rc == YALM_OK && !pair && n_big < a.N && a.N >= 128) {
			// the last 128 columns as one more large tile: it computes the columns below n_big a
			// second time (the same kernel on the same operands: the same values) and the tail
			const int c0 = a.N - 128;
			const int rc2 = pf_gemm_bf16(q->a16, a.K, a.M, a.K, (const uint16_t *)a.W + (size_t)c0 * a.ldw, 128, a.C + c0,
			                             a.ldc, a.bias ? a.bias + c0 : nullptr, act1, q->stream);
			if (rc2 != YALM_ERR_UNSUPPORTED)
				return rc2;
		}
		if (rc == YALM_OK && n_big < a.N) {
			GemmArgs t = a;
			t.W = (const uint16_t *)a.W + (size_t)n_big * a.ldw;
			t.C = a.C + n_big;
			t.bias = a.bias ? a.bias + n_big : nullptr;
			t.N = a.N - n_big;
			return gemm_t<WBF16>(q, t, 1, max_m);
		}
		if (rc != YALM_ERR_UNSUPPORTED)
			return rc;
	}
	return gemm_t<WBF16>(q, a, batches, max_m);
}
static GemmArgs plain(const float *A, int lda, const void *W, int ldw, float *C, int ldc, int M, int N, int K) {
	GemmArgs a;
	a.A = A;
	a.lda = lda;
	a.W = W;
	a.ldw = ldw;
	a.C = C;
	a.ldc = ldc;
	a.M = M;
	a.N = N;
	a.K = K;
	return a;
}

template <class CT>
static int attn_t(Seq *q, const float *Qa, const void *cache, int rank, int H, int n, float scale, float *ctx) {
	const int NR = n * H;
	if (sizeof(CT) == 2 && NR > 4 * ATT_BR) { // portions over a bf16 cache: the MFMA form
		const dim3 gm(cdiv(NR, ATM_BR));
		const int ks = cdiv(rank, 32);
#define ATM_LAUNCH(KS)                                                                                                 \
	seq_latent_attn_mfma_kernel<KS><<<gm, SEQ_THREADS, 0, q->stream>>>(Qa, (const uint16_t *)cache, rank, H, NR, scale,   \
	                                                                  q->st, ctx)
		if (ks <= 1) ATM_LAUNCH(1);
		else if (ks <= 2) ATM_LAUNCH(2);
		else if (ks <= 4) ATM_LAUNCH(4);
		else ATM_LAUNCH(8);
#undef ATM_LAUNCH
		HIPCHK(hipGetLastError());
		return YALM_OK;
	}
	// few rows (single tokens, short portions): the visible keys are split over workgroups
	const int S = NR <= 4 * ATT_BR ? q->att_splits : 1;
	const dim3 g(cdiv(NR, ATT_BR), S);
	const size_t lds = att_lds_bytes(rank);
	const int na = cdiv(att_rank4(rank), 64);
#define ATT_LAUNCH(NA)                                                                                                 \
	seq_latent_attn_kernel<CT, NA><<<g, SEQ_THREADS, lds, q->stream>>>(Qa, (const CT *)cache, rank, H, NR, scale, q->st, ctx, \
	                                                                  q->att_part)
	if (na <= 1) ATT_LAUNCH(1);
	else if (na <= 2) ATT_LAUNCH(2);
	else ATT_LAUNCH(4);
#undef ATT_LAUNCH
	if (S > 1)
		seq_latent_merge_kernel<<<NR, SEQ_THREADS, 0, q->stream>>>(q->att_part, S, rank, ctx);
	HIPCHK(hipGetLastError());
	return YALM_OK;
}

static int mixer_latent(Seq *q, int li, int n) {
	const yalm_seq_layer &l = q->L[li];
	const yalm_seq_config &c = q->c;
	const bool bf = c.weight_dtype == YALM_BF16;
	const int zin = in_rows(l), H = l.heads, D = l.dim, V = l.vdim, rk = l.kv_rank;
	float *cq = q->B[0], *qh = q->B[1], *qa = q->B[2], *ctx = q->B[3];
	TRY(gemm(q, plain(q->In, c.width, l.w_in, c.width, q->Z, zin, n, zin, c.width)));
	if (l.kv_from >= 0)
		seq_norm_kernel<float><<<n, SEQ_THREADS, 0, q->stream>>>(q->Z, zin, l.q_norm, c.norm_eps, l.q_rank, cq, l.q_rank,
		                                                         nullptr, q->st, 0);
	else if (bf)
		seq_norm2_kernel<uint16_t><<<dim3(n, 2), SEQ_THREADS, 0, q->stream>>>(q->Z, zin, l.q_rank, l.q_norm, cq, rk, l.kv_norm,
		                                                                    (uint16_t *)q->cache[li], c.norm_eps, q->st);
	else
		seq_norm2_kernel<float><<<dim3(n, 2), SEQ_THREADS, 0, q->stream>>>(q->Z, zin, l.q_rank, l.q_norm, cq, rk, l.kv_norm,
		                                                                 (float *)q->cache[li], c.norm_eps, q->st);
	HIPCHK(hipGetLastError());
	TRY(gemm(q, plain(cq, l.q_rank, l.w_uq, l.q_rank, qh, H * D, n, H * D, l.q_rank)));
	{ // q~[h] = W_uk[h]^T q[h]: per head [n][dim] x [rank][dim]^T
		GemmArgs a = plain(qh, H * D, l.w_ukt, D, qa, H * rk, n, rk, D);
		a.a_bs = D;
		a.w_bs = (long)rk * D;
		a.c_bs = rk;
		TRY(gemm(q, a, H));
	}
	TRY(bf ? attn_t<uint16_t>(q, qa, q->cache[li], rk, H, n, l.attn_scale, ctx)
	       : attn_t<float>(q, qa, q->cache[li], rk, H, n, l.attn_scale, ctx));
	{ // o[h] = W_uv[h] ctx[h]
		GemmArgs a = plain(ctx, H * rk, l.w_uv, rk, qh, H * V, n, V, rk);
		a.a_bs = rk;
		a.w_bs = (long)V * rk;
		a.c_bs = V;
		TRY(gemm(q, a, H));
	}
	return gemm(q, plain(qh, H * V, l.w_o, H * V, q->Yout, c.width, n, c.width, H * V));
}

static int conv_launch(Seq *q, const float *Z, int ldz, int col0, int C, int taps, const float *w, const float *bias,
                       int silu, float *state, float *out, int n) {
	if (n <= SEQ_CONV_STEP_T) {
		seq_conv_step_kernel<<<cdiv(C, SEQ_THREADS), SEQ_THREADS, 0, q->stream>>>(Z, ldz, col0, C, taps, w, bias, silu, state,
		                                                                          out, C, n);
	} else {
		seq_conv_kernel<<<dim3(cdiv(C, SEQ_THREADS), n), SEQ_THREADS, 0, q->stream>>>(Z, ldz, col0, C, taps, w, bias, silu,
		                                                                              state, out, C, n);
		if (taps > 1)
			seq_conv_state_kernel<<<cdiv(C, SEQ_THREADS), SEQ_THREADS, 0, q->stream>>>(Z, ldz, col0, C, taps, state, n);
	}
	HIPCHK(hipGetLastError());
	return YALM_OK;
}

static int mixer_rglru(Seq *q, int li, int n) {
	const yalm_seq_layer &l = q->L[li];
	const yalm_seq_config &c = q->c;
	const int W = l.rec_width, bs = W / l.blocks;
	float *u = q->B[0], *r = q->B[1], *ig = q->B[2], *so = q->B[3];
	{
		GemmArgs a = plain(q->In, c.width, l.w_in, c.width, q->Z, 2 * W, n, 2 * W, c.width);
		a.bias = l.in_bias;
		TRY(gemm(q, a));
	}
	TRY(conv_launch(q, q->Z, 2 * W, W, W, l.conv, l.conv_w, l.conv_b, 0, q->conv[li], u, n));
	{ // both block-diagonal gates in f32, one launch: batches [0, blocks) recurrence gate, the rest input gate
		GemmArgs a = plain(u, W, l.gate_a, bs, r, W, n, bs, bs);
		a.a_bs = bs;
		a.w_bs = (long)bs * bs;
		a.c_bs = bs;
		a.bias = l.gate_a_b;
		a.bias_bs = bs;
		a.epi = EPI_SIGMOID;
		a.z_split = l.blocks;
		a.W_b = l.gate_i;
		a.C_b = ig;
		a.bias_b = l.gate_i_b;
		TRY(gemm(q, a, 2 * l.blocks, -1, true));
	}
	if (n <= GEMV_MAX_M) {
		seq_rglru_scan_kernel<<<cdiv(W, SEQ_THREADS), SEQ_THREADS, 0, q->stream>>>(r, ig, u, W, q->Z, 2 * W, l.lam,
		                                                                           q->S[li], so, n);
	} else {
		seq_rglru_coef_kernel<<<dim3(cdiv(W, SEQ_THREADS), n), SEQ_THREADS, 0, q->stream>>>(r, ig, u, W, q->Z, 2 * W, l.lam,
		                                                                                 n);
		seq_rglru_walk_kernel<<<cdiv(W, SEQ_THREADS), SEQ_THREADS, 0, q->stream>>>(r, ig, u, W, q->S[li], so, n);
	}
	HIPCHK(hipGetLastError());
	return gemm(q, plain(so, W, l.w_o, W, q->Yout, c.width, n, c.width, W));
}

// The recurrence kernel over a portion: the gated delta rule (ssm = false; gv: one decay per head
// and key channel) or the state-space walk (ssm = true). K: key / state size, P: value size.
static int delta_launch(Seq *q, const float *qkv, int ldq, int qo, int ko, int vo, int KH, int K, int H, int P,
                        const float *bg, const float *gv, const float *dskip, float *state, float *o, int n, bool ssm) {
	// lanes per column of the state: 16 (twice the workgroups, half the rows per lane) but for the smallest keys
	const int lpc = K <= 32 ? 8 : 16;
	const dim3 g(cdiv(P, SEQ_THREADS / lpc), H);
#define DELTA_LAUNCH(RR, TC, LPC)                                                                                      \
	do {                                                                                                               \
		if (ssm)                                                                                                       \
			seq_delta_kernel<RR, TC, true, false, LPC><<<g, SEQ_THREADS, 0, q->stream>>>(                              \
			    qkv, ldq, qo, ko, vo, KH, K, H, P, bg, nullptr, dskip, state, o, n);                                   \
		else if (gv)                                                                                                   \
			seq_delta_kernel<RR, TC, false, true, LPC><<<g, SEQ_THREADS, 0, q->stream>>>(                              \
			    qkv, ldq, qo, ko, vo, KH, K, H, P, bg, gv, nullptr, state, o, n);                                      \
		else                                                                                                           \
			seq_delta_kernel<RR, TC, false, false, LPC><<<g, SEQ_THREADS, 0, q->stream>>>(                             \
			    qkv, ldq, qo, ko, vo, KH, K, H, P, bg, nullptr, nullptr, state, o, n);                                 \
	} while (0)
	if (K <= 32) DELTA_LAUNCH(4, 16, 8);
	else if (K <= 64) DELTA_LAUNCH(4, 16, 16);
	else if (K <= 128) DELTA_LAUNCH(8, 16, 16);
	else DELTA_LAUNCH(16, 8, 16);
#undef DELTA_LAUNCH
	HIPCHK(hipGetLastError());
	return YALM_OK;
}

static int mixer_delta(Seq *q, int li, int n) {
	const yalm_seq_layer &l = q->L[li];
	const yalm_seq_config &c = q->c;
	const int H = l.heads, KH = l.kv_heads, D = l.dim, V = l.vdim;
	const int CQ = KH * D, CV = H * V, cc = 2 * CQ + CV, zin = in_rows(l);
	const int gcol = cc, bcol = cc + (l.gate_rank > 0 ? l.gate_rank : CV), acol = bcol + H;
	float *qkv = q->B[0], *bg = q->B[1], *o = q->B[2], *on = q->B[3];
	// one decay per head and key channel: its inputs, then the decays, follow the [n][2 H] factors
	float *gv = l.decay_rank > 0 ? bg + (size_t)n * 2 * H : nullptr;
	TRY(gemm(q, plain(q->In, c.width, l.w_in, c.width, q->Z, zin, n, zin, c.width)));
	TRY(conv_launch(q, q->Z, zin, 0, cc, l.conv, l.conv_w, nullptr, 1, q->conv[li], qkv, n));
	if (gv) // the low-rank decay's second factor
		TRY(gemm(q, plain(q->Z + acol, zin, l.w_a2, l.decay_rank, gv, H * D, n, H * D, l.decay_rank)));
	seq_delta_prep_kernel<<<n, SEQ_THREADS, 0, q->stream>>>(qkv, cc, KH, D, q->Z, zin, bcol, acol, H, l.a_log, l.dt_bias,
	                                                        bg, gv);
	HIPCHK(hipGetLastError());
	const float *gl = q->Z;
	int ldg = zin, gc = gcol;
	if (l.gate_rank > 0) { // the low-rank gate's second factor; the gated read-out then overwrites its logits
		TRY(gemm(q, plain(q->Z + gcol, zin, l.w_g2, l.gate_rank, on, CV, n, CV, l.gate_rank)));
		gl = on;
		ldg = CV;
		gc = 0;
	}
	TRY(delta_launch(q, qkv, cc, 0, CQ, 2 * CQ, KH, D, H, V, bg, gv, nullptr, q->S[li], o, n, false));
	seq_delta_out_kernel<<<n, SEQ_THREADS, 0, q->stream>>>(o, H, V, l.out_norm, c.norm_eps, gl, ldg, gc, on,
	                                                       l.gate_act == YALM_GATE_SIGMOID);
	HIPCHK(hipGetLastError());
	return gemm(q, plain(on, CV, l.w_o, CV, q->Yout, c.width, n, c.width, CV));
}

// Selective state-space layer: one input projection (gate | x | B | C | step), the convolution
// with silu over x | B | C, per-head step sizes and decays, the recurrence (the delta rule's
// kernel in its state-space form: B as keys, C as queries, x as values), the gated result
// rms-normed in equal parts, the output projection.
static int mixer_ssm(Seq *q, int li, int n) {
	const yalm_seq_layer &l = q->L[li];
	const yalm_seq_config &c = q->c;
	const int H = l.heads, P = l.vdim, N = l.ssm_state, G = l.ssm_groups;
	const int inner = H * P, GN = G * N, cc = inner + 2 * GN, zin = in_rows(l);
	float *xbc = q->B[0], *bg = q->B[1], *y = q->B[2], *yn = q->B[3];
	TRY(gemm(q, plain(q->In, c.width, l.w_in, c.width, q->Z, zin, n, zin, c.width)));
	TRY(conv_launch(q, q->Z, zin, inner, cc, l.conv, l.conv_w, l.conv_b, 1, q->conv[li], xbc, n));
	seq_ssm_prep_kernel<<<cdiv(n * H, SEQ_THREADS), SEQ_THREADS, 0, q->stream>>>(q->Z, zin, inner + cc, H, l.a_log,
	                                                                            l.dt_bias, bg, n);
	HIPCHK(hipGetLastError());
	TRY(delta_launch(q, xbc, cc, inner + GN, inner, 0, G, N, H, P, bg, nullptr, l.d_skip, q->S[li], y, n, true));
	seq_gated_part_norm_kernel<<<dim3(n, l.norm_groups), SEQ_THREADS, 0, q->stream>>>(y, inner, l.norm_groups, q->Z, zin, 0,
	                                                                                  l.out_norm, c.norm_eps, yn);
	HIPCHK(hipGetLastError());
	return gemm(q, plain(yn, inner, l.w_o, inner, q->Yout, c.width, n, c.width, inner));
}

// ---- the closing norm of a single token, owed to the product that reads the stream next
static int add_norm(Seq *q, const float *wb, const float *w_next, int n, const yalm_seq_layer *moe);

static bool an_foldable(const Seq *q, int n) {
	return n == 1 && !q->c.pre_norm && !q->dump_on && q->Xalt && q->c.width % 8 == 0 && q->c.width <= 8 * 1024;
}
static int flush_norm(Seq *q, int n) {
	if (!q->pend_wb)
		return YALM_OK;
	const float *wb = q->pend_wb;
	q->pend_wb = nullptr;
	return add_norm(q, wb, nullptr, n, nullptr);
}
template <class WT>
static int gemv_an_t(Seq *q, const GemmArgs &a) {
	const int K = a.K, ki = cdiv(K, 1024);
	const dim3 g(cdiv(a.N, (SEQ_THREADS / 64) * GAN_RPW));
#define GA_LAUNCH(KI)                                                                                                  \
	seq_gemv_an_kernel<WT, KI><<<g, SEQ_THREADS, (size_t)K * sizeof(float), q->stream>>>(                              \
	    q->X, q->Y, q->pend_wb, q->c.norm_eps, (int)q->ln, K, q->X == q->Xbase ? q->Xalt : q->Xbase, a.W, a.N, a.C,    \
	    a.bias, a.epi)
	if (ki <= 1) GA_LAUNCH(1);
	else if (ki <= 2) GA_LAUNCH(2);
	else if (ki <= 4) GA_LAUNCH(4);
	else GA_LAUNCH(8);
#undef GA_LAUNCH
	HIPCHK(hipGetLastError());
	q->X = q->X == q->Xbase ? q->Xalt : q->Xbase; // the stream now lives in the other row
	q->In = q->X;
	q->pend_wb = nullptr;
	return YALM_OK;
}
// A product whose A operand is the sublayer input q->In. With a closing norm owed and a single
// token, the norm + residual sum run inside the product's kernel; else the norm first.
static int gemm_in(Seq *q, GemmArgs a) {
	if (q->pend_wb) {
		if (a.M == 1 && !a.W2 && (a.epi == EPI_NONE || a.epi == EPI_GELU) && a.ldw == a.K && a.K == q->c.width &&
		    (size_t)a.W % 16 == 0 && !a.rows && !a.w_sel && a.z_split == 0 && a.A == q->In)
			return q->c.weight_dtype == YALM_F32 ? gemv_an_t<WF32>(q, a) : gemv_an_t<WBF16>(q, a);
		TRY(flush_norm(q, a.M));
		a.A = q->In;
	}
	return gemm(q, a);
}

template <int KS>
static int attn_mfma_launch(Seq *q, const void *kc, const void *vc, int n, const AttnArgs &a, const float *Q,
                            const float *gate, float *ctx) {
	const int rep = a.H / a.G, HW = rep >= 4 ? 4 : (rep >= 2 ? 2 : 1), NT = cdiv(a.V, 16);
	const dim3 g(cdiv(n, 16 * (4 / HW)), a.G, cdiv(rep, HW));
	const uint16_t *Kc = (const uint16_t *)kc, *Vc = (const uint16_t *)vc;
#define SAM_LAUNCH(N)                                                                                                  \
	seq_attn_mfma_kernel<KS, N><<<g, SEQ_THREADS, 0, q->stream>>>(Q, Kc, Vc, a, n, HW, q->st, gate, ctx)
	if (NT <= 2) SAM_LAUNCH(2);
	else if (NT <= 4) SAM_LAUNCH(4);
	else SAM_LAUNCH(8);
#undef SAM_LAUNCH
	HIPCHK(hipGetLastError());
	return YALM_OK;
}

// kc / vc: the key and value rows, row = position (the layer's caches, or a portion's expanded
// keys and values whose pointer is moved back by the first row's position)
template <class CT>
static int attn_core_t(Seq *q, int li, int n, const AttnArgs &a, const float *Q, const float *gate, float *ctx,
                       const void *kc = nullptr, const void *vc = nullptr, const float *gate_e = nullptr, int ldg = 0) {
	if (!kc) {
		kc = q->cache[li];
		vc = q->vcache[li];
	}
	// gate_e: elementwise gate logits [t][ldg], head h's at column h V: applied by the split merge
	// where there is one, else by a launch of its own after the attention
	auto gate_after = [&]() {
		if (gate_e)
			seq_gate_mul_kernel<<<dim3(cdiv(a.H * a.V, SEQ_THREADS), n), SEQ_THREADS, 0, q->stream>>>(ctx, a.H * a.V, gate_e,
			                                                                                      ldg, 0, a.H * a.V);
		HIPCHK(hipGetLastError());
		return (int)YALM_OK;
	};
	const bool talk = a.talk != nullptr;
	const int DK = talk ? a.G * a.D : a.D;
	if (sizeof(CT) == 2 && n > GEMV_MAX_M && DK <= 512 && a.V <= 128) { // portions over bf16 caches: the MFMA form
		const int ks = cdiv(DK, 32);
		if (ks <= 1) TRY(attn_mfma_launch<1>(q, kc, vc, n, a, Q, gate, ctx));
		else if (ks <= 2) TRY(attn_mfma_launch<2>(q, kc, vc, n, a, Q, gate, ctx));
		else if (ks <= 4) TRY(attn_mfma_launch<4>(q, kc, vc, n, a, Q, gate, ctx));
		else if (ks <= 8) TRY(attn_mfma_launch<8>(q, kc, vc, n, a, Q, gate, ctx));
		else TRY(attn_mfma_launch<16>(q, kc, vc, n, a, Q, gate, ctx));
		return gate_after();
	}
	const int Hb = a.H / a.G, Gb = talk ? a.G : 1, V4n = (a.V + 3) / 4, D4 = (a.D + 3) & ~3;
	const CT *Kc = (const CT *)kc, *Vc = (const CT *)vc;
	const int rep = a.H / a.G;
	// many heads over few key/value heads: blocks of heads per workgroup, at most 16 heads each
	// and small enough that key splits x key/value heads x blocks fill half the chip
	int hb = rep;
	if (!talk)
		while (hb > 1 && (hb > 16 || (rep >= 8 && (long)q->attn_splits[li] * a.G * cdiv(rep, hb) < 128)))
			hb = (hb + 1) / 2;
	const int hz = cdiv(rep, hb);
	const size_t dec_lds = sa_decode_lds_bytes(hb, DK, talk ? a.H * a.D : 0, a.H);
	if (n == 1 && !a.q_mixed && dec_lds <= 96 * 1024) { // a decoded token: lanes read the cache rows themselves
		const int S = q->attn_splits[li];
		const dim3 g(S, a.G, hz);
		const size_t lds = dec_lds;
		const int na = cdiv(hb * V4n, SEQ_THREADS);
#define SD_LAUNCH(NA)                                                                                                  \
	do {                                                                                                               \
		static bool attr_set = false;                                                                                  \
		if (!attr_set) {                                                                                               \
			HIPCHK(hipFuncSetAttribute((const void *)seq_attn_decode_kernel<CT, NA>,                                    \
			                           hipFuncAttributeMaxDynamicSharedMemorySize, 128 * 1024));                       \
			attr_set = true;                                                                                           \
		}                                                                                                              \
		seq_attn_decode_kernel<CT, NA><<<g, SEQ_THREADS, lds, q->stream>>>(Q, Kc, Vc, a, q->st,                        \
		                                                                   S == 1 ? gate : nullptr, ctx, q->att_part, \
		                                                                   hz > 1 ? hb : 0);                           \
	} while (0)
		if (na <= 1) SD_LAUNCH(1);
		else if (na <= 2) SD_LAUNCH(2);
		else if (na <= 4) SD_LAUNCH(4);
		else if (na <= 8) SD_LAUNCH(8);
		else SD_LAUNCH(16);
#undef SD_LAUNCH
		if (S > 1) {
			seq_latent_merge_kernel<<<a.H, SEQ_THREADS, 0, q->stream>>>(q->att_part, S, a.V, ctx, gate, gate_e, ldg, a.H);
			HIPCHK(hipGetLastError());
			return YALM_OK;
		}
		return gate_after();
	}
	// tokens per workgroup: up to 32 rows, their queries within 64 KB of LDS
	int TQ = std::max(1, std::min(32 / Hb, n));
	while (TQ > 1 && (size_t)TQ * Hb * Gb * D4 * sizeof(float) > 64 * 1024)
		--TQ;
	const int R = TQ * Hb;
	const int S = n <= GEMV_MAX_M ? q->attn_splits[li] : 1;
	const dim3 g(cdiv(n, TQ), S, a.G);
	const size_t lds = sa_lds_bytes(R, Gb, a.D, a.V);
	if (lds > 160 * 1024 - 64) {
		set_err("attention: one token's queries of a key/value head's heads over the whole key row do not fit in LDS");
		return YALM_ERR_UNSUPPORTED;
	}
	const int na = cdiv(R * V4n, SEQ_THREADS);
#define SA_LAUNCH(NA)                                                                                                  \
	do {                                                                                                               \
		static bool attr_set = false; /* the kernel may use more dynamic LDS than the default limit */               \
		if (!attr_set) {                                                                                               \
			HIPCHK(hipFuncSetAttribute((const void *)seq_attn_kernel<CT, NA>, hipFuncAttributeMaxDynamicSharedMemorySize, \
			                           160 * 1024 - 64));                                                              \
			attr_set = true;                                                                                           \
		}                                                                                                              \
		seq_attn_kernel<CT, NA><<<g, SEQ_THREADS, lds, q->stream>>>(Q, Kc, Vc, a, n, TQ, q->st,                        \
		                                                            S == 1 ? gate : nullptr, ctx, q->att_part);        \
	} while (0)
	if (na <= 1) SA_LAUNCH(1);
	else if (na <= 2) SA_LAUNCH(2);
	else if (na <= 4) SA_LAUNCH(4);
	else if (na <= 8) SA_LAUNCH(8);
	else SA_LAUNCH(16);
#undef SA_LAUNCH
	if (S > 1) {
		seq_latent_merge_kernel<<<n * a.H, SEQ_THREADS, 0, q->stream>>>(q->att_part, S, a.V, ctx, gate, gate_e, ldg, a.H);
		HIPCHK(hipGetLastError());
		return YALM_OK;
	}
	return gate_after();
}

// Softmax attention over cached keys and values: one input projection (queries, keys, values,
// output gates), then rotation / norms / cache write, the attention itself, the output projection.
static int mixer_attn(Seq *q, int li, int n) {
	const yalm_seq_layer &l = q->L[li];
	const yalm_seq_config &c = q->c;
	const bool bf = c.weight_dtype == YALM_BF16;
	const int zin = in_rows(l), H = l.heads, V = l.vdim;
	float *Q = q->B[0], *gate = q->B[1], *ctx = q->B[2];
	// per-head gate rows are taken by the projection kernel itself; elementwise gate rows are
	// ordinary output columns of the input projection
	const int zmain = zin - (l.out_gate == 1 ? H : 0);
	{
		GemmArgs g = plain(q->In, c.width, l.w_in, c.width, q->Z, zin, n, zmain, c.width);
		g.bias = l.in_bias;
		TRY(gemm_in(q, g));
	}
	AttnArgs a;
	a.H = H;
	a.G = l.kv_heads;
	a.D = l.dim;
	a.V = V;
	a.mask_kind = l.mask_kind;
	a.mask_size = l.mask_size;
	a.qk_norm = l.qk_norm;
	a.v_norm = l.v_norm;
	a.sink = l.sink;
	a.sink_w = l.sink_w;
	a.KL = l.kv_heads * l.dim;
	a.VL = l.kv_heads * l.vdim;
	a.out_gate = l.out_gate == 1;
	a.rot_dims = l.rot_dims;
	a.rot_mag = q->rot_mag[li];
	a.rot_freq = q->rot_freq[li];
	a.scale = l.attn_scale;
	a.q_w = l.q_norm;
	a.k_w = l.kv_norm;
	a.temp = l.head_temp;
	a.talk = l.talk;
	a.rel_dist = q->rel_dist[li];
	a.rel_far = q->rel_far[li];
	a.q_temp_coef = l.q_temp_coef;
	a.q_temp_every = l.q_temp_every;
	a.eps = c.norm_eps;
	// portions: the projection kernel (one workgroup per token) mixes the queries itself
	a.q_mixed = l.talk && n > GEMV_MAX_M ? 1 : 0;
	const size_t rot_lds = ((size_t)std::max(l.rot_dims, 2) + (a.q_mixed ? (size_t)H * l.dim : 0)) * sizeof(float);
	// a few tokens: their head jobs spread over several workgroups
	const int jobs = H + 2 * l.kv_heads + (a.out_gate ? H : 0);
	const dim3 pg(n, n <= GEMV_MAX_M ? cdiv(jobs, SEQ_THREADS / 64) : 1);
	const float *gbias = l.in_bias && a.out_gate ? l.in_bias + zmain : nullptr;
	if (bf)
		seq_attn_prep_kernel<uint16_t><<<pg, SEQ_THREADS, rot_lds, q->stream>>>(
		    q->Z, zin, a, q->st, Q, (uint16_t *)q->cache[li], (uint16_t *)q->vcache[li], gate, q->In, c.width,
		    (const uint16_t *)l.w_in + (size_t)zmain * c.width, gbias);
	else
		seq_attn_prep_kernel<float><<<pg, SEQ_THREADS, rot_lds, q->stream>>>(
		    q->Z, zin, a, q->st, Q, (float *)q->cache[li], (float *)q->vcache[li], gate, q->In, c.width,
		    (const float *)l.w_in + (size_t)zmain * c.width, gbias);
	HIPCHK(hipGetLastError());
	const float *gp = a.out_gate ? gate : nullptr;
	const float *ge = l.out_gate == 2 ? q->Z + (zin - H * V) : nullptr; // elementwise gate logits close the Z rows
	TRY(bf ? attn_core_t<uint16_t>(q, li, n, a, Q, gp, ctx, nullptr, nullptr, ge, zin)
	       : attn_core_t<float>(q, li, n, a, Q, gp, ctx, nullptr, nullptr, ge, zin));
	GemmArgs o = plain(ctx, H * V, l.w_o, H * V, q->Yout, c.width, n, c.width, H * V);
	o.bias = l.o_bias;
	return gemm(q, o);
}

// Latent attention with directly projected queries, a rotated key part shared by all heads, a
// mask and a sink. With k_j = W_uk c_j and v_j = W_uv c_j: q.k_j = (W_uk^T q).c_j and sum_j p_j
// v_j = W_uv sum_j p_j c_j, so head h attends with the query [W_uk[h]^T q_plain | q_rot] over
// the cache rows [c_j | k_rot_j] themselves and sums their first kv_rank entries: the softmax-
// attention kernels with one key/value head, key size kv_rank + rot_dim, value size kv_rank,
// the value rows aliasing the key rows.
// Do the f32 FMA attention tiles fit in LDS for n tokens of H heads over G key/value heads?
static bool attn_fma_fits(int H, int G, int D, int V, int n) {
	const int Hb = H / G, D4 = (D + 3) & ~3;
	int TQ = std::max(1, std::min(32 / std::max(Hb, 1), n));
	while (TQ > 1 && (size_t)TQ * Hb * D4 * sizeof(float) > 64 * 1024)
		--TQ;
	return sa_lds_bytes(TQ * Hb, 1, D, V) <= 160 * 1024 - 64;
}

static int mixer_latent_direct(Seq *q, int li, int n) {
	const yalm_seq_layer &l = q->L[li];
	const yalm_seq_config &c = q->c;
	const bool bf = c.weight_dtype == YALM_BF16;
	const int zin = in_rows(l), H = l.heads, D = l.dim, R = l.rot_dim, V = l.vdim, rk = l.kv_rank, KR = rk + R;
	float *qp = q->B[0], *qa = q->B[1], *ctx = q->B[2], *oh = q->B[3];
	const void *w_uv = l.w_uv ? l.w_uv : (const char *)l.w_ukv + (size_t)H * D * rk * (bf ? 2 : 4);
	// Portions expand the latents they see into per-head keys and values (one product with the
	// stacked up-projections) and attend with ordinary heads of dim + rot_dim / vdim entries:
	// fewer multiply-adds per (query, key) pair than over the latent (2 kv_rank + rot_dim), and
	// head sizes the matrix-core attention takes. Single tokens and short portions attend over
	// the latent itself, unless its rows are too long for the f32 tiles.
	const int klo = attn_first_key(l.mask_kind, l.mask_size, q->cur_pos), rows = q->cur_pos + n - klo;
	const bool absorbed_ok = n == 1 || (bf && n > GEMV_MAX_M && KR <= 512 && rk <= 128) || attn_fma_fits(H, 1, KR, rk, n);
	const bool expand = l.w_ukv && n > 1 && rows <= q->ex_rows && (n >= 32 || !absorbed_ok);
	TRY(gemm(q, plain(q->In, c.width, l.w_in, c.width, q->Z, zin, n, zin, c.width)));
	const size_t rot_lds = (size_t)std::max(l.rot_dims, 2) * sizeof(float);
	const dim3 pg(n, n <= GEMV_MAX_M ? 4 : 1); // a few tokens: each token's work spread over four workgroups
	if (bf)
		seq_latent_prep_kernel<uint16_t><<<pg, SEQ_THREADS, rot_lds, q->stream>>>(
		    q->Z, zin, H, D, R, rk, l.rot_dims, q->rot_freq[li], l.kv_norm, c.norm_eps, l.attn_scale, q->st, qp, qa,
		    (uint16_t *)q->cache[li], (int)expand);
	else
		seq_latent_prep_kernel<float><<<pg, SEQ_THREADS, rot_lds, q->stream>>>(
		    q->Z, zin, H, D, R, rk, l.rot_dims, q->rot_freq[li], l.kv_norm, c.norm_eps, l.attn_scale, q->st, qp, qa,
		    (float *)q->cache[li], (int)expand);
	HIPCHK(hipGetLastError());
	AttnArgs a;
	a.H = H;
	a.mask_kind = l.mask_kind;
	a.mask_size = l.mask_size;
	a.qk_norm = YALM_QK_NONE;
	a.v_norm = 0;
	a.sink = l.sink;
	a.sink_w = l.sink_w;
	a.out_gate = 0;
	a.rot_dims = 0;
	a.rot_mag = 1.0f;
	a.rot_freq = nullptr;
	a.scale = l.attn_scale;
	a.q_w = a.k_w = a.temp = a.talk = nullptr;
	a.eps = c.norm_eps;
	a.q_mixed = 0;
	if (expand) {
		const int QH = D + R, NKV = H * (D + V);
		const float *lat;
		int ldl;
		if (bf) { // the cached rows as the product's f32 operand
			seq_cache_rows_f32_kernel<<<rows, SEQ_THREADS, 0, q->stream>>>((const uint16_t *)q->cache[li], KR, klo, rk, q->ex_c);
			HIPCHK(hipGetLastError());
			lat = q->ex_c;
			ldl = rk;
		} else {
			lat = (const float *)q->cache[li] + (size_t)klo * KR;
			ldl = KR;
		}
		TRY(gemm(q, plain(lat, ldl, l.w_ukv, rk, q->ex_kv, NKV, rows, NKV, rk)));
		if (bf)
			seq_latent_expand_kernel<uint16_t><<<rows, SEQ_THREADS, 0, q->stream>>>(
			    q->ex_kv, (const uint16_t *)q->cache[li], klo, H, D, R, V, rk, (uint16_t *)q->ex_k, (uint16_t *)q->ex_v);
		else
			seq_latent_expand_kernel<float><<<rows, SEQ_THREADS, 0, q->stream>>>(
			    q->ex_kv, (const float *)q->cache[li], klo, H, D, R, V, rk, (float *)q->ex_k, (float *)q->ex_v);
		HIPCHK(hipGetLastError());
		a.G = H;
		a.D = QH;
		a.V = V;
		a.KL = H * QH;
		a.VL = H * V;
		// the attention kernels index rows by position: row klo is the buffers' first
		const size_t eb = bf ? 2 : 4;
		const void *kc = (const char *)q->ex_k - (size_t)klo * a.KL * eb;
		const void *vc = (const char *)q->ex_v - (size_t)klo * a.VL * eb;
		TRY(bf ? attn_core_t<uint16_t>(q, li, n, a, qa, nullptr, oh, kc, vc)
		       : attn_core_t<float>(q, li, n, a, qa, nullptr, oh, kc, vc));
	} else {
		{ // columns [0, kv_rank) of head h's query: W_uk[h]^T q_plain[h], per head [n][dim] x [rank][dim]^T
			GemmArgs g = plain(qp, H * D, l.w_ukt, D, qa, H * KR, n, rk, D);
			g.a_bs = D;
			g.w_bs = (long)rk * D;
			g.c_bs = KR;
			TRY(gemm(q, g, H));
		}
		a.G = 1;
		a.D = KR;
		a.V = rk;
		a.KL = KR;
		a.VL = KR;
		TRY(bf ? attn_core_t<uint16_t>(q, li, n, a, qa, nullptr, ctx) : attn_core_t<float>(q, li, n, a, qa, nullptr, ctx));
		{ // o[h] = W_uv[h] ctx[h]
			GemmArgs b = plain(ctx, H * rk, w_uv, rk, oh, H * V, n, V, rk);
			b.a_bs = rk;
			b.w_bs = (long)V * rk;
			b.c_bs = V;
			TRY(gemm(q, b, H));
		}
	}
	GemmArgs o = plain(oh, H * V, l.w_o, H * V, q->Yout, c.width, n, c.width, H * V);
	o.bias = l.o_bias;
	return gemm(q, o);
}

// w_down gelu(w_up x)
static int ff_plain(Seq *q, int li, int n, float *out) {
	const yalm_seq_layer &l = q->L[li];
	const yalm_seq_config &c = q->c;
	GemmArgs a = plain(q->In, c.width, l.w_up, c.width, q->B[0], l.ff, n, l.ff, c.width);
	a.epi = l.ff_act == YALM_ACT_RELU2 ? EPI_RELU2 : EPI_GELU;
	TRY(gemm_in(q, a));
	return gemm(q, plain(q->B[0], l.ff, l.w_down, l.ff, out, c.width, n, c.width, l.ff));
}

// the epilogue of a gated pair: the layer's ff_act, or the kind's own form
static int glu_epi(const yalm_seq_layer &l, int dflt) {
	switch (l.ff_act) {
	case YALM_ACT_GELU: return EPI_GLU_GELU;
	case YALM_ACT_CLAMP: return EPI_GLU_CLAMP;
	case YALM_ACT_SILU: return EPI_GLU_SILU;
	default: return dflt;
	}
}

static int ff_dense(Seq *q, int li, int n, float *out) {
	const yalm_seq_layer &l = q->L[li];
	const yalm_seq_config &c = q->c;
	GemmArgs a = plain(q->In, c.width, l.w_gate, c.width, q->B[0], l.ff, n, l.ff, c.width);
	a.W2 = l.w_up;
	a.epi = glu_epi(l, EPI_GLU_GELU);
	a.limit = l.limit;
	TRY(gemm(q, a));
	return gemm(q, plain(q->B[0], l.ff, l.w_down, l.ff, out, c.width, n, c.width, l.ff));
}

static int ff_moe(Seq *q, int li, int n) {
	const yalm_seq_layer &l = q->L[li];
	const yalm_seq_config &c = q->c;
	const int E = l.experts, top = l.top, ff = l.ff, slots = n * top;
	float *hx = q->B[0], *yx = q->B[1], *hs = q->B[2], *ys = q->B[3];
	seq_router_kernel<<<n, SEQ_THREADS, (2 * E + l.groups) * sizeof(float), q->stream>>>(q->In, c.width, l.router, E, top, l.groups,
	                                                                    l.groups_keep, l.router_scale,
	                                                                    l.shared_ff > 0 ? l.shared_sg : nullptr, q->idx,
	                                                                    q->wt, q->sgate, l.router_kind, l.router_bias);
	HIPCHK(hipGetLastError());
	const int epi = glu_epi(l, EPI_GLU_CLAMP);
	if (n <= GEMV_MAX_M) { // one batch per (token, choice): its expert's matrices picked on the device
		GemmArgs a = plain(q->In, c.width, l.w_gate, c.width, hx, ff, 1, ff, c.width);
		a.W2 = l.w_up;
		a.a_bs = c.width;
		a.a_zdiv = top;
		a.w_sel = q->idx;
		a.w_bs = (long)ff * c.width;
		a.c_bs = ff;
		a.epi = epi;
		a.limit = l.limit;
		TRY(gemm(q, a, slots));
		GemmArgs b = plain(hx, ff, l.w_down, ff, yx, c.width, 1, c.width, ff);
		b.a_bs = ff;
		b.w_sel = q->idx;
		b.w_bs = (long)c.width * ff;
		b.c_bs = c.width;
		TRY(gemm(q, b, slots));
	} else { // tokens grouped by expert: one batch per expert over its row list
		seq_fill_int_kernel<<<cdiv(E, 256), 256, 0, q->stream>>>(q->counts, E, 0);
		seq_moe_lists_kernel<<<cdiv(slots, SEQ_THREADS), SEQ_THREADS, 0, q->stream>>>(q->idx, slots, q->counts, q->lists,
		                                                                              q->cap);
		HIPCHK(hipGetLastError());
		GemmArgs a = plain(q->In, c.width, l.w_gate, c.width, hx, ff, n, ff, c.width);
		a.W2 = l.w_up;
		a.w_bs = (long)ff * c.width;
		a.rows = q->lists;
		a.rows_bs = q->cap;
		a.counts = q->counts;
		a.a_div = top;
		a.epi = epi;
		a.limit = l.limit;
		TRY(gemm(q, a, E, n));
		GemmArgs b = plain(hx, ff, l.w_down, ff, yx, c.width, n, c.width, ff);
		b.w_bs = (long)c.width * ff;
		b.rows = q->lists;
		b.rows_bs = q->cap;
		b.counts = q->counts;
		TRY(gemm(q, b, E, n));
	}
	if (l.shared_ff > 0) {
		GemmArgs a = plain(q->In, c.width, l.ws_gate, c.width, hs, l.shared_ff, n, l.shared_ff, c.width);
		a.W2 = l.ws_up;
		a.epi = epi;
		a.limit = l.shared_limit;
		TRY(gemm(q, a));
		TRY(gemm(q, plain(hs, l.shared_ff, l.ws_down, l.shared_ff, ys, c.width, n, c.width, l.shared_ff)));
	}
	return YALM_OK; // the combine of yx (B[1]) and ys (B[3]) happens in the closing norm's launch (add_norm, par_close)
}

// The seam after a parallel block: both sublayers' results join the stream (the experts' combine
// happens here), the next entry's pre_add and opening norm follow in the same launch.
static int par_close(Seq *q, int li, int n) {
	const yalm_seq_config &c = q->c;
	const yalm_seq_layer &l = q->L[li];
	const yalm_seq_layer *nx = li + 1 < c.n_layers ? &q->L[li + 1] : nullptr;
	const bool moe = l.ff_kind == YALM_FF_MOE;
	const bool gated = moe && l.shared_ff > 0 && l.shared_sg;
	const bool joined = q->side_of[li] >= 0; // two mixers side by side: their normed results meet in this launch
	float *dump = q->dump_on && q->dump ? q->dump + (size_t)li * n * c.width : nullptr;
#define PC_ARGS                                                                                                        \
	q->X, q->Y, l.ls1, (l.ff_kind != YALM_FF_NONE && !moe) ? q->Y2 : nullptr, l.ls2, moe ? q->B[1] : nullptr, q->wt,    \
	    moe ? l.top : 0, moe && l.shared_ff > 0 ? q->B[3] : nullptr, gated ? q->sgate : nullptr, dump,                 \
	    nx ? nx->pre_add : nullptr, c.norm_eps, c.width, nx ? nx->norm1 : nullptr, q->Hn, (int)q->ln,                  \
	    (nx && nx->ff_kind != YALM_FF_NONE) ? nx->norm2 : nullptr, q->Hn2, joined ? q->Y3 : nullptr, l.join_w,        \
	    l.side_join_w, l.join_scale
	if (c.width <= 4 * SEQ_THREADS)
		seq_par_close_reg_kernel<4><<<n, SEQ_THREADS, 0, q->stream>>>(PC_ARGS);
	else if (c.width <= 8 * SEQ_THREADS)
		seq_par_close_reg_kernel<8><<<n, SEQ_THREADS, 0, q->stream>>>(PC_ARGS);
	else if (c.width <= 16 * SEQ_THREADS)
		seq_par_close_reg_kernel<16><<<n, SEQ_THREADS, 0, q->stream>>>(PC_ARGS);
	else
		seq_par_close_kernel<<<n, SEQ_THREADS, (size_t)c.width * sizeof(float), q->stream>>>(PC_ARGS);
#undef PC_ARGS
	HIPCHK(hipGetLastError());
	return YALM_OK;
}

// moe: the layer's routed experts feed the norm (their combine happens inside it) instead of Y
static int add_norm(Seq *q, const float *wb, const float *w_next, int n, const yalm_seq_layer *moe) {
	const int w = q->c.width;
	if (!moe && w <= 16 * SEQ_THREADS) { // the row in registers
#define AN_LAUNCH(E)                                                                                                   \
	seq_add_norm_reg_kernel<E><<<n, SEQ_THREADS, 0, q->stream>>>(q->X, q->Y, wb, q->c.norm_eps, w, w_next, q->Hn, (int)q->ln)
		if (w <= 4 * SEQ_THREADS) AN_LAUNCH(4);
		else if (w <= 8 * SEQ_THREADS) AN_LAUNCH(8);
		else AN_LAUNCH(16);
#undef AN_LAUNCH
	} else {
		seq_add_norm_kernel<<<n, SEQ_THREADS, w * sizeof(float), q->stream>>>(
		    q->X, q->Y, wb, q->c.norm_eps, w, w_next, q->Hn, moe ? q->B[1] : nullptr, q->wt, moe ? moe->top : 0,
		    moe && moe->shared_ff > 0 ? q->B[3] : nullptr, q->sgate, (int)q->ln);
	}
	HIPCHK(hipGetLastError());
	return YALM_OK;
}

// One portion of n <= cap tokens through every layer, from the states and caches earlier
// portions left; tokens_dev == nullptr: the greedy loop's device-resident token. The
// position is st->pos on the device (set by the caller).
static int enqueue_portion(Seq *q, const int *tokens_dev, int n) {
	const yalm_seq_config &c = q->c;
	const bool pre = c.pre_norm != 0; // else the sublayers read the stream itself and no opening norm is computed
	const float *first_norm = pre ? q->L[0].norm1 : nullptr;
	const bool par = c.block_kind == YALM_BLOCK_PARALLEL;
	// a parallel block whose feed-forward has a norm of its own reads Hn2 = norm2(x)
	const float *first_norm2 = (par && q->L[0].ff_kind != YALM_FF_NONE) ? q->L[0].norm2 : nullptr;
	if (!pre) { // every portion starts in the same row of the stream (the greedy graph's pointers are static)
		q->X = q->Xbase;
		q->In = q->X;
	}
	q->pend_wb = nullptr;
	const bool fold = an_foldable(q, n);
	// the closing norm of a sublayer: applied now, or owed to the product that reads the stream next
	auto close = [&](const float *wb, const float *w_next, const yalm_seq_layer *moe) {
		if (fold && !moe && !w_next) {
			q->pend_wb = wb;
			return (int)YALM_OK;
		}
		return add_norm(q, wb, w_next, n, moe);
	};
	if (c.weight_dtype == YALM_F32)
		seq_embed_kernel<WF32><<<n, SEQ_THREADS, 0, q->stream>>>(q->st, tokens_dev, q->embed, q->inv_freq, c.width,
		                                                         c.vocab, c.embed_scale, q->X, first_norm, c.norm_eps,
		                                                         q->Hn, (int)q->ln, q->L[0].pre_add, q->embed_norm, first_norm2,
		                                                         q->Hn2);
	else
		seq_embed_kernel<WBF16><<<n, SEQ_THREADS, 0, q->stream>>>(q->st, tokens_dev, q->embed, q->inv_freq, c.width,
		                                                          c.vocab, c.embed_scale, q->X, first_norm, c.norm_eps,
		                                                          q->Hn, (int)q->ln, q->L[0].pre_add, q->embed_norm, first_norm2,
		                                                          q->Hn2);
	HIPCHK(hipGetLastError());
	auto run_mixer = [&](int mi) {
		const yalm_seq_layer &m = q->L[mi];
		if (latent_direct(m))
			return mixer_latent_direct(q, mi, n);
		if (m.mixer == YALM_MIX_LATENT)
			return mixer_latent(q, mi, n);
		if (m.mixer == YALM_MIX_RGLRU)
			return mixer_rglru(q, mi, n);
		if (m.mixer == YALM_MIX_ATTN)
			return mixer_attn(q, mi, n);
		if (m.mixer == YALM_MIX_SSM)
			return mixer_ssm(q, mi, n);
		return mixer_delta(q, mi, n);
	};
	for (int li = 0; li < c.n_layers; ++li) {
		const yalm_seq_layer &l = q->L[li];
		const float *next = pre && li + 1 < c.n_layers ? q->L[li + 1].norm1 : nullptr;
		const int side = q->side_of[li];
		if (l.mixer != YALM_MIX_ATTN || side >= 0)
			TRY(flush_norm(q, n)); // only a lone attention mixer's input projection takes an owed norm
		q->Yout = q->Y;
		TRY(run_mixer(li));
		if (side >= 0) { // the second mixer reads the same input; the two normed results are summed into Y
			q->Yout = q->Y3;
			const int rc = run_mixer(side);
			q->Yout = q->Y;
			TRY(rc);
			if (!par) { // serial blocks: joined here; a parallel block's seam joins them itself
				seq_pair_join_kernel<<<n, SEQ_THREADS, 0, q->stream>>>(q->Y, q->Y3, l.join_w, l.side_join_w, l.join_scale,
				                                                       c.norm_eps, c.width);
				HIPCHK(hipGetLastError());
			}
		}
		if (par) { // both sublayers read norms of the same stream; the feed-forward's result goes beside the mixer's
			const float *mix_in = q->In;
			if (l.norm2 && l.ff_kind != YALM_FF_NONE)
				q->In = q->Hn2;
			int rc = YALM_OK;
			if (l.ff_kind == YALM_FF_DENSE)
				rc = ff_dense(q, li, n, q->Y2);
			else if (l.ff_kind == YALM_FF_PLAIN)
				rc = ff_plain(q, li, n, q->Y2);
			else if (l.ff_kind == YALM_FF_MOE)
				rc = ff_moe(q, li, n);
			q->In = mix_in;
			TRY(rc);
			TRY(par_close(q, li, n));
			continue;
		}
		if (l.ff_kind == YALM_FF_NONE) {
			TRY(close(l.norm1b, next, nullptr));
		} else {
			TRY(close(l.norm1b, pre ? l.norm2 : nullptr, nullptr));
			if (l.ff_kind != YALM_FF_PLAIN)
				TRY(flush_norm(q, n));
			TRY(l.ff_kind == YALM_FF_DENSE ? ff_dense(q, li, n, q->Y)
			                               : (l.ff_kind == YALM_FF_PLAIN ? ff_plain(q, li, n, q->Y) : ff_moe(q, li, n)));
			TRY(close(l.norm2b, next, l.ff_kind == YALM_FF_MOE ? &l : nullptr));
		}
		if (q->dump_on && q->dump)
			HIPCHK(hipMemcpyAsync(q->dump + (size_t)li * n * c.width, q->X, (size_t)n * c.width * sizeof(float),
			                      hipMemcpyDeviceToDevice, q->stream));
	}
	return flush_norm(q, n); // the last sublayer's norm, if still owed
}

// Final norm of the asked rows and their logits into q->logits ([n_rows][vocab], n_rows <= LOGIT_ROWS).
static int enqueue_logits(Seq *q, const int *rows_dev, int n_rows) {
	const yalm_seq_config &c = q->c;
	seq_norm_kernel<float><<<n_rows, SEQ_THREADS, 0, q->stream>>>(q->X, c.width, q->final_norm, c.norm_eps, c.width,
	                                                              q->Hn, c.width, rows_dev, q->st, 0, (int)q->ln,
	                                                              c.logit_scale);
	HIPCHK(hipGetLastError());
	return gemm(q, plain(q->Hn, c.width, q->head, c.width, q->logits, c.vocab, n_rows, c.vocab, c.width));
}

extern "C" int yalm_seq_step(yalm_seq q, const int *tokens, int n, const int *want, int n_want, float *logits_host) {
	ARGCHK(q && tokens && n > 0, "yalm_seq_step: null decoder or no tokens");
	ARGCHK(n_want == 0 || (want && logits_host), "yalm_seq_step: logits asked for without a buffer");
	ARGCHK(q->host_pos + n <= q->c.max_tokens, "yalm_seq_step: the sequence would pass max_tokens");
	for (int i = 0; i < n_want; ++i)
		ARGCHK(want[i] >= 0 && want[i] < n && (i == 0 || want[i] > want[i - 1]), "yalm_seq_step: want must ascend within the tokens");
	const yalm_seq_config &c = q->c;
	int wi = 0;
	q->dump_n = 0;
	for (int t0 = 0; t0 < n; t0 += q->cap) {
		const int m = std::min(q->cap, n - t0);
		HIPCHK(hipMemcpyAsync(q->tok, tokens + t0, (size_t)m * sizeof(int), hipMemcpyHostToDevice, q->stream));
		set_step_kernel<<<1, 1, 0, q->stream>>>(q->st, 0, q->host_pos, 0);
		HIPCHK(hipGetLastError());
		q->cur_pos = q->host_pos;
		if (q->dump_on) {
			if (!q->dump)
				TRY(sallocT(q, &q->dump, (size_t)c.n_layers * q->cap * c.width));
			q->dump_n = m;
		}
		TRY(enqueue_portion(q, q->tok, m));
		q->host_pos += m;
		int w1 = wi;
		while (w1 < n_want && want[w1] < t0 + m)
			++w1;
		while (wi < w1) { // this portion's asked rows, LOGIT_ROWS at a time
			const int k = std::min(w1 - wi, (int)LOGIT_ROWS);
			std::vector<int> rel(k);
			for (int i = 0; i < k; ++i)
				rel[i] = want[wi + i] - t0;
			HIPCHK(hipMemcpyAsync(q->want, rel.data(), (size_t)k * sizeof(int), hipMemcpyHostToDevice, q->stream));
			HIPCHK(hipStreamSynchronize(q->stream)); // rel leaves scope
			TRY(enqueue_logits(q, q->want, k));
			HIPCHK(hipMemcpyAsync(logits_host + (size_t)wi * c.vocab, q->logits, (size_t)k * c.vocab * sizeof(float),
			                      hipMemcpyDeviceToHost, q->stream));
			HIPCHK(hipStreamSynchronize(q->stream));
			wi += k;
		}
	}
	if (n_want)
		HIPCHK(hipStreamSynchronize(q->stream));
	return YALM_OK;
}

static int enqueue_greedy_token(Seq *q) {
	TRY(enqueue_portion(q, nullptr, 1));
	TRY(enqueue_logits(q, q->want, 1));
	argmax_kernel<<<1, 1024, 0, q->stream>>>(q->logits, q->c.vocab, q->st, q->gen_tokens, q->gen_cap);
	HIPCHK(hipGetLastError());
	return YALM_OK;
}

static int ensure_greedy_graph(Seq *q) {
	if (q->greedy_exec)
		return YALM_OK;
	HIPCHK(hipStreamBeginCapture(q->stream, hipStreamCaptureModeRelaxed));
	const int r = enqueue_greedy_token(q);
	hipGraph_t g = nullptr;
	const hipError_t e = hipStreamEndCapture(q->stream, &g);
	if (r != YALM_OK)
		return r;
	HIPCHK(e);
	q->greedy_graph = g;
	HIPCHK(hipGraphInstantiate(&q->greedy_exec, g, nullptr, nullptr, 0));
	return YALM_OK;
}

extern "C" int yalm_seq_generate_greedy(yalm_seq q, int token, int n_steps, int *out_tokens) {
	ARGCHK(q && out_tokens && n_steps > 0 && n_steps <= q->gen_cap, "yalm_seq_generate_greedy: bad argument");
	ARGCHK(q->host_pos + n_steps <= q->c.max_tokens, "yalm_seq_generate_greedy: the sequence would pass max_tokens");
	ARGCHK(token >= 0 && token < q->c.vocab, "yalm_seq_generate_greedy: token out of range");
	const bool graph = !q->dump_on; // the layer dump's copies stay out of the graph
	if (graph)
		TRY(ensure_greedy_graph(q));
	set_step_kernel<<<1, 1, 0, q->stream>>>(q->st, token, q->host_pos, 1);
	seq_fill_int_kernel<<<1, 1, 0, q->stream>>>(q->want, 1, 0);
	HIPCHK(hipGetLastError());
	for (int i = 0; i < n_steps; ++i) {
		if (graph)
			HIPCHK(hipGraphLaunch(q->greedy_exec, q->stream));
		else
			TRY(enqueue_greedy_token(q));
	}
	HIPCHK(hipMemcpyAsync(out_tokens, q->gen_tokens, (size_t)n_steps * sizeof(int), hipMemcpyDeviceToHost, q->stream));
	HIPCHK(hipStreamSynchronize(q->stream));
	q->host_pos += n_steps;
	return YALM_OK;
}

extern "C" int yalm_seq_layer_dump(yalm_seq q, int on) {
	ARGCHK(q, "yalm_seq_layer_dump: null decoder");
	q->dump_on = on != 0;
	return YALM_OK;
}

extern "C" int yalm_seq_get_layers(yalm_seq q, float *host, size_t count) {
	ARGCHK(q && host, "yalm_seq_get_layers: null argument");
	ARGCHK(q->dump && count == (size_t)q->c.n_layers * q->dump_n * q->c.width,
	       "yalm_seq_get_layers: count must be n_layers * tokens of the last portion * width");
	HIPCHK(hipStreamSynchronize(q->stream));
	HIPCHK(hipMemcpy(host, q->dump, count * sizeof(float), hipMemcpyDeviceToHost));
	return YALM_OK;
}

extern "C" int yalm_seq_time_step(yalm_seq q, int n, int pos0, int iters, float *avg_ms) {
	ARGCHK(q && avg_ms && n > 0 && n <= q->cap && iters > 0 && pos0 >= 0 && pos0 + n <= q->c.max_tokens,
	       "yalm_seq_time_step: bad argument");
	std::vector<int> tk(n);
	for (int i = 0; i < n; ++i)
		tk[i] = (int)(((unsigned)i * 2654435761u) % (unsigned)q->c.vocab);
	HIPCHK(hipMemcpy(q->tok, tk.data(), (size_t)n * sizeof(int), hipMemcpyHostToDevice));
	seq_fill_int_kernel<<<1, 1, 0, q->stream>>>(q->want, 1, n - 1);
	hipEvent_t e0, e1;
	HIPCHK(hipEventCreate(&e0));
	HIPCHK(hipEventCreate(&e1));
	int rc = YALM_OK;
	for (int it = -1; it < iters && rc == YALM_OK; ++it) { // one untimed run first
		if (it == 0)
			(void)hipEventRecord(e0, q->stream);
		set_step_kernel<<<1, 1, 0, q->stream>>>(q->st, 0, pos0, 0);
		q->cur_pos = pos0;
		rc = enqueue_portion(q, q->tok, n);
		if (rc == YALM_OK)
			rc = enqueue_logits(q, q->want, 1);
	}
	(void)hipEventRecord(e1, q->stream);
	hipError_t e = hipEventSynchronize(e1);
	float ms = 0.0f;
	if (e == hipSuccess)
		e = hipEventElapsedTime(&ms, e0, e1);
	(void)hipEventDestroy(e0);
	(void)hipEventDestroy(e1);
	TRY(rc);
	HIPCHK(e);
	*avg_ms = ms / iters;
	return YALM_OK;
}
