// seq_attn.h — softmax attention over cached keys and values for the layer-list engine
// (YALM_MIX_ATTN in include/yalm_hip.h): grouped key/value heads, rotary positions on the
// first rot_dims entries of a head (interleaved pairs, rescaled frequencies), query / key /
// value norms, a per-head score temperature, scores mixed across heads, causal / sliding
// window / chunked masks, a softmax with an optional zero-score sink, a per-head output gate.
// Every option is a runtime argument, so another design can combine them differently.
//
// Positions and angles, the norms, scores, softmax weights and their weighted sums are f32
// (the angle itself is evaluated in double: position * frequency loses bits in f32 at large
// positions). The caches hold bf16 (WBF16 models) or f32 (WF32 models).
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
};

// First key position that position p sees.
__host__ __device__ __forceinline__ int attn_first_key(int mask_kind, int mask_size, int p) {
	if (mask_kind == YALM_MASK_WINDOW)
		return p - mask_size + 1 > 0 ? p - mask_size + 1 : 0;
	if (mask_kind == YALM_MASK_CHUNK)
		return (p / mask_size) * mask_size;
	return 0;
}

template <class CT>
__device__ __forceinline__ void cache_store(CT *p, float v) {
	if constexpr (sizeof(CT) == 2)
		*p = f2bf(v);
	else
		*p = v;
}

// ------------------------------------------------------------------ projections -> queries, cache rows, gates
// One workgroup per token t at position p = st->pos + t, a wave per head. Z row: [q: H D | k: G D |
// v: G V | gate: H] (biases already added). Queries leave scaled by scale * temp[h] in Q
// [t][H D]; keys and values go to the cache rows p; gate[t][h] = sigmoid(z_gate[h]).
// Dynamic LDS: rot_dims floats (cos | sin).
template <class CT>
__global__ __launch_bounds__(SEQ_THREADS) void seq_attn_prep_kernel(const float *__restrict__ Z, int ldz, AttnArgs a,
                                                                    const StepState *__restrict__ st,
                                                                    float *__restrict__ Q, CT *__restrict__ Kc,
                                                                    CT *__restrict__ Vc, float *__restrict__ gate) {
	extern __shared__ float rot[];
	__shared__ float red[SEQ_THREADS / 64];
	const int t = blockIdx.x, tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
	const int p = st->pos + t;
	const int half = a.rot_dims >> 1;
	for (int i = tid; i < half; i += SEQ_THREADS) {
		const double ang = (double)p * a.rot_freq[i];
		rot[i] = (float)cos(ang) * a.rot_mag;
		rot[half + i] = (float)sin(ang) * a.rot_mag;
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
	const int jobs = a.H + 2 * a.G;
	for (int job = wave; job < jobs; job += SEQ_THREADS / 64) {
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
					const float c = rot[d >> 1], s = rot[half + (d >> 1)];
					v = (d & 1) ? w * c + u * s : u * c - w * s;
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
		if (kind == 2 ? a.v_norm != 0 : a.qk_norm == YALM_QK_HEAD_UNIT)
			mul = 1.0f / sqrtf(ss / (float)n + a.eps);
		if (kind == 0)
			mul *= a.scale * (a.temp ? a.temp[hh] : 1.0f);
#pragma unroll
		for (int e = 0; e < 4; ++e) {
			const int d = lane + 64 * e;
			if (d >= n)
				continue;
			const float v = val[e] * mul;
			if (kind == 0)
				Q[(size_t)t * QN + hh * a.D + d] = v;
			else if (kind == 1)
				cache_store<CT>(Kc + (size_t)p * KN + hh * a.D + d, v);
			else
				cache_store<CT>(Vc + (size_t)p * VN + hh * a.V + d, v);
		}
	}
	if (a.out_gate)
		for (int h = tid; h < a.H; h += SEQ_THREADS)
			gate[(size_t)t * a.H + h] = sq_sigmoid(z[QN + KN + VN + h]);
}

// ------------------------------------------------------------------ attention, f32 FMA form
// A workgroup owns TQ tokens x Hb heads (rows r = tq Hb + hl) and walks its share of the keys
// they see in tiles of SA_KT. With score mixing (talk) a workgroup holds all heads of its
// tokens (Hb = H, every key/value head in turn); without, the heads of one key/value head
// (gridDim.z = G). Per tile: raw scores of every row (a lane per key), the mix across heads,
// mask and running softmax per row, then the weighted sums of the value tile, each thread NA4
// groups of 4 value entries of one row. Key splits (gridDim.y = S > 1; single tokens and short
// portions): split s leaves (sums, running maximum, running sum) per row in `part` for
// seq_latent_merge_kernel; the sink (a key of score 0 without a value) is split 0's starting
// state. S == 1 writes the normalised, gated sums to Ctx [t][H V].
#define SA_KT 64
#define SA_MAX_NA4 16

__host__ __device__ inline int sa_ldk(int D, int V) {
	const int d4 = (D + 3) & ~3, v4 = (V + 3) & ~3;
	return (d4 > v4 ? d4 : v4) + 4;
}
static inline size_t sa_lds_bytes(int R, int H, int D, int V, bool talk) {
	const int d4 = (D + 3) & ~3;
	return sizeof(float) * ((size_t)R * d4 + (size_t)SA_KT * sa_ldk(D, V) + (size_t)R * SA_KT * (talk ? 2 : 1) +
	                        (talk ? (size_t)H * H : 0) + 5 * (size_t)R);
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

template <class CT, int NA4>
__global__ __launch_bounds__(SEQ_THREADS) void seq_attn_kernel(const float *__restrict__ Q, const CT *__restrict__ Kc,
                                                               const CT *__restrict__ Vc, AttnArgs a, int n_tok, int TQ,
                                                               const StepState *__restrict__ st,
                                                               const float *__restrict__ gate, float *__restrict__ Ctx,
                                                               float *__restrict__ part) {
	extern __shared__ __attribute__((aligned(16))) float lds[];
	const int H = a.H, G = a.G, D = a.D, V = a.V, rep = H / G;
	const bool talk = a.talk != nullptr;
	const int Hb = talk ? H : rep, Gb = talk ? G : 1;
	const int h0 = talk ? 0 : blockIdx.z * rep, g0 = talk ? 0 : blockIdx.z;
	const int R = TQ * Hb;
	const int D4 = (D + 3) & ~3, q4n = D4 >> 2, V4n = (V + 3) >> 2, ldk = sa_ldk(D, V);
	float *qs = lds;                          // [R][D4]
	float *cs = qs + R * D4;                  // [SA_KT][ldk]: the key tile, then the value tile
	float *ps = cs + SA_KT * ldk;             // [R][SA_KT] raw scores, then softmax weights
	float *ps2 = ps + R * SA_KT;              // talk: [R][SA_KT] mixed scores
	float *tk = ps2 + (talk ? R * SA_KT : 0); // talk: [H][H]
	float *mrun = tk + (talk ? H * H : 0);    // [R]
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
	for (int i = tid; i < R * D4; i += SEQ_THREADS) {
		const int r = i / D4, d = i % D4;
		const int t = t0 + r / Hb, h = h0 + r % Hb;
		qs[i] = (t < n_tok && d < D) ? Q[((size_t)t * H + h) * D + d] : 0.0f;
	}
	if (talk)
		for (int i = tid; i < H * H; i += SEQ_THREADS)
			tk[i] = a.talk[i];
	const bool sink0 = a.sink && split == 0;
	for (int r = tid; r < R; r += SEQ_THREADS) {
		const int t = t0 + r / Hb;
		mrun[r] = sink0 ? 0.0f : -FLT_MAX;
		lrun[r] = sink0 ? 1.0f : 0.0f;
		alpha[r] = 1.0f;
		rlo[r] = t < n_tok ? attn_first_key(a.mask_kind, a.mask_size, pos0 + t) : 0x7fffffff;
		rhi[r] = t < n_tok ? pos0 + t : -1;
	}
	float4_t acc[NA4];
#pragma unroll
	for (int x = 0; x < NA4; ++x)
		acc[x] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};
	const int nrows_g = TQ * rep; // rows that read one key/value head
	for (int kt = k_begin; kt < k_end; kt += SA_KT) {
		// ---- raw scores
		for (int gl = 0; gl < Gb; ++gl) {
			__syncthreads(); // the previous readers of cs are done
			sa_fill_tile<CT>(cs, ldk, Kc, G * D, (g0 + gl) * D, D, kt, k_end);
			__syncthreads();
			const float4_t *cj = (const float4_t *)(cs + lane * ldk);
			for (int i0 = wave * 4; i0 < nrows_g; i0 += 4 * (SEQ_THREADS / 64)) {
				int rr[4];
#pragma unroll
				for (int x = 0; x < 4; ++x) {
					const int i = min(i0 + x, nrows_g - 1);
					rr[x] = (i / rep) * Hb + gl * rep + (i % rep);
				}
				float s[4] = {0.0f, 0.0f, 0.0f, 0.0f};
				for (int d = 0; d < q4n; ++d) {
					const float4_t c = cj[d];
#pragma unroll
					for (int x = 0; x < 4; ++x) {
						const float4_t qv = *(const float4_t *)(qs + rr[x] * D4 + 4 * d);
						s[x] = fmaf(qv[0], c[0], s[x]);
						s[x] = fmaf(qv[1], c[1], s[x]);
						s[x] = fmaf(qv[2], c[2], s[x]);
						s[x] = fmaf(qv[3], c[3], s[x]);
					}
				}
#pragma unroll
				for (int x = 0; x < 4; ++x)
					if (i0 + x < nrows_g)
						ps[rr[x] * SA_KT + lane] = s[x];
			}
		}
		__syncthreads();
		// ---- mix across heads
		const float *sc = ps;
		if (talk) {
			for (int pair = tid; pair < TQ * SA_KT; pair += SEQ_THREADS) {
				const int tq = pair / SA_KT, key = pair % SA_KT;
				const float *in = ps + (size_t)tq * H * SA_KT + key;
				for (int h = 0; h < H; ++h) {
					float m = 0.0f;
					for (int g = 0; g < H; ++g)
						m = fmaf(tk[h * H + g], in[g * SA_KT], m);
					ps2[(tq * H + h) * SA_KT + key] = m;
				}
			}
			__syncthreads();
			sc = ps2;
		}
		// ---- mask and running softmax, a wave per row
		for (int r = wave; r < R; r += SEQ_THREADS / 64) {
			const int j = kt + lane;
			const bool vis = j >= rlo[r] && j <= rhi[r] && j < k_end;
			const float sv = vis ? sc[r * SA_KT + lane] : -FLT_MAX;
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
		for (int gl = 0; gl < Gb; ++gl) {
			__syncthreads(); // the weights are written / the previous readers of cs are done
			sa_fill_tile<CT>(cs, ldk, Vc, G * V, (g0 + gl) * V, V, kt, k_end);
			__syncthreads();
#pragma unroll
			for (int x = 0; x < NA4; ++x) {
				const int u = tid + x * SEQ_THREADS;
				if (u >= R * V4n)
					continue;
				const int r = u / V4n, d4 = u % V4n;
				if ((h0 + r % Hb) / rep != g0 + gl)
					continue;
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
						const float4_t c = *(const float4_t *)(cs + (4 * j4 + e) * ldk + 4 * d4);
						v[0] = fmaf(p[e], c[0], v[0]);
						v[1] = fmaf(p[e], c[1], v[1]);
						v[2] = fmaf(p[e], c[2], v[2]);
						v[3] = fmaf(p[e], c[3], v[3]);
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
