// C ABI of libtinygemma_hip.so (declared in include/tinygemma_hip.h): library state, weight
// upload / re-tiling, sessions, and the kernel sequences of forward_prefill / forward_decode.

#include <fcntl.h>
#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <sys/stat.h>
#include <unistd.h>

#include <algorithm>
#include <chrono>
#include <map>

#include "tg_internal.h"

// ---------------------------------------------------------------------------------------------
// library state and errors
// ---------------------------------------------------------------------------------------------
namespace {

thread_local std::string g_err;
bool g_inited = false;
int g_gemm_mfma = 1;            // prefill GEMM: 1 = int8 MFMA on three digit planes, 0 = exact-order fp32 on the vector ALUs
int8_t *g_apack = nullptr;      // scratch of the stand-alone GEMM entry points
size_t g_apack_bytes = 0;
float *g_rowscale = nullptr;
size_t g_rowscale_n = 0;
int g_prefetch_plan = 0;        // which launch prefetches which weights (experiment knob)
int g_prefetch_blocks = 128;   // extra workgroups per launch that prefetch the next launch's weights (0: off; multiple of 8)
// Workgroups per GEMV launch before workgroups start looping over tiles.  2048 = 8 per compute unit, all resident at
// once: the LM head's 2048 tiles each get their own (47 us per launch streamed from HBM, 50-54 us with 1024 that
// walk two tiles each).
int g_gemv_max_blocks = 2048;
// How greedy decode steps are issued.  0: stream launches; 1: replay of a captured step that reads its position from device
// memory; 2: replay with the position-dependent nodes re-described before every replay (the kernels and grids of the
// stream launches); -1 (default): 2 for models whose step is bound by the host's launch rate, else 0 (decode_graph_mode).
int g_use_graphs = -1;
int g_device = -1;
hipStream_t g_stream = nullptr;
char g_devname[256] = "";
int g_n_cu = 256;
bool g_gemm_split = true;       // prefill: products that would leave most compute units idle run in 2 or 4 parts of K
int g_attn_merge_chunk = 64;  // decode attention: past this many keys per workgroup, use more workgroups and a merge launch
bool g_chain_picks = true;  // inside a batch of greedy decode steps the next step's first launch finishes the previous pick
bool g_keep_taps = false;  // prefill keeps a copy of the residual stream after every block (parity checks)
// Decode: all layers of a step in one launch of resident workgroups (tg_decode_fused.hip) instead of 5 launches per layer.
// g_fused_ng: GEMV workgroups of that launch (0: one per compute unit, less the attention workgroups).
int g_fused = 0, g_fused_ng = 0, g_fused_spins = 1 << 20;
unsigned long long *g_fused_ts = nullptr;  // device buffer of tg_debug_fused_timestamps while it runs
// Counts changes of the tuning knobs.  A captured decode step bakes the knobs of its capture into its launches
// (prefetch workgroups, grid limits, attention geometry), so a session drops its captured graphs when this has moved.
unsigned g_knob_epoch = 0;

bool legal_in(int d) { return d == 640 || d == 2048 || d == 1024 || d == 256 || d == 1152 || d == 6912; }            // static_switch.hpp:7-30
bool legal_out(int d) { return d == 640 || d == 262144 || d == 2048 || d == 256 || d == 1024 || d == 1152 || d == 6912; }  // :32-58

int ensure_init() {
	if (g_inited) return TG_OK;
	return tg_init(0);
}

// A matrix on the device.  `W` is the GEMV layout: ntiles tiles of C columns, each a contiguous
// [K/4][C][4] slab (C chosen per matrix so that narrow matrices still give hundreds of
// workgroups).  `Wg` (optional) is the same matrix in 128-column tiles of [K/16][128][16] for the
// int8 MFMA prefill GEMM (B-operand order).
struct PackedMat {
	int8_t *W = nullptr;
	float *scales = nullptr;   // per virtual column, GEMV tile order
	int8_t *Wg = nullptr;
	float *scales_g = nullptr; // per virtual column, GEMM tile order
	int K = 0, N = 0;          // N = number of (virtual) columns
	int ntiles = 0, C = 0, lc_shift = 0;
	int ntiles_g = 0;
};

// Largest tile width that still yields >= 256 workgroups (at least 4 columns; 8 for the fused
// up|gate matrix, whose tile holds C/2 up and C/2 gate columns).
int choose_tile_cols(int N, int min_c) {
	int C = TG_CT;
	while (C > min_c && (N % C != 0 || N / C < 256)) C >>= 1;
	return C;
}

TgColMap plain_map(const int8_t *W, const float *scales, int N) {
	TgColMap m;
	memset(&m, 0, sizeof(m));
	m.src[0] = W;
	m.scales[0] = scales;
	m.n[0] = N;
	return m;
}

void free_packed(PackedMat *p);

// Builds the device layouts of one matrix from sources already on the device (reference layout; see TgColMap):
// GEMV tiles always, MFMA tiles if with_gemm.  min_c: smallest GEMV tile width allowed.  For an interleaved
// map (up|gate) `m.half` is ignored on entry and set per layout: half a tile of each.
int build_packed(PackedMat *p, TgColMap m, int K, int N, int min_c, bool with_gemm) {
	const bool interleave = m.half != 0;
	p->K = K;
	p->N = N;
	p->C = choose_tile_cols(N, min_c);
	p->lc_shift = 0;
	while ((4 << p->lc_shift) < p->C) p->lc_shift++;
	p->ntiles = N / p->C;
	TG_HIP(hipMalloc((void **)&p->W, (size_t)K * N));
	TG_HIP(hipMalloc((void **)&p->scales, (size_t)N * sizeof(float)));
	if (interleave) m.half = p->C / 2;
	tg_launch_retile_gemv(p->W, p->scales, m, K, N, p->C, g_stream);
	if (with_gemm) {
		p->ntiles_g = N / TG_CT;
		TG_HIP(hipMalloc((void **)&p->Wg, (size_t)K * N));
		TG_HIP(hipMalloc((void **)&p->scales_g, (size_t)N * sizeof(float)));
		if (interleave) m.half = TG_CT / 2;
		tg_launch_retile_mfma(p->Wg, p->scales_g, m, K, N, g_stream);
	}
	TG_HIP(hipGetLastError());
	return TG_OK;
}

// Plain host matrix [K][N] (reference layout): staged on the device, then re-tiled there.
int upload_packed(PackedMat *p, const int8_t *host_rowmajor, const float *host_scales, int K, int N, bool with_gemm) {
	int8_t *raw = nullptr;
	float *rs = nullptr;
	auto done = [&](int rc) {
		(void)hipStreamSynchronize(g_stream);
		if (raw) (void)hipFree(raw);
		if (rs) (void)hipFree(rs);
		return rc;
	};
	if (hipMalloc((void **)&raw, (size_t)K * N) != hipSuccess || hipMalloc((void **)&rs, (size_t)N * sizeof(float)) != hipSuccess)
		return done(tg_fail(TG_ERR_HIP, "hipMalloc of the staging copy failed"));
	if (hipMemcpyAsync(raw, host_rowmajor, (size_t)K * N, hipMemcpyHostToDevice, g_stream) != hipSuccess ||
	    hipMemcpyAsync(rs, host_scales, (size_t)N * sizeof(float), hipMemcpyHostToDevice, g_stream) != hipSuccess)
		return done(tg_fail(TG_ERR_HIP, "upload of the staging copy failed"));
	return done(build_packed(p, plain_map(raw, rs, N), K, N, 4, with_gemm));
}

void free_packed(PackedMat *p) {
	void *ps[] = {p->W, p->scales, p->Wg, p->scales_g};
	for (void *q : ps)
		if (q) (void)hipFree(q);
	p->W = p->Wg = nullptr;
	p->scales = p->scales_g = nullptr;
}

TgGemv gemv_base(const PackedMat &p) {
	TgGemv g;
	memset(&g, 0, sizeof(g));
	g.W = p.W;
	g.scales = p.scales;
	g.K = p.K;
	g.ntiles = p.ntiles;
	g.C = p.C;
	g.lc_shift = p.lc_shift;
	g.max_blocks = g_gemv_max_blocks;
	return g;
}

// C[m][N] = scales * (A[m][K] . W) through the selected GEMM; apack/rowscale are scratch for the MFMA path.
//   prepacked : the producer of A already wrote the digit planes and row factors
//   amax_in   : row maxima of A left by its producer (saves the pass over A that finds them)
//   amax_out  : GEGLU only: [rows], cleared by the caller; this product folds max|C[row][:]| into it
//   kparts    : MFMA path, STORE only, and only what tg_gemm_mfma_k_parts says: the product runs in 2 or 4 parts of K,
//               part p's partial result goes to C + p * part_stride and the consumer adds them
void launch_gemm(float *C, const float *A, int lda, const PackedMat &p, int m, int epi, const float *lut, float gmin, float geps,
                 int lut_size, int8_t *apack, float *rowscale, bool prepacked = false, const float *amax_in = nullptr,
                 float *amax_out = nullptr, int kparts = 1, size_t part_stride = 0) {
	if (g_gemm_mfma) {
		if (!prepacked) tg_launch_quant_pack(A, lda, m, p.K, apack, rowscale, amax_in, g_stream);
		tg_launch_gemm_mfma(C, apack, rowscale, p.Wg, p.scales_g, m, p.K, p.ntiles_g, epi, lut, gmin, geps, lut_size, amax_out, kparts,
		                    part_stride, g_stream);
	} else {
		(void)lda;  // the exact kernel reads dense rows (lda == K at every call site)
		tg_launch_gemm(C, A, p.W, p.scales, m, p.K, p.ntiles, p.C, epi, lut, gmin, geps, lut_size, g_stream);
	}
}

// Prefetch job for the GEMV tiles of `p` (see TgPrefetch).
TgPrefetch prefetch_of(const PackedMat &p) {
	TgPrefetch f;
	f.ptr = g_prefetch_blocks > 0 ? p.W : nullptr;
	f.slab = (uint32_t)p.K * (uint32_t)p.C;
	f.ntiles = p.ntiles;
	f.nblocks = g_prefetch_blocks;
	return f;
}

int attn_range_error() {
	return tg_fail(TG_ERR_STATE, "prefill attention: a q, k or v value is NaN or lies outside the fp16 range (+-65504) of the two-plane operand format; "
	                             "the result is not valid.  tg_set_attn_prefill_format(0) selects the three-plane bf16 format, which has fp32's range");
}

int upload_floats(float **dst, const float *src, size_t n) {
	TG_HIP(hipMalloc((void **)dst, n * sizeof(float)));
	TG_HIP(hipMemcpy(*dst, src, n * sizeof(float), hipMemcpyHostToDevice));
	return TG_OK;
}

}  // namespace

int tg_fail(int code, const std::string &msg) {
	g_err = msg;
	return code;
}

hipStream_t tg_probe_stream() { return g_inited ? g_stream : nullptr; }  // for the timing probes of tg_probe.hip
int tg_probe_n_cu() { return g_n_cu; }

struct tg_qweight {
	PackedMat p;
};

struct LayerDev {
	PackedMat qkv, o, ug, d;
	float *rms_q = nullptr, *rms_k = nullptr, *apre = nullptr, *apost = nullptr, *mpre = nullptr, *mpost = nullptr;
	bool is_sw = false;
};

struct tg_model {
	tg_config cfg;
	bool loaded = false;
	int n_sessions = 0;     // live sessions: while there are any, the weights are neither reloaded nor freed under them
	bool orphaned = false;  // tg_model_destroy was called with live sessions: the last of them deletes the struct
	int8_t *wte = nullptr;  // [vocab][hidden], reference layout (rows are gathered, never streamed)
	float *wte_scales = nullptr;
	float *rmsw = nullptr;
	PackedMat lm;
	std::vector<LayerDev> L;
};

namespace {
// Device copy of the balanced work list of the causal (window < 0) or the local prefill layers of S tokens, with
// its scratch.
struct AttnPlanDev {
	TgAttnPrefillPlan p;
	bool use = false;
	int S = -1, tq = 0, window = -1;  // what the lists were built for
	void *bufs[5] = {nullptr, nullptr, nullptr, nullptr, nullptr};
	std::vector<int4> items, split;  // host copies stay alive until the uploads have completed
	std::vector<int2> tiles;
	int build(int n_tokens, int win) {
		const int tile = tg_attn_prefill_query_tile(n_tokens, g_n_cu);
		if (n_tokens == S && tile == tq && win == window) return TG_OK;
		release();
		const int rc = build_uncached(n_tokens, tile, win);
		if (rc != TG_OK) release();  // nothing half-built stays behind as a cache hit
		return rc;
	}
	int build_uncached(int n_tokens, int tile, int win) {
		int nslots = 0;
		use = tg_attn_prefill_plan(n_tokens, g_n_cu, tile, win, items, split, nslots);
		S = n_tokens;
		tq = tile;
		window = win;
		if (!use) return TG_OK;
		TG_HIP(hipMalloc(&bufs[0], items.size() * sizeof(int4)));
		TG_HIP(hipMalloc(&bufs[1], split.size() * sizeof(int4)));
		TG_HIP(hipMalloc(&bufs[2], tg_attn_prefill_part_floats(nslots, tile) * sizeof(float)));
		TG_HIP(hipMalloc(&bufs[3], tg_attn_prefill_ml_floats(nslots, tile) * sizeof(float)));
		TG_HIP(hipMemcpyAsync(bufs[0], items.data(), items.size() * sizeof(int4), hipMemcpyHostToDevice, g_stream));
		TG_HIP(hipMemcpyAsync(bufs[1], split.data(), split.size() * sizeof(int4), hipMemcpyHostToDevice, g_stream));
		tiles.assign((size_t)((n_tokens + tile - 1) / tile), int2{-1, 1});
		for (const int4 &sp : split) tiles[(size_t)sp.x] = int2{sp.y, sp.z};
		TG_HIP(hipMalloc(&bufs[4], tiles.size() * sizeof(int2)));
		TG_HIP(hipMemcpyAsync(bufs[4], tiles.data(), tiles.size() * sizeof(int2), hipMemcpyHostToDevice, g_stream));
		p.items = (const int4 *)bufs[0];
		p.split = (const int4 *)bufs[1];
		p.tiles = (const int2 *)bufs[4];
		p.nitems = (int)items.size();
		p.nsplit = (int)split.size();
		p.part_o = (float *)bufs[2];
		p.part_ml = (float *)bufs[3];
		return TG_OK;
	}
	const TgAttnPrefillPlan *get() const { return use ? &p : nullptr; }
	void release() {
		for (void *&b : bufs) {
			if (b) (void)hipFree(b);
			b = nullptr;
		}
		use = false;
		S = -1;
		tq = 0;
		window = -1;
	}
};
}  // namespace

struct tg_session {
	tg_model *m = nullptr;
	float *cos_g = nullptr, *sin_g = nullptr, *cos_l = nullptr, *sin_l = nullptr;  // [n_pos][head_dim/2]
	float *lut = nullptr;
	float gmin = 0, geps = 0;
	int lut_size = 0;
	std::vector<float *> kc, vc;
	std::vector<int> max_pos;
	float *xr = nullptr;      // [(2L+1)][hidden] residual stream after every block of the last decode
	float *qkv = nullptr, *attn_out = nullptr, *o_out = nullptr, *hbuf = nullptr, *d_out = nullptr, *logits = nullptr;
	float *part_acc = nullptr, *part_ml = nullptr;      // attention partials [nb][4][256], [nb][4][2]
	float *merged_acc = nullptr, *merged_ml = nullptr;  // long contexts: every TG_ATTN_FOLD partials folded into one
	float *blk_val = nullptr;
	int *blk_idx = nullptr;
	bool counted = false;     // this session is included in m->n_sessions
	unsigned graph_epoch = 0; // g_knob_epoch the cached graphs were captured under
	float *zeros = nullptr;   // [hidden] of 0: as the pending block output of a post-norm + residual prologue it adds nothing
	float *blk_x = nullptr, *blk_y = nullptr;  // [hidden] input / output of the block-level entry points
	int *ctr = nullptr;       // device: [0] position_ptr, [1] buffer_ptr local, [2] buffer_ptr global, [3] step, [4] token,
	                          // [5] set by the prefill attention when an operand does not fit its fp16 planes
	int *tok_log = nullptr;
	int tok_log_cap = 0;
	int pos = 0, bp_local = 0, bp_global = 0, steps = 0;  // host mirrors
	float *taps = nullptr;    // prefill taps [(2L+1)][rows][hidden] (kept only for short prompts)
	int tap_rows = 0;
	std::map<uint64_t, hipGraphExec_t> graphs;  // captured decode steps, keyed by the attention launch geometry
	// graphs of mode 2, keyed by which layer kinds have a merge launch: the template graph stays alive (its nodes name
	// what is updated in the executable graph); attn / merge / oproj: the nodes by layer (merge: null where there is none)
	struct PatchedGraph {
		hipGraph_t graph = nullptr;
		hipGraphExec_t exec = nullptr;
		int steps = 1;  // decode steps in the graph; the node lists are indexed step * layers + layer
		std::vector<hipGraphNode_t> attn, merge, oproj;
	};
	std::map<uint64_t, PatchedGraph> pgraphs;
	bool graphs_failed = false;  // the runtime refused a capture or a node update of mode 2: plain launches from then on
	// min-p sampling (allocated on first use): scratch of the three sampler launches and the caller's uniform draws
	float *probs = nullptr, *seg = nullptr, *bsum = nullptr, *bmax = nullptr, *randf = nullptr;
	int randf_cap = 0;
	// The greedy pick of the last enqueued decode step exists only as the per-workgroup maxima of its LM-head launch:
	// the first launch of the next step finishes it (and does the per-token bookkeeping), or flush_pick() does.
	bool pick_pending = false;
	bool sampling = false;  // decode steps enqueued now draw their token instead of taking the argmax
	float s_minp = 1.0f, s_temp = 1.0f;
	int rand_base = 0;      // token-log index of the token that uses randf[0]
	// prefill workspace (the reference's PrefillState, decode.hpp:281-351): one arena, grown on demand, kept until the
	// session is destroyed, and the work lists of the causal layers for the last prompt length
	void *pf_ws = nullptr;
	size_t pf_ws_bytes = 0;
	AttnPlanDev pf_plan, pf_plan_local;
	// one-kernel decode step (tg_decode_fused.hip): built on first use; fused_state 0 = not built yet, 1 = usable,
	// -1 = not usable for this model or device, or a wait timed out (the session then stays on the launch path)
	int fused_state = 0, fused_variant = -1;
	unsigned fused_epoch = 0;      // g_knob_epoch that fused.ng and fused_variant were derived under
	bool fused_unchecked = false;  // fused launches have been enqueued since the error word was last read
	TgFused fused;                 // the launch-independent fields
	TgFusedLayer *fused_layers = nullptr;
	float *fused_xch = nullptr;
	unsigned *fused_sync = nullptr;
	unsigned fused_all = 0, fused_attn = 0;  // host mirrors of the arrival counters
};

namespace {
constexpr int ATTN_MAX_BLOCKS = TG_ATTN_MAX_BLOCKS;
constexpr int PREFILL_TAP_MAX_ROWS = 1024;

bool layer_is_local(const tg_config &c, int l) { return (l % c.window_pattern) != (c.window_pattern - 1); }  // transformer.hpp:43

int check_config(const tg_config *c) {
	if (!c) return tg_fail(TG_ERR_BAD_ARG, "null config");
	if (c->head_dim != 256 || c->n_head != 4 || c->n_kv != 1)
		return tg_fail(TG_ERR_UNSUPPORTED_SHAPE, "attention kernels are built for 4 query heads, 1 KV head, head_dim 256 (config.hpp:47-48)");
	if (!legal_in(c->hidden_size) || !legal_out(c->hidden_size))
		return tg_fail(TG_ERR_UNSUPPORTED_SHAPE, "Unsupported ROW dimension: " + std::to_string(c->hidden_size));
	if (!legal_in(c->intermediate_size) || !legal_out(c->intermediate_size))
		return tg_fail(TG_ERR_UNSUPPORTED_SHAPE, "Unsupported COL dimension: " + std::to_string(c->intermediate_size));
	if (!legal_out(c->n_vocab)) return tg_fail(TG_ERR_UNSUPPORTED_SHAPE, "Unsupported COL dimension: " + std::to_string(c->n_vocab));
	if (c->hidden_size > 1152) return tg_fail(TG_ERR_UNSUPPORTED_SHAPE, "hidden_size above 1152");
	if (c->n_layers < 1 || c->n_pos < 1 || c->n_pos_local < 1 || c->window_pattern < 1) return tg_fail(TG_ERR_BAD_ARG, "bad config");
	return TG_OK;
}
}  // namespace

// ---- the entry point that allocates nothing --------------------------------------------------------------------
// Scratch of the int8 matrix GEMM (digit planes of the activations + row factors) for callers that cannot allocate:
// a fixed array in the library's device image.  Each GPU the library runs on holds it until the process ends.
// In host code the array's name is only a handle for hipGetSymbolAddress; kernels get g_static_scratch.
#define TG_STATIC_ELEMS ((size_t)TG_QGEMM_STATIC_MAX_ELEMS)
#define TG_STATIC_PLANE_BYTES (3 * TG_STATIC_ELEMS)
#define TG_STATIC_ROWS (TG_STATIC_ELEMS / 256)  // the narrowest legal inDim is 256
static __device__ __align__(256) unsigned char tg_static_scratch[TG_STATIC_PLANE_BYTES + 2 * TG_STATIC_ROWS * sizeof(float)];
static unsigned char *g_static_scratch = nullptr;  // device address of tg_static_scratch on g_device (set by tg_init)

static int static_scratch_init() {
	void *p = nullptr;
	TG_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(tg_static_scratch)));
	g_static_scratch = (unsigned char *)p;
	return TG_OK;
}

extern "C" {

// ---------------------------------------------------------------------------------------------
// library
// ---------------------------------------------------------------------------------------------
int tg_init(int device) {
	if (g_inited) {
		if (device != g_device) return tg_fail(TG_ERR_BAD_ARG, "already initialised on another device");
		return TG_OK;
	}
	int n = 0;
	if (hipGetDeviceCount(&n) != hipSuccess || n <= 0) return tg_fail(TG_ERR_NO_DEVICE, "no HIP device");
	if (device < 0 || device >= n) return tg_fail(TG_ERR_NO_DEVICE, "no such device");
	TG_HIP(hipSetDevice(device));
	hipDeviceProp_t prop;
	TG_HIP(hipGetDeviceProperties(&prop, device));
	snprintf(g_devname, sizeof(g_devname), "%s (%s, %d CUs)", prop.name, prop.gcnArchName, prop.multiProcessorCount);
	g_n_cu = prop.multiProcessorCount > 0 ? prop.multiProcessorCount : 256;
	TG_HIP(hipStreamCreate(&g_stream));
	g_gemm_lds_cus = g_n_cu;
	if (int rc = static_scratch_init()) return rc;
	g_device = device;
	g_inited = true;
	return TG_OK;
}

const char *tg_last_error(void) { return g_err.c_str(); }

const char *tg_status_string(int code) {
	switch (code) {
		case TG_OK: return "ok";
		case TG_ERR_UNSUPPORTED_SHAPE: return "unsupported dimension";
		case TG_ERR_FILE_OPEN: return "Could not open file.";
		case TG_ERR_FILE_SHORT: return "weight file shorter than the configuration requires";
		case TG_ERR_BAD_ARG: return "bad argument";
		case TG_ERR_HIP: return "HIP runtime error";
		case TG_ERR_NO_DEVICE: return "no HIP device";
		case TG_ERR_STATE: return "session state does not allow this call";
		default: return "unknown";
	}
}

void *tg_stream(void) { return (void *)g_stream; }

int tg_synchronize(void) {
	if (ensure_init() != TG_OK) return TG_ERR_NO_DEVICE;
	TG_HIP(hipStreamSynchronize(g_stream));
	return TG_OK;
}

const char *tg_device_name(void) {
	if (ensure_init() != TG_OK) return "";
	return g_devname;
}

int tg_config_named(const char *name, tg_config *out) {
	if (!name || !out) return tg_fail(TG_ERR_BAD_ARG, "null argument");
	tg_config c = {0, 0, 0, 262144, 32768, 512, 256, 4, 1, 1000000.0f, 10000.0f, 6};  // config.hpp:46-48
	if (strcmp(name, "270m") == 0) {
		c.hidden_size = 640; c.intermediate_size = 2048; c.n_layers = 18;
	} else if (strcmp(name, "1B") == 0) {
		c.hidden_size = 1152; c.intermediate_size = 6912; c.n_layers = 26;
	} else {
		return tg_fail(TG_ERR_BAD_ARG, std::string("unknown model size: ") + name);
	}
	*out = c;
	return TG_OK;
}

// ---------------------------------------------------------------------------------------------
// device helpers
// ---------------------------------------------------------------------------------------------
int tg_dev_alloc(void **p, size_t bytes) {
	if (int rc = ensure_init()) return rc;
	TG_HIP(hipMalloc(p, bytes));
	return TG_OK;
}
int tg_dev_free(void *p) {
	TG_HIP(hipFree(p));
	return TG_OK;
}
int tg_copy_h2d(void *dst, const void *src, size_t bytes) {
	TG_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, g_stream));
	TG_HIP(hipStreamSynchronize(g_stream));
	return TG_OK;
}
int tg_dev_copy(void *dst, const void *src, size_t bytes) {
	if (!dst || !src || bytes % 16) return tg_fail(TG_ERR_BAD_ARG, "bad argument");
	tg_launch_copy(dst, src, bytes, g_stream);
	TG_HIP(hipGetLastError());
	return TG_OK;
}
int tg_copy_d2h(void *dst, const void *src, size_t bytes) {
	TG_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, g_stream));
	TG_HIP(hipStreamSynchronize(g_stream));
	return TG_OK;
}

// ---------------------------------------------------------------------------------------------
// kernel level
// ---------------------------------------------------------------------------------------------
int tg_qweight_create(const int8_t *B, const float *scales, int inDim, int outDim, tg_qweight **out) {
	if (int rc = ensure_init()) return rc;
	if (!B || !scales || !out) return tg_fail(TG_ERR_BAD_ARG, "null argument");
	if (!legal_in(inDim)) return tg_fail(TG_ERR_UNSUPPORTED_SHAPE, "Unsupported ROW dimension: " + std::to_string(inDim));
	if (!legal_out(outDim)) return tg_fail(TG_ERR_UNSUPPORTED_SHAPE, "Unsupported COL dimension: " + std::to_string(outDim));
	tg_qweight *w = new tg_qweight();
	int rc = upload_packed(&w->p, B, scales, inDim, outDim, outDim <= 16384);
	if (rc != TG_OK) {
		free_packed(&w->p);
		delete w;
		return rc;
	}
	*out = w;
	return TG_OK;
}

void tg_qweight_destroy(tg_qweight *w) {
	if (!w) return;
	(void)hipStreamSynchronize(g_stream);
	free_packed(&w->p);
	delete w;
}

int tg_qgemv_dev(float *y_dev, const float *x_dev, const tg_qweight *w, int logits_variant) {
	(void)logits_variant;  // one kernel serves both reference variants (they differ only in rounding order)
	if (!y_dev || !x_dev || !w) return tg_fail(TG_ERR_BAD_ARG, "null argument");
	TgGemv g = gemv_base(w->p);
	g.x = x_dev;
	g.y = y_dev;
	tg_launch_gemv(g, TG_ROLE_PLAIN, g_stream);
	TG_HIP(hipGetLastError());
	return TG_OK;
}

int tg_qgemm_dev(float *C_dev, const float *A_dev, const tg_qweight *w, int m) {
	if (!C_dev || !A_dev || !w || m < 1) return tg_fail(TG_ERR_BAD_ARG, "bad argument");
	if (g_gemm_mfma && !w->p.Wg) return tg_fail(TG_ERR_UNSUPPORTED_SHAPE, "no MFMA tiling was built for this matrix (outDim too large)");
	if (g_gemm_mfma) {
		const size_t need = tg_gemm_mfma_apack_bytes(m, w->p.K), need_rs = 2 * tg_gemm_mfma_rows(m);
		if (need > g_apack_bytes || need_rs > g_rowscale_n) {
			TG_HIP(hipStreamSynchronize(g_stream));
			if (g_apack) (void)hipFree(g_apack);
			if (g_rowscale) (void)hipFree(g_rowscale);
			g_apack = nullptr;
			g_rowscale = nullptr;
			g_apack_bytes = 0;  // a failed allocation below must not leave the old sizes standing for the freed buffers
			g_rowscale_n = 0;
			TG_HIP(hipMalloc((void **)&g_apack, need));
			TG_HIP(hipMalloc((void **)&g_rowscale, need_rs * sizeof(float)));
			g_apack_bytes = need;
			g_rowscale_n = need_rs;
		}
	}
	launch_gemm(C_dev, A_dev, w->p.K, w->p, m, TG_EPI_STORE, nullptr, 0, 0, 0, g_apack, g_rowscale);
	TG_HIP(hipGetLastError());
	return TG_OK;
}

// tg_qgemm_dev on the fixed scratch above: no hipMalloc/hipFree, nothing set up on the way.  Calls share the one
// array (the planes of the previous call are overwritten; nothing in it needs to start at zero), so calls that
// overlap on one GPU would race: the library's single stream orders them.
// tg_qgemm_dev with every workgroup of the matrix kernel reporting the clocks it lived for (see tg_gemm_clk)
int tg_debug_gemm_clock(float *C_dev, const float *A_dev, const tg_qweight *w, int m, double *clock_mhz, double *workgroup_us, int *workgroups) {
	if (!clock_mhz || !workgroup_us || !workgroups) return tg_fail(TG_ERR_BAD_ARG, "null argument");
	if (int rc = ensure_init()) return rc;
	constexpr int MAX_WGS = 1 << 16;
	if (!w || m < 1 || (long long)((m + 127) / 128) * w->p.ntiles_g * 2 > MAX_WGS) return tg_fail(TG_ERR_BAD_ARG, "bad argument (at most 32768 output tiles)");
	unsigned long long *buf = nullptr;
	if (int rc = tg_gemm_clk_begin(&buf, MAX_WGS, g_stream)) return rc;
	// five launches back to back: the readings left in the buffer are those of the last one, at the clock the part has
	// settled on under this load
	int rc = TG_OK;
	for (int i = 0; i < 5 && rc == TG_OK; i++) rc = tg_qgemm_dev(C_dev, A_dev, w, m);
	if (rc == TG_OK && hipStreamSynchronize(g_stream) != hipSuccess) rc = tg_fail(TG_ERR_HIP, "hipStreamSynchronize failed");
	const int rc2 = tg_gemm_clk_end(buf, MAX_WGS, clock_mhz, workgroup_us, workgroups);
	return rc != TG_OK ? rc : rc2;
}

int tg_qgemm_dev_static(float *C_dev, const float *A_dev, const tg_qweight *w, int m) {
	if (!g_inited || !g_static_scratch) return tg_fail(TG_ERR_STATE, "tg_init has not run: this entry point sets nothing up itself");
	if (!C_dev || !A_dev || !w || m < 1) return tg_fail(TG_ERR_BAD_ARG, "bad argument");
	if (g_gemm_mfma && !w->p.Wg) return tg_fail(TG_ERR_UNSUPPORTED_SHAPE, "no MFMA tiling was built for this matrix (outDim too large)");
	const size_t rows = tg_gemm_mfma_rows(m);
	if (rows * (size_t)w->p.K > TG_STATIC_ELEMS)
		return tg_fail(TG_ERR_BAD_ARG, "m (rounded up to a multiple of 128) x inDim exceeds TG_QGEMM_STATIC_MAX_ELEMS = " +
		                                   std::to_string(TG_STATIC_ELEMS) + ": use tg_qgemm_dev");
	// rows <= TG_STATIC_ELEMS / K <= TG_STATIC_ROWS, so the row factors fit behind the planes
	launch_gemm(C_dev, A_dev, w->p.K, w->p, m, TG_EPI_STORE, nullptr, 0, 0, 0, (int8_t *)g_static_scratch,
	            (float *)(g_static_scratch + TG_STATIC_PLANE_BYTES));
	TG_HIP(hipGetLastError());
	return TG_OK;
}

static int qgemv_host(float *C, const float *A, const int8_t *B, const float *scales, int inDim, int outDim, int variant) {
	if (int rc = ensure_init()) return rc;
	if (!C || !A || !B || !scales) return tg_fail(TG_ERR_BAD_ARG, "null argument");
	tg_qweight *w = nullptr;
	int rc = tg_qweight_create(B, scales, inDim, outDim, &w);
	if (rc != TG_OK) return rc;
	float *x = nullptr, *y = nullptr;
	std::vector<float> yh((size_t)outDim);
	rc = tg_dev_alloc((void **)&x, sizeof(float) * inDim);
	if (rc == TG_OK) rc = tg_dev_alloc((void **)&y, sizeof(float) * outDim);
	if (rc == TG_OK) rc = tg_copy_h2d(x, A, sizeof(float) * inDim);
	if (rc == TG_OK) rc = tg_qgemv_dev(y, x, w, variant);
	if (rc == TG_OK) rc = tg_copy_d2h(yh.data(), y, sizeof(float) * outDim);
	if (x) (void)hipFree(x);
	if (y) (void)hipFree(y);
	tg_qweight_destroy(w);
	if (rc != TG_OK) return rc;
	// The reference accumulates into C and then scales C (linalg.hpp:52-107); with the required
	// zero C this is the plain product.  A non-zero C is carried through the same way.
	for (int c = 0; c < outDim; c++) C[c] = C[c] * scales[c] + yh[c];
	return TG_OK;
}

int tg_qgemv(float *C, const float *A, const int8_t *B, const float *scales, int inDim, int outDim) {
	return qgemv_host(C, A, B, scales, inDim, outDim, 0);
}
int tg_qgemv_logits(float *C, const float *A, const int8_t *B, const float *scales, int inDim, int outDim) {
	return qgemv_host(C, A, B, scales, inDim, outDim, 1);
}

int tg_qgemm(float *C, const float *A, const int8_t *B, const float *scales, int m, int inDim, int outDim) {
	if (int rc = ensure_init()) return rc;
	if (!C || !A || !B || !scales || m < 1) return tg_fail(TG_ERR_BAD_ARG, "bad argument");
	tg_qweight *w = nullptr;
	int rc = tg_qweight_create(B, scales, inDim, outDim, &w);
	if (rc != TG_OK) return rc;
	float *a = nullptr, *c = nullptr;
	rc = tg_dev_alloc((void **)&a, sizeof(float) * (size_t)m * inDim);
	if (rc == TG_OK) rc = tg_dev_alloc((void **)&c, sizeof(float) * (size_t)m * outDim);
	if (rc == TG_OK) rc = tg_copy_h2d(a, A, sizeof(float) * (size_t)m * inDim);
	if (rc == TG_OK) rc = tg_qgemm_dev(c, a, w, m);
	if (rc == TG_OK) rc = tg_copy_d2h(C, c, sizeof(float) * (size_t)m * outDim);
	if (a) (void)hipFree(a);
	if (c) (void)hipFree(c);
	tg_qweight_destroy(w);
	return rc;
}

// ---------------------------------------------------------------------------------------------
// model
// ---------------------------------------------------------------------------------------------
size_t tg_weight_file_bytes(const tg_config *c) {
	if (!c) return 0;
	const size_t h = c->hidden_size, f = c->intermediate_size, V = c->n_vocab, hd = c->head_dim;
	const size_t qo = (size_t)c->n_head * hd, kv = (size_t)c->n_kv * hd;
	size_t per_layer = h * qo + 4 * qo + 2 * (h * kv + 4 * kv) + qo * h + 4 * h + 2 * 4 * hd + 2 * 4 * h + 2 * (h * f + 4 * f) +
	                   f * h + 4 * h + 2 * 4 * h;
	return V * h + 4 * h + 4 * h + per_layer * (size_t)c->n_layers + h * V + 4 * V;
}

int tg_model_create(const tg_config *cfg, tg_model **out) {
	if (int rc = ensure_init()) return rc;
	if (!out) return tg_fail(TG_ERR_BAD_ARG, "null argument");
	if (int rc = check_config(cfg)) return rc;
	tg_model *m = new tg_model();
	m->cfg = *cfg;
	m->L.resize((size_t)cfg->n_layers);
	for (int l = 0; l < cfg->n_layers; l++) m->L[(size_t)l].is_sw = layer_is_local(*cfg, l);
	*out = m;
	return TG_OK;
}

static void model_free_weights(tg_model *m) {
	(void)hipStreamSynchronize(g_stream);
	if (m->wte) (void)hipFree(m->wte);
	if (m->wte_scales) (void)hipFree(m->wte_scales);
	if (m->rmsw) (void)hipFree(m->rmsw);
	m->wte = nullptr; m->wte_scales = nullptr; m->rmsw = nullptr;
	free_packed(&m->lm);
	for (auto &L : m->L) {
		free_packed(&L.qkv); free_packed(&L.o); free_packed(&L.ug); free_packed(&L.d);
		float **ps[] = {&L.rms_q, &L.rms_k, &L.apre, &L.apost, &L.mpre, &L.mpost};
		for (float **p : ps) {
			if (*p) (void)hipFree(*p);
			*p = nullptr;
		}
	}
	m->loaded = false;
}

void tg_model_destroy(tg_model *m) {
	if (!m) return;
	model_free_weights(m);  // loaded = false: every entry point of a session that is still alive returns TG_ERR_STATE from now on
	if (m->n_sessions > 0) {
		m->orphaned = true;  // the sessions still point here; the last tg_session_destroy deletes the struct
		return;
	}
	delete m;
}

}  // extern "C"

// The file goes to the device as it is (the reference layout, transformer.hpp:122-160), in chunks through two
// pinned staging buffers so that producing a chunk (file read or memcpy) overlaps the DMA of the previous one.
// fill(dst, off, len) must produce bytes [off, off + len) of the file at dst.
template <typename Fill>
static int stage_image(uint8_t *d_raw, size_t n, Fill fill) {
	constexpr size_t CHUNK = (size_t)32 << 20;
	void *pin[2] = {nullptr, nullptr};
	hipEvent_t ev[2] = {nullptr, nullptr};
	bool used[2] = {false, false};
	int rc = TG_OK;
	for (int i = 0; i < 2 && rc == TG_OK; i++) {
		if (hipHostMalloc(&pin[i], std::min(CHUNK, n), hipHostMallocDefault) != hipSuccess || hipEventCreate(&ev[i]) != hipSuccess)
			rc = tg_fail(TG_ERR_HIP, "pinned staging buffer allocation failed");
	}
	int i = 0;
	for (size_t off = 0; off < n && rc == TG_OK; off += CHUNK, i ^= 1) {
		const size_t len = std::min(CHUNK, n - off);
		if (used[i] && hipEventSynchronize(ev[i]) != hipSuccess) rc = tg_fail(TG_ERR_HIP, "hipEventSynchronize failed");
		if (rc == TG_OK) rc = fill(pin[i], off, len);
		if (rc == TG_OK && (hipMemcpyAsync(d_raw + off, pin[i], len, hipMemcpyHostToDevice, g_stream) != hipSuccess ||
		                    hipEventRecord(ev[i], g_stream) != hipSuccess))
			rc = tg_fail(TG_ERR_HIP, "upload of a weight chunk failed");
		used[i] = true;
	}
	(void)hipStreamSynchronize(g_stream);
	for (int k = 0; k < 2; k++) {
		if (ev[k]) (void)hipEventDestroy(ev[k]);
		if (pin[k]) (void)hipHostFree(pin[k]);
	}
	return rc;
}

// Walks the device image of the file in the order of transformer.hpp:122-160 and builds the device layouts
// with the re-tiling kernels; small fp32 vectors get their own allocations.
static int build_from_image(tg_model *m, const uint8_t *d_raw) {
	const tg_config &c = m->cfg;
	const size_t h = (size_t)c.hidden_size, f = (size_t)c.intermediate_size, V = (size_t)c.n_vocab, hd = (size_t)c.head_dim;
	const size_t qo = (size_t)c.n_head * hd, kv = (size_t)c.n_kv * hd;
	size_t off = 0;
	auto take = [&](size_t bytes) {
		const uint8_t *p = d_raw + off;
		off += bytes;
		return p;
	};
	auto take_w = [&](size_t n) { return (const int8_t *)take(n); };
	auto take_f = [&](size_t n) { return (const float *)take(4 * n); };
	auto own_f = [&](float **dst, size_t n) -> int {
		const float *src = take_f(n);
		TG_HIP(hipMalloc((void **)dst, n * sizeof(float)));
		TG_HIP(hipMemcpyAsync(*dst, src, n * sizeof(float), hipMemcpyDeviceToDevice, g_stream));
		return TG_OK;
	};
	int rc;
	// wte stays in the reference layout: its rows are gathered, never streamed
	const int8_t *wte = take_w(V * h);
	TG_HIP(hipMalloc((void **)&m->wte, V * h));
	TG_HIP(hipMemcpyAsync(m->wte, wte, V * h, hipMemcpyDeviceToDevice, g_stream));
	if ((rc = own_f(&m->wte_scales, h))) return rc;
	if ((rc = own_f(&m->rmsw, h))) return rc;
	for (int l = 0; l < c.n_layers; l++) {
		LayerDev &L = m->L[(size_t)l];
		// Q | K | V side by side along the output dimension: [h][qo + 2 kv]
		TgColMap qkv;
		memset(&qkv, 0, sizeof(qkv));
		for (int part = 0; part < 3; part++) {
			const size_t n = part == 0 ? qo : kv;
			qkv.src[part] = take_w(h * n);
			qkv.scales[part] = take_f(n);
			qkv.n[part] = (int)n;
		}
		if ((rc = build_packed(&L.qkv, qkv, (int)h, (int)(qo + 2 * kv), 4, true))) return rc;
		const int8_t *o = take_w(qo * h);
		const float *os = take_f(h);
		if ((rc = build_packed(&L.o, plain_map(o, os, (int)h), (int)qo, (int)h, 4, true))) return rc;
		if ((rc = own_f(&L.rms_q, hd))) return rc;
		if ((rc = own_f(&L.rms_k, hd))) return rc;
		if ((rc = own_f(&L.apre, h))) return rc;
		if ((rc = own_f(&L.apost, h))) return rc;
		// up | gate: every tile holds half a tile of up columns followed by the same gate columns, so that
		// gelu(gate) * up never leaves a workgroup
		TgColMap ug;
		memset(&ug, 0, sizeof(ug));
		for (int part = 0; part < 2; part++) {
			ug.src[part] = take_w(h * f);
			ug.scales[part] = take_f(f);
			ug.n[part] = (int)f;
		}
		ug.half = 1;
		if ((rc = build_packed(&L.ug, ug, (int)h, (int)(2 * f), 8, true))) return rc;
		const int8_t *d = take_w(f * h);
		const float *ds = take_f(h);
		if ((rc = build_packed(&L.d, plain_map(d, ds, (int)h), (int)f, (int)h, 4, true))) return rc;
		if ((rc = own_f(&L.mpre, h))) return rc;
		if ((rc = own_f(&L.mpost, h))) return rc;
	}
	const int8_t *lm = take_w(h * V);
	const float *lms = take_f(V);
	if ((rc = build_packed(&m->lm, plain_map(lm, lms, (int)V), (int)h, (int)V, 4, false))) return rc;
	TG_HIP(hipStreamSynchronize(g_stream));
	m->loaded = true;
	return TG_OK;
}

template <typename Fill>
static int load_weights_impl(tg_model *m, Fill fill) {
	// a session holds device pointers into the weights (and captured graphs bake them in): no reload under a live session
	if (m->n_sessions > 0) return tg_fail(TG_ERR_STATE, "the model has live sessions: destroy them before loading weights again");
	model_free_weights(m);
	const size_t n = tg_weight_file_bytes(&m->cfg);
	uint8_t *d_raw = nullptr;
	if (hipMalloc((void **)&d_raw, n) != hipSuccess) return tg_fail(TG_ERR_HIP, "hipMalloc of the file image failed");
	int rc = stage_image(d_raw, n, fill);
	if (rc == TG_OK) rc = build_from_image(m, d_raw);
	(void)hipStreamSynchronize(g_stream);
	(void)hipFree(d_raw);
	if (rc != TG_OK) model_free_weights(m);
	return rc;
}

extern "C" {

int tg_model_load_weights(tg_model *m, const char *path) {
	if (!m || !path) return tg_fail(TG_ERR_BAD_ARG, "null argument");
	const int fd = open(path, O_RDONLY);
	if (fd < 0) return tg_fail(TG_ERR_FILE_OPEN, "Could not open file.");  // transformer.hpp:163
	struct stat st;
	if (fstat(fd, &st) != 0 || (size_t)st.st_size < tg_weight_file_bytes(&m->cfg)) {
		close(fd);
		return tg_fail(TG_ERR_FILE_SHORT, "weight file is shorter than the configuration requires");
	}
	(void)posix_fadvise(fd, 0, 0, POSIX_FADV_SEQUENTIAL);
	int rc = load_weights_impl(m, [&](void *dst, size_t off, size_t len) -> int {
		size_t got = 0;
		while (got < len) {
			const ssize_t r = pread(fd, (char *)dst + got, len - got, (off_t)(off + got));
			if (r <= 0) return tg_fail(TG_ERR_FILE_SHORT, "weight file is shorter than the configuration requires");
			got += (size_t)r;
		}
		return TG_OK;
	});
	close(fd);
	return rc;
}

int tg_model_load_weights_mem(tg_model *m, const void *image, size_t n) {
	if (!m || !image) return tg_fail(TG_ERR_BAD_ARG, "null argument");
	if (n != tg_weight_file_bytes(&m->cfg)) return tg_fail(TG_ERR_FILE_SHORT, "image size does not match the configuration");
	const uint8_t *p = (const uint8_t *)image;
	return load_weights_impl(m, [&](void *dst, size_t off, size_t len) -> int {
		memcpy(dst, p + off, len);
		return TG_OK;
	});
}

// ---------------------------------------------------------------------------------------------
// session
// ---------------------------------------------------------------------------------------------
static int upload_rope(float **cos_d, float **sin_d, const float *cos_h, const float *sin_h, float theta, int n_pos, int hd) {
	const int half = hd / 2;
	std::vector<float> c((size_t)n_pos * half), s((size_t)n_pos * half);
	if (cos_h && sin_h) {
		// decode::RoPE keeps [n_pos][hd] with both halves equal (decode.hpp:190-200): keep one half
		for (int p = 0; p < n_pos; p++)
			for (int d = 0; d < half; d++) {
				c[(size_t)p * half + d] = cos_h[(size_t)p * hd + d];
				s[(size_t)p * half + d] = sin_h[(size_t)p * hd + d];
			}
	} else {
		// decode.hpp:176-201: freq_i = 1/pow(theta, 2i/hd) and angle = p*freq in fp32;
		// cos/sin of that fp32 angle, correctly rounded
		std::vector<float> freqs((size_t)half);
		for (int i = 0; i < half; i++) freqs[(size_t)i] = 1.0f / powf(theta, (float)(2 * i) / (float)hd);
		for (int p = 0; p < n_pos; p++)
			for (int d = 0; d < half; d++) {
				const float ang = (float)p * freqs[(size_t)d];
				c[(size_t)p * half + d] = (float)cos((double)ang);
				s[(size_t)p * half + d] = (float)sin((double)ang);
			}
	}
	if (int rc = upload_floats(cos_d, c.data(), c.size())) return rc;
	return upload_floats(sin_d, s.data(), s.size());
}

void tg_session_destroy(tg_session *s) {
	if (!s) return;
	(void)hipStreamSynchronize(g_stream);
	for (auto &kv : s->graphs) (void)hipGraphExecDestroy(kv.second);
	s->graphs.clear();
	for (auto &kv : s->pgraphs) {
		if (kv.second.exec) (void)hipGraphExecDestroy(kv.second.exec);
		if (kv.second.graph) (void)hipGraphDestroy(kv.second.graph);
	}
	s->pgraphs.clear();
	void *ps[] = {s->cos_g, s->sin_g, s->cos_l, s->sin_l, s->lut, s->xr, s->qkv, s->attn_out, s->o_out, s->hbuf, s->d_out,
	              s->logits, s->part_acc, s->part_ml, s->merged_acc, s->merged_ml, s->blk_val, s->blk_idx, s->ctr,
	              s->tok_log, s->pf_ws, s->probs, s->seg, s->bsum, s->bmax, s->randf, s->zeros, s->blk_x, s->blk_y, s->fused_layers,
	              s->fused_xch, s->fused_sync};
	for (void *p : ps)
		if (p) (void)hipFree(p);
	s->pf_plan.release();
	s->pf_plan_local.release();
	for (float *p : s->kc)
		if (p) (void)hipFree(p);
	for (float *p : s->vc)
		if (p) (void)hipFree(p);
	if (s->counted) {
		tg_model *m = s->m;
		m->n_sessions -= 1;
		if (m->orphaned && m->n_sessions == 0) delete m;
	}
	delete s;
}

int tg_session_create(tg_model *m, const float *rope_cos, const float *rope_sin, const float *rope_sw_cos,
                      const float *rope_sw_sin, const float *gelu_table, float gelu_min, float gelu_max, int gelu_size,
                      tg_session **out) {
	if (!m || !out) return tg_fail(TG_ERR_BAD_ARG, "null argument");
	if (!m->loaded) return tg_fail(TG_ERR_STATE, "model has no weights");
	if (gelu_size < 1 || !(gelu_max > gelu_min)) return tg_fail(TG_ERR_BAD_ARG, "bad GeLU table range");
	const tg_config &c = m->cfg;
	tg_session *s = new tg_session();
	s->m = m;
	int rc = TG_OK;
	auto fail = [&](int code) {
		tg_session_destroy(s);
		return code;
	};
	if ((rc = upload_rope(&s->cos_g, &s->sin_g, rope_cos, rope_sin, c.rope_theta, c.n_pos, c.head_dim))) return fail(rc);
	if ((rc = upload_rope(&s->cos_l, &s->sin_l, rope_sw_cos, rope_sw_sin, c.rope_theta_local, c.n_pos, c.head_dim))) return fail(rc);
	// lut::GeLUTable, ops.hpp:29-39
	s->gmin = gelu_min;
	s->geps = (float)(gelu_max - gelu_min) / (float)gelu_size;
	s->lut_size = gelu_size;
	{
		std::vector<float> t((size_t)gelu_size);
		if (gelu_table) {
			memcpy(t.data(), gelu_table, sizeof(float) * (size_t)gelu_size);
		} else {
			const float c0 = 0.7978845608f, c1 = 0.044715f;
			for (int i = 0; i < gelu_size; i++) {
				const float x = gelu_min + (float)i * s->geps;
				const double a = (double)x;
				t[(size_t)i] = (float)((0.5 * a) * (1.0 + tanh((double)c0 * (a + (double)c1 * (a * a * a)))));
			}
		}
		if ((rc = upload_floats(&s->lut, t.data(), t.size()))) return fail(rc);
	}
	const int L = c.n_layers, h = c.hidden_size, hd = c.head_dim, qo = c.n_head * hd;
	s->kc.assign((size_t)L, nullptr);
	s->vc.assign((size_t)L, nullptr);
	s->max_pos.assign((size_t)L, 0);
	for (int l = 0; l < L; l++) {
		const int mp = m->L[(size_t)l].is_sw ? c.n_pos_local : c.n_pos;  // decode.hpp:30
		s->max_pos[(size_t)l] = mp;
		const size_t bytes = sizeof(float) * (size_t)mp * hd;
		if (hipMalloc((void **)&s->kc[(size_t)l], bytes) != hipSuccess || hipMalloc((void **)&s->vc[(size_t)l], bytes) != hipSuccess)
			return fail(tg_fail(TG_ERR_HIP, "KV cache allocation failed"));
	}
	s->tok_log_cap = c.n_pos + 1;
#define TG_ALLOC(ptr, bytes)                                                                         \
	if (hipMalloc((void **)&(ptr), (bytes)) != hipSuccess) return fail(tg_fail(TG_ERR_HIP, "session allocation failed: " #ptr))
	TG_ALLOC(s->xr, sizeof(float) * (size_t)(2 * L + 1) * h);
	TG_ALLOC(s->qkv, sizeof(float) * (size_t)(qo + 2 * hd));
	TG_ALLOC(s->attn_out, sizeof(float) * (size_t)qo);
	TG_ALLOC(s->o_out, sizeof(float) * (size_t)h);
	TG_ALLOC(s->hbuf, sizeof(float) * (size_t)c.intermediate_size);
	TG_ALLOC(s->d_out, sizeof(float) * (size_t)h);
	TG_ALLOC(s->logits, sizeof(float) * (size_t)c.n_vocab);
	TG_ALLOC(s->part_acc, sizeof(float) * (size_t)ATTN_MAX_BLOCKS * c.n_head * hd);
	TG_ALLOC(s->part_ml, sizeof(float) * (size_t)ATTN_MAX_BLOCKS * c.n_head * 2);
	TG_ALLOC(s->merged_acc, sizeof(float) * (size_t)TG_ATTN_MERGE_MAX * c.n_head * hd);
	TG_ALLOC(s->merged_ml, sizeof(float) * (size_t)TG_ATTN_MERGE_MAX * c.n_head * 2);
	TG_ALLOC(s->blk_val, sizeof(float) * (size_t)m->lm.ntiles);
	TG_ALLOC(s->blk_idx, sizeof(int) * (size_t)m->lm.ntiles);
	TG_ALLOC(s->ctr, sizeof(int) * 8);
	TG_ALLOC(s->tok_log, sizeof(int) * (size_t)s->tok_log_cap);
	TG_ALLOC(s->zeros, sizeof(float) * (size_t)h);
	TG_ALLOC(s->blk_x, sizeof(float) * (size_t)h);
	TG_ALLOC(s->blk_y, sizeof(float) * (size_t)h);
#undef TG_ALLOC
	if (hipMemset(s->zeros, 0, sizeof(float) * (size_t)h) != hipSuccess) return fail(tg_fail(TG_ERR_HIP, "hipMemset failed"));
	if ((rc = tg_session_reset(s))) return fail(rc);
	m->n_sessions += 1;
	s->counted = true;
	*out = s;
	return TG_OK;
}

int tg_session_reset(tg_session *s) {
	if (!s) return tg_fail(TG_ERR_BAD_ARG, "null session");
	const tg_config &c = s->m->cfg;
	TG_HIP(hipStreamSynchronize(g_stream));
	for (size_t l = 0; l < s->kc.size(); l++) {
		const size_t bytes = sizeof(float) * (size_t)s->max_pos[l] * c.head_dim;
		TG_HIP(hipMemset(s->kc[l], 0, bytes));
		TG_HIP(hipMemset(s->vc[l], 0, bytes));
	}
	TG_HIP(hipMemset(s->ctr, 0, sizeof(int) * 8));
	TG_HIP(hipMemset(s->xr, 0, sizeof(float) * (size_t)(2 * c.n_layers + 1) * c.hidden_size));
	TG_HIP(hipDeviceSynchronize());
	s->pos = s->bp_local = s->bp_global = s->steps = 0;
	s->pick_pending = false;
	s->taps = nullptr;
	s->tap_rows = 0;
	return TG_OK;
}

int tg_session_position(const tg_session *s) { return s ? s->pos : -1; }

// ---------------------------------------------------------------------------------------------
// forward_decode: 5 launches per layer + 1 for the head
// ---------------------------------------------------------------------------------------------
// Keys per attention workgroup.  While TG_ATTN_MERGE_MAX workgroups of at most g_attn_merge_chunk keys cover the
// context, the output projection merges their partials in its prologue.  Longer contexts are bound by how long one
// workgroup walks its keys, so they are spread over up to TG_ATTN_MAX_BLOCKS workgroups (32 keys each or more) and a
// merge launch folds every TG_ATTN_FOLD partials into one first: the extra launch costs less than a few dozen keys per workgroup.
static int attn_chunk_for(int valid, bool *needs_merge) {
	auto up16 = [](int x) { return (x + 15) / 16 * 16; };
	const int c = up16((valid + TG_ATTN_MERGE_MAX - 1) / TG_ATTN_MERGE_MAX);
	*needs_merge = c > g_attn_merge_chunk;
	if (!*needs_merge) return c;
	return std::max(32, up16((valid + TG_ATTN_MAX_BLOCKS - 1) / TG_ATTN_MAX_BLOCKS));
}

// Event pool for tg_decode_profile: one event before every launch of a step plus one at the end.
struct StepProfile {
	std::vector<hipEvent_t> ev;
	std::vector<int> cls;
	size_t used = 0;
	hipError_t mark(int kernel_class) {
		if (used == ev.size()) {
			hipEvent_t e;
			hipError_t rc = hipEventCreate(&e);
			if (rc != hipSuccess) return rc;
			ev.push_back(e);
			cls.push_back(0);
		}
		cls[used] = kernel_class;
		return hipEventRecord(ev[used++], g_stream);
	}
};

// For tg_debug_repeat_kernel: launch only the kernels of one class of one layer, `repeat` times.
struct StepOnly {
	int kclass, layer, repeat;
};

static int session_usable(const tg_session *s) {
	if (!s) return tg_fail(TG_ERR_BAD_ARG, "null session");
	if (!s->m || !s->m->loaded) return tg_fail(TG_ERR_STATE, "the session's model has no weights (destroyed, or a load failed)");
	return TG_OK;
}

// ---- the one-kernel decode step ---------------------------------------------------------------------------
static TgFusedMat fused_mat(const PackedMat &p) { return TgFusedMat{p.K, p.C, p.lc_shift, p.ntiles}; }

// Keys per attention workgroup of the fused step: TG_FUSED_ATTN_WGS workgroups cover the context.  Up to
// TG_ATTN_MERGE_MAX * g_attn_merge_chunk keys that is what the launch path does as well; 0: too many keys for it.
static int fused_chunk(int valid) {
	const int c = (valid + TG_FUSED_ATTN_WGS - 1) / TG_FUSED_ATTN_WGS;
	const int c16 = (c + 15) / 16 * 16;
	return c16 <= 256 ? c16 : 0;
}

// Builds the per-session tables of the fused step on first use.  Leaves fused_state at 1 (usable) or -1.
static int fused_prepare(tg_session *s) {
	if (s->fused_state != 0) return TG_OK;
	s->fused_state = -1;
	tg_model *m = s->m;
	const tg_config &c = m->cfg;
	const int L = c.n_layers;
	if (!tg_fused_supported(g_n_cu)) return TG_OK;
	TgFused &f = s->fused;
	memset(&f, 0, sizeof(f));
	f.L = L;
	f.hidden = c.hidden_size;
	f.mqkv = fused_mat(m->L[0].qkv);
	f.mo = fused_mat(m->L[0].o);
	f.mug = fused_mat(m->L[0].ug);
	f.md = fused_mat(m->L[0].d);
	auto al = [](int floats) { return (floats + 63) / 64 * 64; };  // regions start on 256-byte boundaries
	int off = 0;
	f.off_qkv = off;
	off += al(c.n_head * c.head_dim + 2 * c.head_dim);
	f.off_pacc = off;
	off += al(TG_FUSED_ATTN_WGS * c.n_head * c.head_dim);
	f.off_pml = off;
	off += al(TG_FUSED_ATTN_WGS * c.n_head * 2);
	f.off_o = off;
	off += al(c.hidden_size);
	f.off_h = off;
	off += al(c.intermediate_size);
	f.off_d = off;
	off += al(c.hidden_size);
	f.layer_stride = (size_t)off;
	std::vector<TgFusedLayer> hl((size_t)L);
	for (int l = 0; l < L; l++) {
		const LayerDev &Ld = m->L[(size_t)l];
		TgFusedLayer &o = hl[(size_t)l];
		o.Wqkv = Ld.qkv.W;
		o.Wo = Ld.o.W;
		o.Wug = Ld.ug.W;
		o.Wd = Ld.d.W;
		o.sqkv = Ld.qkv.scales;
		o.so = Ld.o.scales;
		o.sug = Ld.ug.scales;
		o.sd = Ld.d.scales;
		o.apre = Ld.apre;
		o.apost = Ld.apost;
		o.mpre = Ld.mpre;
		o.mpost = Ld.mpost;
		o.rms_q = Ld.rms_q;
		o.rms_k = Ld.rms_k;
		o.kc = s->kc[(size_t)l];
		o.vc = s->vc[(size_t)l];
		o.max_pos = s->max_pos[(size_t)l];
		o.is_sw = Ld.is_sw ? 1 : 0;
	}
	TG_HIP(hipMalloc((void **)&s->fused_layers, sizeof(TgFusedLayer) * (size_t)L));
	TG_HIP(hipMemcpy(s->fused_layers, hl.data(), sizeof(TgFusedLayer) * (size_t)L, hipMemcpyHostToDevice));
	TG_HIP(hipMalloc((void **)&s->fused_xch, sizeof(float) * f.layer_stride * (size_t)L));
	TG_HIP(hipMemset(s->fused_xch, 0, sizeof(float) * f.layer_stride * (size_t)L));
	TG_HIP(hipMalloc((void **)&s->fused_sync, sizeof(unsigned) * TG_FUSED_SYNC_WORDS));
	TG_HIP(hipMemset(s->fused_sync, 0, sizeof(unsigned) * TG_FUSED_SYNC_WORDS));
	s->fused_all = s->fused_attn = 0;
	f.layers = s->fused_layers;
	f.wte = m->wte;
	f.wte_scales = m->wte_scales;
	f.vocab = c.n_vocab;
	f.emb_scale = (float)sqrt((double)c.hidden_size);  // ops.hpp:586
	f.cos_g = s->cos_g;
	f.sin_g = s->sin_g;
	f.cos_l = s->cos_l;
	f.sin_l = s->sin_l;
	f.lut = s->lut;
	f.gmin = s->gmin;
	f.geps = s->geps;
	f.lut_size = s->lut_size;
	f.xr = s->xr;
	f.xch = s->fused_xch;
	f.sync = s->fused_sync;
	s->fused_state = 1;
	s->fused_epoch = g_knob_epoch - 1;  // the workgroup count and the kernel variant are chosen by fused_usable
	return TG_OK;
}

// Whether the next decode step of the session can run as one launch, and its attention geometry if so.
static bool fused_usable(tg_session *s, int *chunk_local, int *chunk_global) {
	if (!g_fused || s->fused_state != 1) return false;
	if (s->fused_epoch != g_knob_epoch) {  // the knobs have moved: workgroups of the launch, kernel instantiation
		s->fused_epoch = g_knob_epoch;
		s->fused.ng = g_fused_ng > 0 ? g_fused_ng : g_n_cu - TG_FUSED_ATTN_WGS;
		// one workgroup per compute unit, so that all of them are resident at once
		s->fused_variant = s->fused.ng + TG_FUSED_ATTN_WGS <= g_n_cu ? tg_fused_variant(s->fused) : -1;
	}
	if (s->fused_variant < 0) return false;
	const tg_config &c = s->m->cfg;
	*chunk_local = fused_chunk(std::min(s->pos + 1, c.n_pos_local));
	*chunk_global = fused_chunk(std::min(s->pos + 1, c.n_pos));
	return *chunk_local > 0 && *chunk_global > 0;
}

// The layers of a decode step as one launch; the LM head follows as a launch of its own.
static void launch_fused_layers(tg_session *s, int chunk_local, int chunk_global) {
	tg_model *m = s->m;
	const tg_config &c = m->cfg;
	TgFused f = s->fused;
	f.tok = s->ctr + 4;
	if (s->pick_pending) {  // this launch finishes the previous step's greedy pick
		f.am_val = s->blk_val;
		f.am_idx = s->blk_idx;
		f.am_n = m->lm.ntiles;
		f.am_ctr = s->ctr;
		f.am_log = s->tok_log;
		s->pick_pending = false;
	}
	f.pos = s->pos;
	f.bp_local = s->bp_local;
	f.bp_global = s->bp_global;
	f.chunk_local = chunk_local;
	f.chunk_global = chunk_global;
	f.all_base = s->fused_all;
	f.attn_base = s->fused_attn;
	f.max_spins = g_fused_spins;
	f.ts = g_fused_ts;
	tg_launch_decode_fused(f, s->fused_variant, g_stream);
	// what the launch adds to the counters: 4 arrivals of every GEMV workgroup per layer, one of every attention
	// workgroup that has keys
	s->fused_all += 4u * (unsigned)c.n_layers * (unsigned)f.ng;
	for (int l = 0; l < c.n_layers; l++) {
		const int valid = std::min(s->pos + 1, s->max_pos[(size_t)l]);
		const int ch = m->L[(size_t)l].is_sw ? chunk_local : chunk_global;
		s->fused_attn += (unsigned)((valid + ch - 1) / ch);
	}
	s->fused_unchecked = true;
}

// After a stream synchronisation: did a wait inside a fused launch give up?  Then the results since the last check are
// not valid; the session stays on the launch path from here on.
static int fused_check(tg_session *s) {
	if (!s->fused_unchecked) return TG_OK;
	s->fused_unchecked = false;
	unsigned err = 0;
	TG_HIP(hipMemcpy(&err, s->fused_sync + 16 * 32, sizeof(unsigned), hipMemcpyDeviceToHost));
	if (err == 0) return TG_OK;
	s->fused_state = -1;
	s->fused_all = s->fused_attn = 0;
	TG_HIP(hipMemset(s->fused_sync, 0, sizeof(unsigned) * TG_FUSED_SYNC_WORDS));
	return tg_fail(TG_ERR_STATE, "one-kernel decode step: a bounded wait between workgroups gave up (the workgroups were not all resident, or the device "
	                             "is shared); the decode steps since the last read-back are not valid.  Reset the session; it now uses one launch per projection");
}

// ---- the launches of a decode step, one function per kernel (modules.hpp:135-220, 242-246) ----
// Every projection's launch also does what precedes it in the reference's sequence: the post-norm + residual add of the
// block before it (`pend` = that block's output, `w_post` its post-norm weights, `x` the residual it is added to; the
// sum goes to `xr_out`) and its own pre-norm.  A `pend` of zeros adds nothing (its norm is 0), which is how the
// block-level entry points start a block from a caller's residual stream with the same kernels.

// pre-norm + Q|K|V of layer l (modules.hpp:137-144); embed: the residual is the embedding of the device-side token
static void launch_qkv(tg_session *s, int l, bool embed, const float *pend, const float *w_post, const float *x, float *xr_out) {
	tg_model *m = s->m;
	const tg_config &c = m->cfg;
	const LayerDev &Ld = m->L[(size_t)l];
	TgGemv g = gemv_base(Ld.qkv);
	g.hidden = c.hidden_size;
	g.w_pre = Ld.apre;
	g.xr_out = xr_out;
	g.y = s->qkv;
	g.pf = prefetch_of(Ld.o);
	if (g_prefetch_plan == 1) g.pf2 = prefetch_of(Ld.ug);
	if (embed) {
		g.wte = m->wte;
		g.wte_scales = m->wte_scales;
		g.tok = s->ctr + 4;
		if (s->pick_pending) {  // this launch finishes the previous step's greedy pick
			g.am_val = s->blk_val;
			g.am_idx = s->blk_idx;
			g.am_n = m->lm.ntiles;
			g.am_ctr = s->ctr;
			g.am_log = s->tok_log;
			s->pick_pending = false;
		}
		g.vocab = c.n_vocab;
		g.emb_scale = (float)sqrt((double)c.hidden_size);  // ops.hpp:586
		tg_launch_gemv(g, TG_ROLE_QKV_EMBED, g_stream);
	} else {
		g.pend = pend;
		g.w_post = w_post;
		g.x = x;
		tg_launch_gemv(g, TG_ROLE_QKV, g_stream);
	}
}

// Attention launch geometry of layer l at the session's position.
struct AttnGeom {
	TgAttnDecode a;
	bool needs_merge;
	int nblk;
};
static AttnGeom attn_geometry(tg_session *s, int l, bool full_grid) {
	const tg_config &c = s->m->cfg;
	const LayerDev &Ld = s->m->L[(size_t)l];
	AttnGeom ag;
	TgAttnDecode &a = ag.a;
	memset(&a, 0, sizeof(a));
	a.qkv = s->qkv;
	a.rms_q = Ld.rms_q;
	a.rms_k = Ld.rms_k;
	a.cos_t = Ld.is_sw ? s->cos_l : s->cos_g;
	a.sin_t = Ld.is_sw ? s->sin_l : s->sin_g;
	a.kc = s->kc[(size_t)l];
	a.vc = s->vc[(size_t)l];
	a.max_pos = s->max_pos[(size_t)l];
	a.pos = s->ctr;
	a.bp_index = Ld.is_sw ? 1 : 2;
	// a captured step is replayed at other positions: only then are the counters read from device memory
	a.host_pos = full_grid ? -1 : s->pos;
	a.host_bp = full_grid ? -1 : (Ld.is_sw ? s->bp_local : s->bp_global);
	a.host_cur = full_grid ? -1 : a.host_bp % a.max_pos;
	const int valid = std::min(s->pos + 1, a.max_pos);
	ag.needs_merge = false;
	a.chunk = attn_chunk_for(valid, &ag.needs_merge);
	a.part_acc = s->part_acc;
	a.part_ml = s->part_ml;
	a.n_head = c.n_head;
	a.pf = prefetch_of(g_prefetch_plan == 1 ? Ld.d : Ld.ug);
	// a captured step is replayed at later positions with the same chunk: launch the largest grid that
	// chunk can need (workgroups past the valid keys exit at once)
	ag.nblk = full_grid ? (ag.needs_merge ? std::min(TG_ATTN_MAX_BLOCKS, (a.max_pos + a.chunk - 1) / a.chunk) : TG_ATTN_MERGE_MAX)
	                    : (valid + a.chunk - 1) / a.chunk;
	return ag;
}
// q/k norm, RoPE, KV write, attention partials (modules.hpp:146-161); the merge launch on long contexts
static void launch_attn(tg_session *s, const AttnGeom &ag) {
	tg_launch_attn_decode(ag.a, ag.nblk, g_stream);
	if (ag.needs_merge) tg_launch_attn_merge(ag.a, ag.nblk, s->merged_acc, s->merged_ml, g_stream);
}
// merge of the attention partials + O projection (modules.hpp:161-164)
static TgGemv oproj_gemv(tg_session *s, int l, const AttnGeom &ag) {
	const LayerDev &Ld = s->m->L[(size_t)l];
	TgGemv g = gemv_base(Ld.o);
	g.pos = s->ctr;
	g.host_pos = ag.a.host_pos;
	g.attn_max_pos = ag.a.max_pos;
	g.attn_chunk = ag.needs_merge ? TG_ATTN_FOLD * ag.a.chunk : ag.a.chunk;  // folded: one partial per TG_ATTN_FOLD workgroups
	g.part_acc = ag.needs_merge ? s->merged_acc : s->part_acc;
	g.part_ml = ag.needs_merge ? s->merged_ml : s->part_ml;
	g.y = s->o_out;
	if (g_prefetch_plan == 0) g.pf = prefetch_of(Ld.d);
	return g;
}
static void launch_oproj(tg_session *s, int l, const AttnGeom &ag) { tg_launch_gemv(oproj_gemv(s, l, ag), TG_ROLE_OPROJ, g_stream); }
// post-norm + residual of the attention block, pre-norm, up|gate, gelu(gate)*up (modules.hpp:166-168, 205-215)
static void launch_upgate(tg_session *s, int l, const float *pend, const float *x, float *xr_out) {
	tg_model *m = s->m;
	const LayerDev &Ld = m->L[(size_t)l];
	TgGemv g = gemv_base(Ld.ug);
	g.hidden = m->cfg.hidden_size;
	g.pend = pend;
	g.w_post = Ld.apost;
	g.x = x;
	g.xr_out = xr_out;
	g.w_pre = Ld.mpre;
	g.y = s->hbuf;
	g.lut = s->lut;
	g.gmin = s->gmin;
	g.geps = s->geps;
	g.lut_size = s->lut_size;
	if (l + 1 < m->cfg.n_layers) g.pf = prefetch_of(m->L[(size_t)l + 1].qkv);
	tg_launch_gemv(g, TG_ROLE_UPGATE, g_stream);
}
// down projection (modules.hpp:216-217)
static void launch_down(tg_session *s, int l) {
	TgGemv g = gemv_base(s->m->L[(size_t)l].d);
	g.x = s->hbuf;
	g.y = s->d_out;
	tg_launch_gemv(g, TG_ROLE_DOWN, g_stream);
}
// last post-norm + residual, final norm, LM head, first stage of the argmax (modules.hpp:242-246, ops.hpp:744)
static void launch_lmhead(tg_session *s, const float *pend, const float *w_post, const float *x, float *xr_out) {
	tg_model *m = s->m;
	TgGemv g = gemv_base(m->lm);
	g.hidden = m->cfg.hidden_size;
	g.pend = pend;
	g.w_post = w_post;
	g.x = x;
	g.xr_out = xr_out;
	g.w_pre = m->rmsw;
	g.y = s->logits;
	g.blk_val = s->blk_val;
	g.blk_idx = s->blk_idx;
	tg_launch_gemv(g, TG_ROLE_LMHEAD, g_stream);
}

// The finishing launch of a pending greedy pick (see tg_session::pick_pending).
static void flush_pick(tg_session *s) {
	if (!s->pick_pending) return;
	tg_launch_argmax_finish(s->blk_val, s->blk_idx, s->m->lm.ntiles, s->ctr, s->tok_log, 1, g_stream);
	s->pick_pending = false;
}

// One decode step.  chain: the greedy pick may stay pending for the next step's first launch to finish (the caller
// flushes after its last step); otherwise the step ends with the finishing launch.
static int enqueue_decode_step(tg_session *s, StepProfile *prof, bool full_grid, const StepOnly *only = nullptr, bool chain = false) {
	if (int rc = session_usable(s)) return rc;
	tg_model *m = s->m;
	const tg_config &c = m->cfg;
	const int L = c.n_layers, h = c.hidden_size;
	if (s->pos >= c.n_pos) return tg_fail(TG_ERR_STATE, "context is full (n_pos)");
	if (s->steps >= s->tok_log_cap) return tg_fail(TG_ERR_STATE, "token log is full");
#define TG_DO(k, l, stmt)                                                        \
	if (!only || (only->kclass == (k) && only->layer == (l)))                        \
		for (int r_ = 0; r_ < (only ? only->repeat : 1); r_++) {                     \
			stmt;                                                                    \
		}
#define TG_MARK(k)                                 \
	if (prof) {                                    \
		TG_HIP(prof->mark(k));                     \
	}
	// all layers in one launch where that is possible (not when single kernels are timed or repeated, not in a captured step)
	int fch_l = 0, fch_g = 0;
	bool fused = false;
	if (g_fused && !prof && !only && !full_grid) {
		if (int rc = fused_prepare(s)) return rc;
		fused = fused_usable(s, &fch_l, &fch_g);
	}
	const float *last_pend = s->d_out;
	if (fused) {
		launch_fused_layers(s, fch_l, fch_g);
		last_pend = s->fused_xch + (size_t)(L - 1) * s->fused.layer_stride + s->fused.off_d;
	}
	for (int l = 0; l < L && !fused; l++) {
		float *xr_in = s->xr + (size_t)(2 * l) * h, *xr_mid = s->xr + (size_t)(2 * l + 1) * h;
		TG_MARK(TG_KC_QKV);
		if (l == 0) {
			TG_DO(TG_KC_QKV, l, launch_qkv(s, l, true, nullptr, nullptr, nullptr, xr_in));
		} else {
			TG_DO(TG_KC_QKV, l, launch_qkv(s, l, false, s->d_out, m->L[(size_t)l - 1].mpost, s->xr + (size_t)(2 * l - 1) * h, xr_in));
		}
		const AttnGeom ag = attn_geometry(s, l, full_grid);
		TG_MARK(TG_KC_ATTN);
		TG_DO(TG_KC_ATTN, l, launch_attn(s, ag));
		TG_MARK(TG_KC_OPROJ);
		TG_DO(TG_KC_OPROJ, l, launch_oproj(s, l, ag));
		TG_MARK(TG_KC_UPGATE);
		TG_DO(TG_KC_UPGATE, l, launch_upgate(s, l, s->o_out, xr_in, xr_mid));
		TG_MARK(TG_KC_DOWN);
		TG_DO(TG_KC_DOWN, l, launch_down(s, l));
	}
	TG_MARK(TG_KC_LMHEAD);
	TG_DO(TG_KC_LMHEAD, 0, launch_lmhead(s, last_pend, m->L[(size_t)L - 1].mpost, s->xr + (size_t)(2 * L - 1) * h, s->xr + (size_t)(2 * L) * h));
	TG_MARK(TG_KC_ARGMAX);
	if (!only) {
		if (s->sampling)
			tg_launch_minp(s->logits, c.n_vocab, s->s_minp, s->s_temp, s->randf, -1, s->rand_base, s->probs, s->seg, s->bsum, s->bmax,
			               s->ctr, s->tok_log, 0, nullptr, g_stream);
		else if (chain && !prof && !full_grid)
			s->pick_pending = true;
		else
			tg_launch_argmax_finish(s->blk_val, s->blk_idx, m->lm.ntiles, s->ctr, s->tok_log, 1, g_stream);
	}
	TG_MARK(-1);
#undef TG_MARK
#undef TG_DO
	TG_HIP(hipGetLastError());
	if (only) return TG_OK;
	s->pos += 1;
	s->bp_local += 1;
	s->bp_global += 1;
	s->steps += 1;
	return TG_OK;
}


int tg_forward_decode(tg_session *s, int32_t id, float *logits, int32_t *argmax) {
	if (int rc = session_usable(s)) return rc;
	TG_HIP(hipMemcpyAsync(s->ctr + 4, &id, sizeof(int), hipMemcpyHostToDevice, g_stream));
	if (int rc = enqueue_decode_step(s, nullptr, false)) return rc;
	if (logits) TG_HIP(hipMemcpyAsync(logits, s->logits, sizeof(float) * (size_t)s->m->cfg.n_vocab, hipMemcpyDeviceToHost, g_stream));
	int32_t tok = -1;
	TG_HIP(hipMemcpyAsync(&tok, s->ctr + 4, sizeof(int), hipMemcpyDeviceToHost, g_stream));
	TG_HIP(hipStreamSynchronize(g_stream));
	if (int rc = fused_check(s)) return rc;
	if (argmax) *argmax = tok;
	if (s->taps) {  // taps now describe the decode step
		s->taps = nullptr;
		s->tap_rows = 0;
	}
	return TG_OK;
}

static uint64_t decode_graph_key(const tg_session *s) {
	const tg_config &c = s->m->cfg;
	bool ml = false, mg = false;
	const int cl = attn_chunk_for(std::min(s->pos + 1, c.n_pos_local), &ml);
	const int cg = attn_chunk_for(std::min(s->pos + 1, c.n_pos), &mg);
	return (uint64_t)cl | ((uint64_t)ml << 15) | ((uint64_t)cg << 16) | ((uint64_t)mg << 31);
}

static void session_drop_graphs(tg_session *s) {
	for (auto &kv : s->graphs) (void)hipGraphExecDestroy(kv.second);
	s->graphs.clear();
	for (auto &kv : s->pgraphs) {
		if (kv.second.exec) (void)hipGraphExecDestroy(kv.second.exec);
		if (kv.second.graph) (void)hipGraphDestroy(kv.second.graph);
	}
	s->pgraphs.clear();
}

// ---- graph replay, mode 2 ----------------------------------------------------------------------------------------
// A decode step captured with the launches of the stream path (position known on the host: exact grids, nothing read
// from the device-side counters in front of a kernel's loads).  Three launches per layer depend on the position: the
// attention (grid, chunk, ring slot, RoPE row), its merge launch where there is one, and the output projection (number
// of partials).  Their nodes are looked up once in the captured graph and given new parameters before every replay;
// everything else in a step is position independent.  The host then issues one graph launch and 2-3 node updates per
// layer instead of 5-6 kernel launches: a decode step of the 270m shape, 91 launches of 3.6 us on the device, is bound
// by the host's launch rate whenever the launching thread sits on a slow core (2.5 or 4.2 us per launch: 3,070 or
// 2,500-2,600 tok/s from process to process).
constexpr int TG_GRAPH_STEPS = 4;  // decode steps per replayed graph where a batch has that many left (a graph launch costs the device 5-6 us;
                                   // graphs of two and three steps for the tails would be further kinds to capture on first use)

// which layer kinds have a merge launch at the session's position + ahead
static uint64_t patched_graph_topology(const tg_session *s, int ahead) {
	const tg_config &c = s->m->cfg;
	bool ml = false, mg = false;
	(void)attn_chunk_for(std::min(s->pos + ahead + 1, c.n_pos_local), &ml);
	(void)attn_chunk_for(std::min(s->pos + ahead + 1, c.n_pos), &mg);
	return (uint64_t)ml | ((uint64_t)mg << 1);
}
// A graph is one of: which layers merge, whether picks are chained, whether a pick is pending when its first step starts
// (that step's first launch then finishes it; the first step of a batch has none), how many steps it holds.
static uint64_t patched_graph_key(const tg_session *s, bool chained, int nsteps) {
	return patched_graph_topology(s, 0) | ((uint64_t)chained << 2) | ((uint64_t)s->pick_pending << 3) | ((uint64_t)nsteps << 4);
}

// Captures nsteps consecutive steps.  chained: a step's first launch finishes the greedy pick that is pending when it
// starts, if any, and its own pick stays pending (the caller flushes after its last step); else every step ends with
// the finishing launch.
static int patched_graph_capture(tg_session *s, tg_session::PatchedGraph *pg, bool chained, int nsteps) {
	const int L = s->m->cfg.n_layers, pos0 = s->pos;
	pg->steps = nsteps;
	TG_HIP(hipStreamBeginCapture(g_stream, hipStreamCaptureModeThreadLocal));
	int rc = TG_OK;
	for (int k = 0; k < nsteps && rc == TG_OK; k++) rc = enqueue_decode_step(s, nullptr, false, nullptr, chained);  // advances the host mirrors
	const hipError_t e = hipStreamEndCapture(g_stream, &pg->graph);
	if (rc != TG_OK) return rc;
	if (e != hipSuccess) return tg_fail(TG_ERR_HIP, std::string("hipStreamEndCapture: ") + hipGetErrorString(e));
	size_t n = 0;
	TG_HIP(hipGraphGetNodes(pg->graph, nullptr, &n));
	std::vector<hipGraphNode_t> nodes(n);
	TG_HIP(hipGraphGetNodes(pg->graph, nodes.data(), &n));
	pg->attn.assign((size_t)(nsteps * L), nullptr);
	pg->merge.assign((size_t)(nsteps * L), nullptr);
	pg->oproj.assign((size_t)(nsteps * L), nullptr);
	for (hipGraphNode_t node : nodes) {
		hipGraphNodeType type;
		TG_HIP(hipGraphNodeGetType(node, &type));
		if (type != hipGraphNodeTypeKernel) continue;
		hipKernelNodeParams kp;
		TG_HIP(hipGraphKernelNodeGetParams(node, &kp));
		const int kind = tg_decode_node_kind(kp.func);
		if (kind == 0 || kp.kernelParams == nullptr) continue;
		// which layer: by the cache (attention, merge) or the weights (projection) the node's descriptor names; which
		// step: by the position it was captured with
		int layer = -1, step = -1;
		if (kind == 3) {
			const TgGemv *g = static_cast<const TgGemv *>(kp.kernelParams[9]);
			for (int l = 0; l < L; l++)
				if (g->W == s->m->L[(size_t)l].o.W) layer = l;
			step = g->host_pos - pos0;
		} else {
			const TgAttnDecode *a = static_cast<const TgAttnDecode *>(kp.kernelParams[kind == 1 ? 9 : 0]);
			for (int l = 0; l < L; l++)
				if (a->kc == s->kc[(size_t)l]) layer = l;
			step = a->host_pos - pos0;
		}
		if (layer < 0 || step < 0 || step >= nsteps) return tg_fail(TG_ERR_STATE, "graph replay: a captured node names no layer or step of this capture");
		std::vector<hipGraphNode_t> &slot = kind == 1 ? pg->attn : (kind == 2 ? pg->merge : pg->oproj);
		if (slot[(size_t)(step * L + layer)] != nullptr) return tg_fail(TG_ERR_STATE, "graph replay: two captured nodes for one launch");
		slot[(size_t)(step * L + layer)] = node;
	}
	for (int i = 0; i < nsteps * L; i++)
		if (pg->attn[(size_t)i] == nullptr || pg->oproj[(size_t)i] == nullptr)
			return tg_fail(TG_ERR_STATE, "graph replay: the captured steps lack a layer's attention or projection node");
	const hipError_t e2 = hipGraphInstantiate(&pg->exec, pg->graph, nullptr, nullptr, 0);
	if (e2 != hipSuccess) return tg_fail(TG_ERR_HIP, std::string("hipGraphInstantiate: ") + hipGetErrorString(e2));
	return TG_OK;
}

// New parameters for the position-dependent nodes of every step of the graph; advances the host mirrors by its steps.
static int patched_graph_update(tg_session *s, const tg_session::PatchedGraph &pg) {
	const int L = s->m->cfg.n_layers;
	TgLaunchDesc d;
	auto set = [&](hipGraphNode_t node) -> hipError_t {
		hipKernelNodeParams kp;
		memset(&kp, 0, sizeof(kp));
		kp.func = const_cast<void *>(d.func);
		kp.gridDim = d.grid;
		kp.blockDim = d.block;
		kp.sharedMemBytes = 0;
		kp.kernelParams = d.args;
		kp.extra = nullptr;
		return hipGraphExecKernelNodeSetParams(pg.exec, node, &kp);
	};
	for (int k = 0; k < pg.steps; k++) {
		for (int l = 0; l < L; l++) {
			const size_t at = (size_t)(k * L + l);
			const AttnGeom ag = attn_geometry(s, l, false);
			tg_desc_attn_decode(ag.a, ag.nblk, &d);
			TG_HIP(set(pg.attn[at]));
			if (ag.needs_merge != (pg.merge[at] != nullptr)) return tg_fail(TG_ERR_STATE, "graph replay: the step's launches differ from the captured ones");
			if (ag.needs_merge) {
				tg_desc_attn_merge(ag.a, ag.nblk, s->merged_acc, s->merged_ml, &d);
				TG_HIP(set(pg.merge[at]));
			}
			tg_desc_gemv(oproj_gemv(s, l, ag), TG_ROLE_OPROJ, &d);
			TG_HIP(set(pg.oproj[at]));
		}
		s->pos += 1;
		s->bp_local += 1;
		s->bp_global += 1;
		s->steps += 1;
	}
	return TG_OK;
}

// nsteps steps from one graph launch; the caller has checked that they fit the context and the token log and that all of
// them have the launches of the first
static int enqueue_patched_graph_steps(tg_session *s, bool chained, int nsteps) {
	const uint64_t key = patched_graph_key(s, chained, nsteps);
	auto it = s->pgraphs.find(key);
	if (it == s->pgraphs.end()) {
		tg_session::PatchedGraph pg;
		const int rc = patched_graph_capture(s, &pg, chained, nsteps);  // the captured steps hold these positions' parameters
		if (rc != TG_OK) {
			if (pg.exec) (void)hipGraphExecDestroy(pg.exec);
			if (pg.graph) (void)hipGraphDestroy(pg.graph);
			return rc;
		}
		s->pgraphs[key] = pg;
		TG_HIP(hipGraphLaunch(pg.exec, g_stream));
		return TG_OK;
	}
	if (int rc = patched_graph_update(s, it->second)) return rc;
	TG_HIP(hipGraphLaunch(it->second.exec, g_stream));
	if (chained) s->pick_pending = true;  // as the captured steps left it: the last step's pick waits for the next step or the flush
	return TG_OK;
}

static bool profiler_attached();
// The mode a session's greedy steps take.  Left to the library (-1), a model whose decode step streams less than 5 MB of
// weights per launch replays updated graphs: the device then needs less time per launch (3.6 us for the 270m shape's
// 3 MB) than a host core that is slow or shared needs to issue one (2.5 us at best, 4.2-4.4 us on other cores of the same
// machine), and the step would follow the host.  The 1B shape (7.7 MB, 4.6 us per launch) stays ahead of the host either
// way and keeps its stream launches (as fast there as the replay).  Never graphs under a profiler.
static int decode_graph_mode_of(const tg_config &c) {
	if (g_use_graphs >= 0) return g_use_graphs;
	if (profiler_attached()) return 0;
	const double h = c.hidden_size, qo = (double)c.n_head * c.head_dim, kv = (double)c.n_kv * c.head_dim, f = c.intermediate_size;
	const double bytes = c.n_layers * (h * (qo + 2 * kv) + qo * h + 3 * h * f) + h * c.n_vocab;
	return bytes / (5.0 * c.n_layers + 1.0) < 5e6 ? 2 : 0;
}
static int decode_graph_mode(const tg_session *s) { return decode_graph_mode_of(s->m->cfg); }

int tg_plan_decode_launch_mode(const tg_config *cfg) {
	if (!cfg || cfg->n_layers < 1) return -1;
	return decode_graph_mode_of(*cfg);
}

int tg_decode_enqueue(tg_session *s, int n_steps) {
	if (!s || n_steps < 0) return tg_fail(TG_ERR_BAD_ARG, "bad argument");
	if (int rc = session_usable(s)) return rc;
	const tg_config &c = s->m->cfg;
	const int graph_mode = decode_graph_mode(s);
	if (graph_mode && s->graph_epoch != g_knob_epoch) {
		// the graphs captured so far hold the launch parameters of other knob settings
		TG_HIP(hipStreamSynchronize(g_stream));
		session_drop_graphs(s);
		s->graph_epoch = g_knob_epoch;
	}
	for (int i = 0; i < n_steps; i++) {
		if (!graph_mode || (graph_mode == 2 && g_fused)) {
			if (int rc = enqueue_decode_step(s, nullptr, false, nullptr, g_chain_picks)) {
				flush_pick(s);
				return rc;
			}
			continue;
		}
		if (graph_mode == 2) {
			// With chained picks a step's pick stays pending for the next step or the flush below; the first step of a
			// batch, which has no pick to finish, is a graph of its own kind.
			int rc;
			if (s->graphs_failed) {
				rc = enqueue_decode_step(s, nullptr, false, nullptr, g_chain_picks);
			} else {
				// a capture or a node update the runtime refuses leaves nothing enqueued: the session's counters go back
				// and this and all later steps of the session are plain launches
				if (s->pos >= c.n_pos) rc = tg_fail(TG_ERR_STATE, "context is full (n_pos)");
				else if (s->steps >= s->tok_log_cap) rc = tg_fail(TG_ERR_STATE, "token log is full");
				else {
					// several steps per graph launch where the batch, the context and the token log have room for them and
					// none of them changes which layers have a merge launch
					// (the first step of a batch goes out alone: the device would otherwise wait until the host has updated the
					// nodes of four steps, 0.4 ms, before it sees the first launch)
					int ns = 1;
					if (i > 0 && n_steps - i >= TG_GRAPH_STEPS && s->pos + TG_GRAPH_STEPS <= c.n_pos && s->steps + TG_GRAPH_STEPS <= s->tok_log_cap) {
						ns = TG_GRAPH_STEPS;
						for (int k = 1; k < TG_GRAPH_STEPS; k++)
							if (patched_graph_topology(s, k) != patched_graph_topology(s, 0)) ns = 1;
					}
					const int pos = s->pos, bpl = s->bp_local, bpg = s->bp_global, steps = s->steps;
					const bool pending = s->pick_pending;
					rc = enqueue_patched_graph_steps(s, g_chain_picks, ns);
					if (rc == TG_OK) {
						i += ns - 1;
					} else if (rc == TG_ERR_HIP || rc == TG_ERR_STATE) {
						(void)hipGetLastError();
						s->pos = pos;
						s->bp_local = bpl;
						s->bp_global = bpg;
						s->steps = steps;
						s->pick_pending = pending;
						s->graphs_failed = true;
						rc = enqueue_decode_step(s, nullptr, false, nullptr, g_chain_picks);
					}
				}
			}
			if (rc != TG_OK) {
				flush_pick(s);
				return rc;
			}
			continue;
		}
		// One HIP graph per attention launch geometry; every other launch parameter of a decode step
		// is position independent (positions and the token id live in device memory).
		const uint64_t key = decode_graph_key(s);
		auto it = s->graphs.find(key);
		if (it == s->graphs.end()) {
			TG_HIP(hipStreamBeginCapture(g_stream, hipStreamCaptureModeThreadLocal));
			const int rc = enqueue_decode_step(s, nullptr, true);  // advances the host mirrors once
			hipGraph_t graph = nullptr;
			const hipError_t e = hipStreamEndCapture(g_stream, &graph);
			if (rc != TG_OK) {
				if (graph) (void)hipGraphDestroy(graph);
				return rc;
			}
			if (e != hipSuccess) return tg_fail(TG_ERR_HIP, std::string("hipStreamEndCapture: ") + hipGetErrorString(e));
			hipGraphExec_t exec = nullptr;
			const hipError_t e2 = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0);
			(void)hipGraphDestroy(graph);
			if (e2 != hipSuccess) return tg_fail(TG_ERR_HIP, std::string("hipGraphInstantiate: ") + hipGetErrorString(e2));
			s->graphs[key] = exec;
			TG_HIP(hipGraphLaunch(exec, g_stream));
		} else {
			if (s->pos >= c.n_pos) return tg_fail(TG_ERR_STATE, "context is full (n_pos)");
			if (s->steps >= s->tok_log_cap) return tg_fail(TG_ERR_STATE, "token log is full");
			TG_HIP(hipGraphLaunch(it->second, g_stream));
			s->pos += 1;
			s->bp_local += 1;
			s->bp_global += 1;
			s->steps += 1;
		}
	}
	flush_pick(s);
	TG_HIP(hipGetLastError());
	if (s->taps) {
		TG_HIP(hipStreamSynchronize(g_stream));
		s->taps = nullptr;
		s->tap_rows = 0;
	}
	return TG_OK;
}

int tg_debug_repeat_kernel(tg_session *s, int kernel_class, int layer, int repeat) {
	if (int rc = session_usable(s)) return rc;
	if (kernel_class < 0 || kernel_class > TG_KC_LMHEAD || repeat < 1 || layer < 0 || layer >= s->m->cfg.n_layers)
		return tg_fail(TG_ERR_BAD_ARG, "bad argument");
	StepOnly only{kernel_class, kernel_class == TG_KC_LMHEAD ? 0 : layer, repeat};
	return enqueue_decode_step(s, nullptr, false, &only);
}

int tg_plan_attention_prefill(int n_tokens, int n_cu, int window, int *query_tile, int32_t *items, int max_items, int *n_items,
                              int *n_split) {
	if (n_tokens < 1 || n_cu < 1 || !query_tile || !n_items || !n_split || (max_items > 0 && !items))
		return tg_fail(TG_ERR_BAD_ARG, "bad argument");
	const int tq = tg_attn_prefill_query_tile(n_tokens, n_cu);
	std::vector<int4> it, sp;
	int nslots = 0;
	const bool use = tg_attn_prefill_plan(n_tokens, n_cu, tq, window, it, sp, nslots);
	*query_tile = tq;
	*n_items = use ? (int)it.size() : 0;
	*n_split = use ? (int)sp.size() : 0;
	for (int i = 0; use && i < (int)it.size() && i < max_items; i++) {
		items[4 * i + 0] = it[(size_t)i].x;
		items[4 * i + 1] = it[(size_t)i].y;
		items[4 * i + 2] = it[(size_t)i].z;
		items[4 * i + 3] = it[(size_t)i].w;
	}
	return TG_OK;
}

int tg_plan_gemm_k_parts(int m, int in_dim, int out_dim, int n_cu) {
	if (m < 1 || n_cu < 1 || !legal_in(in_dim) || !legal_out(out_dim) || out_dim % TG_CT) return 1;
	return tg_gemm_mfma_k_parts(m, in_dim, out_dim / TG_CT, n_cu);
}

int tg_set_attn_merge_chunk(int keys) {
	if (keys < 32 || keys > 256 || keys % 16) return tg_fail(TG_ERR_BAD_ARG, "keys per workgroup: a multiple of 16 in 32..256");
	g_attn_merge_chunk = keys;
	g_knob_epoch++;
	return TG_OK;
}

int tg_set_attn_prefill_mode(int mode) {
	if (mode < 0 || mode > 3) return tg_fail(TG_ERR_BAD_ARG, "mode: 0, 1, 2 or 3");
	g_attn_prefill_split = mode;
	return TG_OK;
}

int tg_set_attn_prefill_format(int f16) {
	if (f16 < 0 || f16 > 2) return tg_fail(TG_ERR_BAD_ARG, "format: 0, 1 or 2");
	g_attn_prefill_f16 = f16;
	return TG_OK;
}

int tg_set_attn_prefill_planes(int mode) {
	if (mode < 0 || mode > 2) return tg_fail(TG_ERR_BAD_ARG, "mode: 0, 1 or 2");
	g_attn_prefill_planes = mode;
	return TG_OK;
}

int tg_set_gemm_split(int enable) {
	g_gemm_split = enable != 0;
	return TG_OK;
}

int tg_session_release_workspace(tg_session *s) {
	if (!s) return tg_fail(TG_ERR_BAD_ARG, "null session");
	TG_HIP(hipStreamSynchronize(g_stream));
	if (s->pf_ws) (void)hipFree(s->pf_ws);
	s->pf_ws = nullptr;
	s->pf_ws_bytes = 0;
	s->taps = nullptr;  // prefill taps live in the workspace
	s->tap_rows = 0;
	s->pf_plan.release();
	s->pf_plan_local.release();
	return TG_OK;
}

int tg_set_taps(int enable) {
	g_keep_taps = enable != 0;
	return TG_OK;
}

int tg_debug_gemm_launches(long long *few_rows, long long *one_per_tile, long long *two_per_unit) {
	if (!few_rows || !one_per_tile || !two_per_unit) return tg_fail(TG_ERR_BAD_ARG, "null pointer");
	*few_rows = g_gemm_launches[0];
	*one_per_tile = g_gemm_launches[1];
	*two_per_unit = g_gemm_launches[2];
	return TG_OK;
}

int tg_set_gemm_lds(int half_tiles_per_cu) {
	if (half_tiles_per_cu < 0 || half_tiles_per_cu > 127) return tg_fail(TG_ERR_BAD_ARG, "0 (off) or the threshold in half tiles per compute unit, up to 63 (+ 64: no half-K copies)");
	g_gemm_lds = half_tiles_per_cu & 63;
	g_gemm_lds_ksplit = (half_tiles_per_cu & 64) ? 0 : 1;  // + 64: without the half-K copies (measurement aid)
	return TG_OK;
}

int tg_set_gemm_mode(int mfma) {
	g_gemm_mfma = mfma != 0;
	return TG_OK;
}

int tg_set_prefetch_plan(int plan) {
	g_prefetch_plan = plan;
	g_knob_epoch++;
	return TG_OK;
}

int tg_set_prefetch_blocks(int n) {
	if (n < 0 || (n & 7)) return tg_fail(TG_ERR_BAD_ARG, "prefetch workgroups must be a non-negative multiple of 8");
	g_prefetch_blocks = n;
	g_knob_epoch++;
	return TG_OK;
}

int tg_set_gemv_max_blocks(int n) {
	g_gemv_max_blocks = n;
	g_knob_epoch++;
	return TG_OK;
}

// A profiler that traces kernels hooks every launch; replaying captured graphs under rocprofv3 --kernel-trace ended the
// process on this software stack (ROCm 7.2), so graph replay is refused while a profiler's tool library is loaded.
static bool profiler_attached() {
	const char *names[] = {"ROCP_TOOL_LIBRARIES", "ROCPROFILER_LIBRARY_CTOR", "ROCPROF_OUTPUT_PATH"};  // what rocprofv3 exports
	for (const char *n : names)
		if (getenv(n) != nullptr) return true;
	const char *pre = getenv("LD_PRELOAD");
	return pre != nullptr && strstr(pre, "rocprof") != nullptr;
}

int tg_set_chain_picks(int enable) {
	g_chain_picks = enable != 0;
	return TG_OK;
}

int tg_set_fused_decode(int enable, int gemv_workgroups, int max_spins) {
	if (gemv_workgroups < 0 || max_spins < 0 || max_spins > (1 << 22)) return tg_fail(TG_ERR_BAD_ARG, "bad argument (max_spins <= 2^22)");
	g_fused = enable != 0;
	g_fused_ng = gemv_workgroups;
	g_fused_spins = max_spins > 0 ? max_spins : 1 << 20;
	g_knob_epoch++;
	return TG_OK;
}

// One fused decode step of the session with timestamps: out[L][24] ticks of the 100 MHz counter (see TgFused::ts)
int tg_debug_fused_timestamps(tg_session *s, unsigned long long *out, int n_layers) {
	if (int rc = session_usable(s)) return rc;
	const int L = s->m->cfg.n_layers;
	if (!out || n_layers != L) return tg_fail(TG_ERR_BAD_ARG, "bad argument");
	unsigned long long *d = nullptr;
	TG_HIP(hipMalloc((void **)&d, sizeof(unsigned long long) * 24 * (size_t)L));
	TG_HIP(hipMemset(d, 0, sizeof(unsigned long long) * 24 * (size_t)L));
	g_fused_ts = d;
	int rc = tg_decode_enqueue(s, 1);
	g_fused_ts = nullptr;
	if (rc == TG_OK && hipStreamSynchronize(g_stream) != hipSuccess) rc = tg_fail(TG_ERR_HIP, "hipStreamSynchronize failed");
	if (rc == TG_OK) rc = fused_check(s);
	if (rc == TG_OK && hipMemcpy(out, d, sizeof(unsigned long long) * 24 * (size_t)L, hipMemcpyDeviceToHost) != hipSuccess) rc = tg_fail(TG_ERR_HIP, "hipMemcpy failed");
	(void)hipFree(d);
	return rc;
}

int tg_reset_knobs() {
	g_fused = 0;
	g_fused_ng = 0;
	g_fused_spins = 1 << 20;
	g_gemm_mfma = 1;
	g_prefetch_plan = 0;
	g_prefetch_blocks = 128;
	g_gemv_max_blocks = 2048;
	g_use_graphs = -1;
	g_gemm_split = true;
	g_gemm_lds = 2;
	g_gemm_lds_ksplit = 1;
	g_attn_merge_chunk = 64;
	g_attn_prefill_split = 1;
	g_attn_prefill_planes = 1;
	g_attn_prefill_f16 = 1;
	g_chain_picks = true;
	g_keep_taps = false;
	g_knob_epoch++;
	return TG_OK;
}

int tg_set_graphs(int enable) {
	if (enable > 0 && profiler_attached())
		return tg_fail(TG_ERR_STATE, "graph replay is not available under a profiler (a kernel trace of replayed graphs ended the process); use plain launches");
	if (enable < -1 || enable > 2) return tg_fail(TG_ERR_BAD_ARG, "mode: -1, 0, 1 or 2");
	g_use_graphs = enable;
	g_knob_epoch++;  // graphs of the other mode are dropped
	return TG_OK;
}

int tg_decode_profile(tg_session *s, int n_steps, double *ms_sum, int *launches) {
	if (!s || n_steps < 1 || !ms_sum || !launches) return tg_fail(TG_ERR_BAD_ARG, "bad argument");
	for (int k = 0; k < TG_KC_COUNT; k++) {
		ms_sum[k] = 0.0;
		launches[k] = 0;
	}
	StepProfile prof;
	int rc = TG_OK;
	for (int i = 0; i < n_steps && rc == TG_OK; i++) {
		prof.used = 0;
		rc = enqueue_decode_step(s, &prof, false);
		if (rc != TG_OK) break;
		if (hipStreamSynchronize(g_stream) != hipSuccess) {
			rc = tg_fail(TG_ERR_HIP, "hipStreamSynchronize failed");
			break;
		}
		for (size_t e = 0; e + 1 < prof.used; e++) {
			float ms = 0.0f;
			if (hipEventElapsedTime(&ms, prof.ev[e], prof.ev[e + 1]) != hipSuccess) {
				rc = tg_fail(TG_ERR_HIP, "hipEventElapsedTime failed");
				break;
			}
			ms_sum[prof.cls[e]] += (double)ms;
			launches[prof.cls[e]] += 1;
		}
	}
	for (hipEvent_t e : prof.ev) (void)hipEventDestroy(e);
	return rc;
}

int tg_session_read_ids(tg_session *s, int32_t *ids, int max_ids, int *n_out) {
	if (!s || !ids) return tg_fail(TG_ERR_BAD_ARG, "null argument");
	TG_HIP(hipStreamSynchronize(g_stream));
	if (int rc = fused_check(s)) return rc;
	const int n = std::min(max_ids, s->steps);
	if (n > 0) TG_HIP(hipMemcpy(ids, s->tok_log, sizeof(int) * (size_t)n, hipMemcpyDeviceToHost));
	if (n_out) *n_out = n;
	return TG_OK;
}

// ---------------------------------------------------------------------------------------------
// forward_prefill
// ---------------------------------------------------------------------------------------------
int tg_attention_prefill(float *o, const float *q, const float *k, const float *v, int S, int is_sw, int sw_context) {
	if (int rc = ensure_init()) return rc;
	if (!o || !q || !k || !v || S < 1 || sw_context < 1) return tg_fail(TG_ERR_BAD_ARG, "bad argument");
	constexpr int NH = 4, HD = 256;
	const size_t rows = (size_t)S;
	std::vector<float> qr(rows * NH * HD), orow(rows * NH * HD);
	for (int hh = 0; hh < NH; hh++)
		for (size_t t = 0; t < rows; t++) memcpy(&qr[(t * NH + hh) * HD], &q[((size_t)hh * rows + t) * HD], sizeof(float) * HD);
	float *dq = nullptr, *dk = nullptr, *dv = nullptr, *dout = nullptr;
	void *dplanes = nullptr;
	AttnPlanDev plan;
	auto done = [&](int rc) {
		(void)hipStreamSynchronize(g_stream);
		void *ps[] = {dq, dk, dv, dout, dplanes};
		for (void *p : ps)
			if (p) (void)hipFree(p);
		plan.release();
		return rc;
	};
	int rc = tg_dev_alloc((void **)&dq, sizeof(float) * rows * NH * HD);
	if (rc == TG_OK) rc = tg_dev_alloc((void **)&dout, sizeof(float) * rows * NH * HD);
	if (rc == TG_OK) rc = tg_dev_alloc((void **)&dk, sizeof(float) * rows * HD);
	if (rc == TG_OK) rc = tg_dev_alloc((void **)&dv, sizeof(float) * rows * HD);
	if (rc == TG_OK) rc = tg_dev_alloc(&dplanes, tg_attn_prefill_planes_bytes(S) + 256);  // + the range flag
	if (rc == TG_OK) rc = tg_copy_h2d(dq, qr.data(), sizeof(float) * rows * NH * HD);
	if (rc == TG_OK) rc = tg_copy_h2d(dk, k, sizeof(float) * rows * HD);
	if (rc == TG_OK) rc = tg_copy_h2d(dv, v, sizeof(float) * rows * HD);
	if (rc == TG_OK) rc = plan.build(S, (is_sw && S > sw_context + 1) ? sw_context : -1);
	if (rc != TG_OK) return done(rc);
	int *dflag = (int *)((unsigned char *)dplanes + tg_attn_prefill_planes_bytes(S));
	if (hipMemsetAsync(dflag, 0, sizeof(int), g_stream) != hipSuccess) return done(tg_fail(TG_ERR_HIP, "hipMemsetAsync failed"));
	tg_launch_attn_prefill(dout, dq, dk, dv, S, NH, HD, NH * HD, HD, NH * HD, is_sw ? 1 : 0, sw_context, plan.get(), g_n_cu, g_stream, false,
	                       dplanes, dflag);
	if (hipGetLastError() != hipSuccess) return done(tg_fail(TG_ERR_HIP, "attention launch failed"));
	rc = tg_copy_d2h(orow.data(), dout, sizeof(float) * rows * NH * HD);
	int hflag = 0;
	if (rc == TG_OK) rc = tg_copy_d2h(&hflag, dflag, sizeof(int));
	if (rc == TG_OK && hflag) rc = attn_range_error();
	if (rc != TG_OK) return done(rc);
	for (int hh = 0; hh < NH; hh++)
		for (size_t t = 0; t < rows; t++) memcpy(&o[((size_t)hh * rows + t) * HD], &orow[(t * NH + hh) * HD], sizeof(float) * HD);
	return done(TG_OK);
}

// ---- forward_prefill in pieces: workspace, the launches of one attention block and of one MLP block ----
namespace {
// PrefillState (decode.hpp:281-351): carved out of one arena the session keeps (hipMalloc/hipFree of a few hundred
// MB per call cost milliseconds), 256-byte aligned pieces, plus the attention work lists of this prompt length.
struct PrefillCtx {
	tg_session *s = nullptr;
	int n = 0;
	bool pk = false;         // int8 matrix path: producers write digit planes (apack + rowscale) instead of fp32 rows
	int tap_rows = 0;        // rows of the residual stream kept per block (0: none; n; or 1 = the last row of a long prompt)
	int *d_ids = nullptr;
	float *x = nullptr, *xn = nullptr, *qkv = nullptr, *ao = nullptr, *t = nullptr, *hb = nullptr, *rowscale = nullptr, *amax = nullptr;
	int8_t *apack = nullptr;
	void *planes = nullptr;  // pre-split K/V plane images of the layer being processed (split-precision attention)
	const TgAttnPrefillPlan *plan_global = nullptr, *plan_local = nullptr;
	int o_parts = 1, d_parts = 1;
	size_t tpart = 0;
};

int prefill_setup(tg_session *s, int n, PrefillCtx *ctx, bool with_taps) {
	tg_model *m = s->m;
	const tg_config &c = m->cfg;
	const int L = c.n_layers, h = c.hidden_size, f = c.intermediate_size, hd = c.head_dim;
	const int qo = c.n_head * hd, nq = qo + 2 * hd;
	const size_t S = (size_t)n;
	// taps: every row of a short prompt, the last row of a long one
	const int tap_rows = !(g_keep_taps && with_taps) ? 0 : (n <= PREFILL_TAP_MAX_ROWS ? n : 1);
	size_t need = 0;
	auto carve = [&](size_t bytes) {
		const size_t off = need;
		need += (bytes + 255) & ~(size_t)255;
		return off;
	};
	const size_t o_ids = carve(sizeof(int) * S), o_x = carve(sizeof(float) * S * h), o_xn = carve(sizeof(float) * S * h),
	             o_qkv = carve(sizeof(float) * S * nq), o_ao = carve(sizeof(float) * S * qo), o_t = carve(sizeof(float) * 4 * S * h),  // up to 4 partial results
	             o_hb = carve(sizeof(float) * S * f),
	             o_apack = carve(g_gemm_mfma ? tg_gemm_mfma_apack_bytes(n, std::max(std::max(f, qo), h)) : 0),
	             o_rs = carve(g_gemm_mfma ? sizeof(float) * 2 * tg_gemm_mfma_rows(n) : 0),
	             o_amax = carve(g_gemm_mfma ? sizeof(float) * tg_gemm_mfma_rows(n) : 0),
	             o_taps = carve(sizeof(float) * (size_t)(2 * L + 1) * (size_t)tap_rows * h),
	             o_planes = carve(tg_attn_prefill_planes_bytes(n));
	if (need > s->pf_ws_bytes) {
		TG_HIP(hipStreamSynchronize(g_stream));
		s->taps = nullptr;  // they live in the workspace
		s->tap_rows = 0;
		if (s->pf_ws) (void)hipFree(s->pf_ws);
		s->pf_ws = nullptr;
		s->pf_ws_bytes = 0;
		TG_HIP(hipMalloc(&s->pf_ws, need));
		s->pf_ws_bytes = need;
	}
	uint8_t *ws = (uint8_t *)s->pf_ws;
	ctx->s = s;
	ctx->n = n;
	ctx->pk = g_gemm_mfma != 0;
	ctx->tap_rows = tap_rows;
	ctx->d_ids = (int *)(ws + o_ids);
	ctx->x = (float *)(ws + o_x);
	ctx->xn = (float *)(ws + o_xn);
	ctx->qkv = (float *)(ws + o_qkv);
	ctx->ao = (float *)(ws + o_ao);
	ctx->t = (float *)(ws + o_t);
	ctx->hb = (float *)(ws + o_hb);
	ctx->rowscale = (float *)(ws + o_rs);
	ctx->apack = (int8_t *)(ws + o_apack);
	ctx->planes = ws + o_planes;
	ctx->amax = g_gemm_mfma ? (float *)(ws + o_amax) : nullptr;  // max|hb| per row, folded by the up|gate product
	s->taps = tap_rows ? (float *)(ws + o_taps) : nullptr;
	s->tap_rows = tap_rows;
	// Work lists of the attention launches.  A local layer whose window covers the whole prompt is a causal layer.
	const bool local_is_causal = n <= c.n_pos_local + 1;
	if (int rc = s->pf_plan.build(n, -1)) return rc;
	if (!local_is_causal) {
		if (int rc = s->pf_plan_local.build(n, c.n_pos_local)) return rc;
	}
	ctx->plan_global = s->pf_plan.get();
	ctx->plan_local = local_is_causal ? ctx->plan_global : s->pf_plan_local.get();
	// products that would otherwise leave most compute units idle (a badly filled last round of workgroups; a short
	// prompt's long-K products) run in 2 or 4 parts of K with separate partial results; the norm that consumes them adds
	// the parts
	ctx->tpart = S * h;
	ctx->o_parts = (ctx->pk && g_gemm_split) ? tg_gemm_mfma_k_parts(n, qo, m->L[0].o.ntiles_g, g_n_cu) : 1;
	ctx->d_parts = (ctx->pk && g_gemm_split) ? tg_gemm_mfma_k_parts(n, f, m->L[0].d.ntiles_g, g_n_cu) : 1;
	return TG_OK;
}

hipError_t prefill_tap(const PrefillCtx &p, int b) {
	if (!p.tap_rows) return hipSuccess;
	const size_t h = (size_t)p.s->m->cfg.hidden_size, rows = (size_t)p.tap_rows;
	return hipMemcpyAsync(p.s->taps + (size_t)b * rows * h, p.x + ((size_t)p.n - rows) * h, sizeof(float) * rows * h, hipMemcpyDeviceToDevice,
	                      g_stream);
}

// xn (or its digit planes) = rmsnorm(x, w_pre): the first norm of a forward, or of a block run on its own
void prefill_first_norm(const PrefillCtx &p, const float *w_pre, bool clear_amax) {
	const int h = p.s->m->cfg.hidden_size;
	tg_launch_norm_rows(p.pk ? nullptr : p.xn, p.x, 1, 0, w_pre, nullptr, nullptr, nullptr, p.n, h, p.pk ? p.apack : nullptr, p.rowscale, g_stream,
	                    clear_amax ? p.amax : nullptr);
}

// modules::attention, prefill branch (modules.hpp:98-133), from the pre-normalised rows to the output projection's
// partial results in p.t; the post-norm + residual is the norm launch that follows
void prefill_attention_launches(const PrefillCtx &p, int l) {
	tg_session *s = p.s;
	tg_model *m = s->m;
	const tg_config &c = m->cfg;
	const int h = c.hidden_size, hd = c.head_dim, qo = c.n_head * hd, nq = qo + 2 * hd, n = p.n;
	const LayerDev &Ld = m->L[(size_t)l];
	const int mp = s->max_pos[(size_t)l];
	// Q|K|V (modules.hpp:106-108)
	launch_gemm(p.qkv, p.xn, h, Ld.qkv, n, TG_EPI_STORE, nullptr, 0, 0, 0, p.apack, p.rowscale, p.pk);
	// q/k norm + RoPE from position 0, KV write (modules.hpp:115-121)
	tg_launch_qk_norm_rope_rows(p.qkv, p.qkv + qo, p.qkv + qo + hd, Ld.rms_q, Ld.rms_k, Ld.is_sw ? s->cos_l : s->cos_g,
	                            Ld.is_sw ? s->sin_l : s->sin_g, s->kc[(size_t)l], s->vc[(size_t)l], mp, n, c.n_head, hd, nq, nq, g_stream);
	// attention (modules.hpp:123): local layers use sw_context = max_pos
	const TgAttnPrefillPlan *lplan = Ld.is_sw ? p.plan_local : p.plan_global;
	tg_launch_attn_prefill(p.ao, p.qkv, p.qkv + qo, p.qkv + qo + hd, n, c.n_head, hd, nq, nq, qo, Ld.is_sw ? 1 : 0, mp, lplan, g_n_cu, g_stream,
	                       p.pk, p.planes, s->ctr + 5);
	// with the int8 MFMA GEMM one launch merges split query tiles and writes the output projection's digit planes
	if (p.pk) tg_launch_attn_prefill_finish(p.ao, n, qo, lplan, g_n_cu, p.apack, p.rowscale, g_stream);
	// O (modules.hpp:127-128)
	launch_gemm(p.t, p.ao, qo, Ld.o, n, TG_EPI_STORE, nullptr, 0, 0, 0, p.apack, p.rowscale, p.pk, nullptr, nullptr, p.o_parts, p.tpart);
}

// modules::mlp, prefill branch (modules.hpp:179-201), from the pre-normalised rows to the down projection's partial
// results in p.t.  The norm launch before it must have cleared p.amax.
void prefill_mlp_launches(const PrefillCtx &p, int l) {
	tg_session *s = p.s;
	const tg_config &c = s->m->cfg;
	const LayerDev &Ld = s->m->L[(size_t)l];
	const int h = c.hidden_size, f = c.intermediate_size, n = p.n;
	// up|gate + gelu*up (modules.hpp:190-195), down (modules.hpp:196-197)
	launch_gemm(p.hb, p.xn, h, Ld.ug, n, TG_EPI_GEGLU, s->lut, s->gmin, s->geps, s->lut_size, p.apack, p.rowscale, p.pk, nullptr, p.amax);
	launch_gemm(p.t, p.hb, f, Ld.d, n, TG_EPI_STORE, nullptr, 0, 0, 0, p.apack, p.rowscale, false, p.amax, nullptr, p.d_parts, p.tpart);
}

// x = rmsnorm(t, w_post) + x, then xn (or its digit planes) = rmsnorm(x, next_pre)  (modules.hpp:130-132, 188, 199-201)
void prefill_block_end(const PrefillCtx &p, int nparts, const float *w_post, const float *next_pre, bool want_fp32, bool clear_amax) {
	const int h = p.s->m->cfg.hidden_size;
	const bool planes = p.pk && !want_fp32;
	tg_launch_norm_rows(planes ? nullptr : p.xn, p.t, nparts, p.tpart, next_pre, w_post, p.x, p.x, p.n, h, planes ? p.apack : nullptr, p.rowscale,
	                    g_stream, clear_amax ? p.amax : nullptr);
}

// KVCache::update_prefill's counters (decode.hpp:99-104) after n tokens
int set_counters_after_prefill(tg_session *s, int n) {
	const tg_config &c = s->m->cfg;
	s->pos = n;
	s->bp_local = (n >= c.n_pos_local) ? c.n_pos_local : n;
	s->bp_global = (n >= c.n_pos) ? c.n_pos : n;
	int ctr[3] = {s->pos, s->bp_local, s->bp_global};
	TG_HIP(hipMemcpyAsync(s->ctr, ctr, sizeof(ctr), hipMemcpyHostToDevice, g_stream));
	TG_HIP(hipStreamSynchronize(g_stream));  // ctr[] is on this function's stack
	return TG_OK;
}
}  // namespace

int tg_forward_prefill(tg_session *s, const int32_t *ids, int n, float *logits, int32_t *argmax) {
	if (!s || !ids) return tg_fail(TG_ERR_BAD_ARG, "null argument");
	if (int rc = session_usable(s)) return rc;
	tg_model *m = s->m;
	const tg_config &c = m->cfg;
	if (n < 1) return tg_fail(TG_ERR_BAD_ARG, "empty prompt");
	if (s->pos != 0) return tg_fail(TG_ERR_STATE, "prefill needs an empty session (decode.hpp:78-79)");
	if (n > c.n_pos) return tg_fail(TG_ERR_STATE, "prompt longer than n_pos");
	const int L = c.n_layers, h = c.hidden_size;
	const size_t S = (size_t)n;
	PrefillCtx p;
	if (int rc = prefill_setup(s, n, &p, true)) return rc;
	TG_HIP(hipMemcpyAsync(p.d_ids, ids, sizeof(int) * S, hipMemcpyHostToDevice, g_stream));
	tg_launch_embed_rows(p.x, p.d_ids, n, m->wte, m->wte_scales, h, c.n_vocab, g_stream);
	TG_HIP(prefill_tap(p, 0));
	// With the int8 MFMA GEMM a norm writes the next GEMM's digit planes itself and the fp32 row is not stored.
	prefill_first_norm(p, m->L[0].apre, false);
	for (int l = 0; l < L; l++) {
		const LayerDev &Ld = m->L[(size_t)l];
		prefill_attention_launches(p, l);
		prefill_block_end(p, p.o_parts, Ld.apost, Ld.mpre, false, true);  // also clears the row maxima the up|gate product folds into
		TG_HIP(prefill_tap(p, 2 * l + 1));
		prefill_mlp_launches(p, l);
		// the last layer's final norm feeds the LM head GEMV, which reads the fp32 row
		const bool last = l + 1 == L;
		prefill_block_end(p, p.d_parts, Ld.mpost, last ? m->rmsw : m->L[(size_t)l + 1].apre, last, false);
		TG_HIP(prefill_tap(p, 2 * l + 2));
	}
	// LM head on the last position only (modules.hpp:232-240): xn already holds rmsnorm(x, RMSw)
	{
		TgGemv g = gemv_base(m->lm);
		g.x = p.xn + (S - 1) * h;
		g.y = s->logits;
		g.blk_val = s->blk_val;
		g.blk_idx = s->blk_idx;
		tg_launch_gemv(g, TG_ROLE_LMHEAD_PLAIN, g_stream);
		tg_launch_argmax_finish(s->blk_val, s->blk_idx, m->lm.ntiles, s->ctr, s->tok_log, 0, g_stream);
	}
	TG_HIP(hipGetLastError());
	s->steps = 1;
	if (int rc = set_counters_after_prefill(s, n)) return rc;
	if (logits) TG_HIP(hipMemcpyAsync(logits, s->logits, sizeof(float) * (size_t)c.n_vocab, hipMemcpyDeviceToHost, g_stream));
	int32_t tok_flag[2] = {-1, 0};
	TG_HIP(hipMemcpyAsync(tok_flag, s->ctr + 4, 2 * sizeof(int), hipMemcpyDeviceToHost, g_stream));
	TG_HIP(hipStreamSynchronize(g_stream));
	if (argmax) *argmax = tok_flag[0];
	if (tok_flag[1]) return attn_range_error();
	return TG_OK;
}

// ---------------------------------------------------------------------------------------------
// block level (parity checks of one modules::attention / mlp / lm_head call at a time)
// ---------------------------------------------------------------------------------------------
static int block_args_ok(tg_session *s, int layer, const float *x, int rows) {
	if (int rc = session_usable(s)) return rc;
	const tg_config &c = s->m->cfg;
	if (!x || rows < 1 || layer < 0 || layer >= c.n_layers) return tg_fail(TG_ERR_BAD_ARG, "bad argument");
	if (rows > c.n_pos) return tg_fail(TG_ERR_STATE, "more rows than n_pos");
	return TG_OK;
}

int tg_session_kv_prefill(tg_session *s, int layer, const float *keys, const float *values, int rows) {
	if (int rc = block_args_ok(s, layer, keys, rows)) return rc;
	if (!values) return tg_fail(TG_ERR_BAD_ARG, "null argument");
	if (s->pos != 0 && s->pos != rows) return tg_fail(TG_ERR_STATE, "the session's position counter is shared by all layers: reset it, or give every layer the same number of rows");
	const int hd = s->m->cfg.head_dim, mp = s->max_pos[(size_t)layer];
	const int start = rows >= mp ? rows - mp : 0;  // decode.hpp:84-86: the tail of a context longer than the cache
	const size_t bytes = sizeof(float) * (size_t)(rows - start) * hd;
	TG_HIP(hipMemcpyAsync(s->kc[(size_t)layer], keys + (size_t)start * hd, bytes, hipMemcpyHostToDevice, g_stream));
	TG_HIP(hipMemcpyAsync(s->vc[(size_t)layer], values + (size_t)start * hd, bytes, hipMemcpyHostToDevice, g_stream));
	return set_counters_after_prefill(s, rows);
}

int tg_block_attention(tg_session *s, int layer, float *x, int rows) {
	if (int rc = block_args_ok(s, layer, x, rows)) return rc;
	tg_model *m = s->m;
	const int h = m->cfg.hidden_size;
	const LayerDev &Ld = m->L[(size_t)layer];
	if (rows == 1) {
		// decode branch (modules.hpp:135-169) with the kernels of a decode step; the launch that follows the output
		// projection in a step (up|gate) forms post-norm + residual, its own product is not used
		if (s->pos >= m->cfg.n_pos) return tg_fail(TG_ERR_STATE, "context is full (n_pos)");
		TG_HIP(hipMemcpyAsync(s->blk_x, x, sizeof(float) * (size_t)h, hipMemcpyHostToDevice, g_stream));
		launch_qkv(s, layer, false, s->zeros, Ld.apost, s->blk_x, nullptr);
		const AttnGeom ag = attn_geometry(s, layer, false);
		launch_attn(s, ag);
		launch_oproj(s, layer, ag);
		launch_upgate(s, layer, s->o_out, s->blk_x, s->blk_y);
		TG_HIP(hipGetLastError());
		TG_HIP(hipMemcpyAsync(x, s->blk_y, sizeof(float) * (size_t)h, hipMemcpyDeviceToHost, g_stream));
		// KVCache::update_single advanced this layer's counters (decode.hpp:68-69); the session has one set for all layers
		s->pos += 1;
		s->bp_local += 1;
		s->bp_global += 1;
		int ctr[3] = {s->pos, s->bp_local, s->bp_global};
		TG_HIP(hipMemcpyAsync(s->ctr, ctr, sizeof(ctr), hipMemcpyHostToDevice, g_stream));
		TG_HIP(hipStreamSynchronize(g_stream));
		s->taps = nullptr;
		s->tap_rows = 0;
		return TG_OK;
	}
	if (s->pos != 0) return tg_fail(TG_ERR_STATE, "prefill needs an empty session (decode.hpp:78-79)");
	PrefillCtx p;
	if (int rc = prefill_setup(s, rows, &p, false)) return rc;
	const size_t bytes = sizeof(float) * (size_t)rows * h;
	TG_HIP(hipMemcpyAsync(p.x, x, bytes, hipMemcpyHostToDevice, g_stream));
	prefill_first_norm(p, Ld.apre, false);
	prefill_attention_launches(p, layer);
	prefill_block_end(p, p.o_parts, Ld.apost, Ld.mpre, false, false);
	TG_HIP(hipGetLastError());
	TG_HIP(hipMemcpyAsync(x, p.x, bytes, hipMemcpyDeviceToHost, g_stream));
	int flag = 0;
	TG_HIP(hipMemcpyAsync(&flag, s->ctr + 5, sizeof(int), hipMemcpyDeviceToHost, g_stream));
	if (int rc = set_counters_after_prefill(s, rows)) return rc;  // synchronises
	return flag ? attn_range_error() : TG_OK;
}

int tg_block_mlp(tg_session *s, int layer, float *x, int rows) {
	if (int rc = block_args_ok(s, layer, x, rows)) return rc;
	tg_model *m = s->m;
	const int h = m->cfg.hidden_size;
	const LayerDev &Ld = m->L[(size_t)layer];
	if (rows == 1) {
		// decode branch (modules.hpp:203-220): the launch that follows the down projection in a step (the next Q|K|V)
		// forms post-norm + residual
		TG_HIP(hipMemcpyAsync(s->blk_x, x, sizeof(float) * (size_t)h, hipMemcpyHostToDevice, g_stream));
		launch_upgate(s, layer, s->zeros, s->blk_x, nullptr);
		launch_down(s, layer);
		launch_qkv(s, layer, false, s->d_out, Ld.mpost, s->blk_x, s->blk_y);
		TG_HIP(hipGetLastError());
		TG_HIP(hipMemcpyAsync(x, s->blk_y, sizeof(float) * (size_t)h, hipMemcpyDeviceToHost, g_stream));
		TG_HIP(hipStreamSynchronize(g_stream));
		return TG_OK;
	}
	PrefillCtx p;
	if (int rc = prefill_setup(s, rows, &p, false)) return rc;
	const size_t bytes = sizeof(float) * (size_t)rows * h;
	TG_HIP(hipMemcpyAsync(p.x, x, bytes, hipMemcpyHostToDevice, g_stream));
	prefill_first_norm(p, Ld.mpre, true);
	prefill_mlp_launches(p, layer);
	prefill_block_end(p, p.d_parts, Ld.mpost, m->rmsw, true, false);
	TG_HIP(hipGetLastError());
	TG_HIP(hipMemcpyAsync(x, p.x, bytes, hipMemcpyDeviceToHost, g_stream));
	TG_HIP(hipStreamSynchronize(g_stream));
	return TG_OK;
}

int tg_block_lm_head(tg_session *s, const float *x, int rows, float *logits) {
	if (int rc = block_args_ok(s, 0, x, rows)) return rc;
	if (!logits) return tg_fail(TG_ERR_BAD_ARG, "null argument");
	tg_model *m = s->m;
	const int h = m->cfg.hidden_size;
	// both branches take the last row (modules.hpp:232-246)
	TG_HIP(hipMemcpyAsync(s->blk_x, x + (size_t)(rows - 1) * h, sizeof(float) * (size_t)h, hipMemcpyHostToDevice, g_stream));
	if (rows == 1) {
		launch_lmhead(s, s->zeros, m->rmsw, s->blk_x, nullptr);  // the decode step's kernel: final norm in its prologue
	} else {
		// the prefill's sequence: a row norm, then the LM head on the normalised row
		tg_launch_norm_rows(s->blk_y, s->blk_x, 1, 0, m->rmsw, nullptr, nullptr, nullptr, 1, h, nullptr, nullptr, g_stream);
		TgGemv g = gemv_base(m->lm);
		g.x = s->blk_y;
		g.y = s->logits;
		g.blk_val = s->blk_val;
		g.blk_idx = s->blk_idx;
		tg_launch_gemv(g, TG_ROLE_LMHEAD_PLAIN, g_stream);
	}
	TG_HIP(hipGetLastError());
	TG_HIP(hipMemcpyAsync(logits, s->logits, sizeof(float) * (size_t)m->cfg.n_vocab, hipMemcpyDeviceToHost, g_stream));
	TG_HIP(hipStreamSynchronize(g_stream));
	return TG_OK;
}


int tg_generate_greedy(tg_session *s, const int32_t *prompt, int n_prompt, int n_decode, int32_t *out_ids, double *s_prefill,
                       double *s_decode) {
	if (!s || !prompt || !out_ids || n_decode < 0) return tg_fail(TG_ERR_BAD_ARG, "bad argument");
	using clk = std::chrono::steady_clock;
	auto t0 = clk::now();
	int32_t tok = -1;
	if (int rc = tg_forward_prefill(s, prompt, n_prompt, nullptr, &tok)) return rc;
	auto t1 = clk::now();
	if (int rc = tg_decode_enqueue(s, n_decode)) return rc;
	int got = 0;
	if (int rc = tg_session_read_ids(s, out_ids, n_decode + 1, &got)) return rc;
	auto t2 = clk::now();
	if (s_prefill) *s_prefill = std::chrono::duration<double>(t1 - t0).count();
	if (s_decode) *s_decode = std::chrono::duration<double>(t2 - t1).count();
	return got == n_decode + 1 ? TG_OK : tg_fail(TG_ERR_STATE, "token log incomplete");
}

namespace {
// scratch of the sampler + room for n draws, uploaded from the host
int sampler_prepare(tg_session *s, const float *randf, int n) {
	const tg_config &c = s->m->cfg;
	if (c.n_vocab % 1024 != 0) return tg_fail(TG_ERR_UNSUPPORTED_SHAPE, "sampler needs a vocabulary that is a multiple of 1024");
	if (!s->probs) {
		TG_HIP(hipMalloc((void **)&s->probs, sizeof(float) * (size_t)c.n_vocab));
		TG_HIP(hipMalloc((void **)&s->seg, sizeof(float) * tg_minp_segments(c.n_vocab)));
		TG_HIP(hipMalloc((void **)&s->bsum, sizeof(float) * tg_minp_blocks(c.n_vocab)));
		TG_HIP(hipMalloc((void **)&s->bmax, sizeof(float) * tg_minp_blocks(c.n_vocab)));
	}
	if (n > s->randf_cap) {
		TG_HIP(hipStreamSynchronize(g_stream));
		if (s->randf) (void)hipFree(s->randf);
		s->randf = nullptr;
		s->randf_cap = 0;
		TG_HIP(hipMalloc((void **)&s->randf, sizeof(float) * (size_t)n));
		s->randf_cap = n;
	}
	// the previous batch of draws may still be in use by launches in flight
	TG_HIP(hipStreamSynchronize(g_stream));
	TG_HIP(hipMemcpy(s->randf, randf, sizeof(float) * (size_t)n, hipMemcpyHostToDevice));
	return TG_OK;
}
bool sampler_args_ok(float minp, float temp) { return temp > 0.0f && minp >= 0.0f; }
}  // namespace

int tg_minp_logits(const float *logits, int n_vocab, float minp, float temp, float randf, int32_t *token_out) {
	if (int rc = ensure_init()) return rc;
	if (!logits || !token_out || !sampler_args_ok(minp, temp)) return tg_fail(TG_ERR_BAD_ARG, "bad argument");
	if (n_vocab < 1024 || n_vocab % 1024 != 0)
		return tg_fail(TG_ERR_UNSUPPORTED_SHAPE, "Unsupported vocabulary size: " + std::to_string(n_vocab));
	const size_t nb = tg_minp_blocks(n_vocab), ns = tg_minp_segments(n_vocab);
	float *buf = nullptr;  // logits | probs | seg | bsum | bmax | randf | token
	const size_t floats = 2 * (size_t)n_vocab + ns + 2 * nb + 2;
	TG_HIP(hipMalloc((void **)&buf, sizeof(float) * floats));
	float *d_logits = buf, *d_probs = buf + n_vocab, *d_seg = d_probs + n_vocab, *d_bsum = d_seg + ns, *d_bmax = d_bsum + nb,
	      *d_rand = d_bmax + nb;
	int *d_tok = reinterpret_cast<int *>(d_rand + 1);
	int rc = TG_OK;
	if (hipMemcpy(d_logits, logits, sizeof(float) * (size_t)n_vocab, hipMemcpyHostToDevice) != hipSuccess ||
	    hipMemcpy(d_rand, &randf, sizeof(float), hipMemcpyHostToDevice) != hipSuccess)
		rc = tg_fail(TG_ERR_HIP, "upload failed");
	if (rc == TG_OK) {
		tg_launch_minp(d_logits, n_vocab, minp, temp, d_rand, 0, 0, d_probs, d_seg, d_bsum, d_bmax, nullptr, nullptr, 2, d_tok, g_stream);
		if (hipStreamSynchronize(g_stream) != hipSuccess || hipMemcpy(token_out, d_tok, sizeof(int), hipMemcpyDeviceToHost) != hipSuccess)
			rc = tg_fail(TG_ERR_HIP, "sampler launch failed");
	}
	(void)hipFree(buf);
	return rc;
}

int tg_decode_enqueue_sampled(tg_session *s, int n_steps, float minp, float temp, const float *randf) {
	if (!s || n_steps < 0) return tg_fail(TG_ERR_BAD_ARG, "bad argument");
	if (!(minp < 1.0f)) return tg_decode_enqueue(s, n_steps);  // transformer.hpp:232: minp >= 1 selects the argmax branch
	if (!randf || !sampler_args_ok(minp, temp)) return tg_fail(TG_ERR_BAD_ARG, "bad argument");
	if (n_steps == 0) return TG_OK;
	if (int rc = sampler_prepare(s, randf, n_steps)) return rc;
	s->sampling = true;
	s->s_minp = minp;
	s->s_temp = temp;
	s->rand_base = s->steps;
	int rc = TG_OK;
	for (int i = 0; i < n_steps && rc == TG_OK; i++) rc = enqueue_decode_step(s, nullptr, false);
	s->sampling = false;
	if (rc == TG_OK && s->taps) {
		TG_HIP(hipStreamSynchronize(g_stream));
		s->taps = nullptr;
		s->tap_rows = 0;
	}
	return rc;
}

int tg_generate(tg_session *s, const int32_t *prompt, int n_prompt, int n_decode, float minp, float temp, const float *randf,
                int32_t *out_ids, double *s_prefill, double *s_decode) {
	if (!(minp < 1.0f)) return tg_generate_greedy(s, prompt, n_prompt, n_decode, out_ids, s_prefill, s_decode);
	if (!s || !prompt || !out_ids || !randf || n_decode < 0 || !sampler_args_ok(minp, temp)) return tg_fail(TG_ERR_BAD_ARG, "bad argument");
	using clk = std::chrono::steady_clock;
	auto t0 = clk::now();
	int32_t tok = -1;
	if (int rc = tg_forward_prefill(s, prompt, n_prompt, nullptr, &tok)) return rc;
	// the prefill logits are still on the device: draw the first token from them (transformer.hpp:208-211)
	if (int rc = sampler_prepare(s, randf, 1)) return rc;
	tg_launch_minp(s->logits, s->m->cfg.n_vocab, minp, temp, s->randf, 0, 0, s->probs, s->seg, s->bsum, s->bmax, s->ctr, s->tok_log, 1,
	               nullptr, g_stream);
	TG_HIP(hipStreamSynchronize(g_stream));
	auto t1 = clk::now();
	if (int rc = tg_decode_enqueue_sampled(s, n_decode, minp, temp, randf + 1)) return rc;
	int got = 0;
	if (int rc = tg_session_read_ids(s, out_ids, n_decode + 1, &got)) return rc;
	auto t2 = clk::now();
	if (s_prefill) *s_prefill = std::chrono::duration<double>(t1 - t0).count();
	if (s_decode) *s_decode = std::chrono::duration<double>(t2 - t1).count();
	return got == n_decode + 1 ? TG_OK : tg_fail(TG_ERR_STATE, "token log incomplete");
}


// ---------------------------------------------------------------------------------------------
// debug taps
// ---------------------------------------------------------------------------------------------
int tg_session_tap(tg_session *s, int b, float *out, int rows) {
	if (!s || !out) return tg_fail(TG_ERR_BAD_ARG, "null argument");
	const tg_config &c = s->m->cfg;
	if (b < 0 || b > 2 * c.n_layers) return tg_fail(TG_ERR_BAD_ARG, "no such block");
	TG_HIP(hipStreamSynchronize(g_stream));
	if (int rc = fused_check(s)) return rc;
	const size_t h = (size_t)c.hidden_size;
	if (s->taps) {
		if (rows != s->tap_rows)
			return tg_fail(TG_ERR_BAD_ARG, "rows must equal the prompt length (1 for a prompt of more than 1024 tokens: only its last row is kept)");
		TG_HIP(hipMemcpy(out, s->taps + (size_t)b * s->tap_rows * h, sizeof(float) * (size_t)rows * h, hipMemcpyDeviceToHost));
	} else {
		if (rows != 1) return tg_fail(TG_ERR_BAD_ARG, "decode taps have one row");
		TG_HIP(hipMemcpy(out, s->xr + (size_t)b * h, sizeof(float) * h, hipMemcpyDeviceToHost));
	}
	return TG_OK;
}

int tg_session_kv(tg_session *s, int layer, float *keys, float *values, int *position_ptr, int *buffer_ptr, int *max_pos) {
	if (!s) return tg_fail(TG_ERR_BAD_ARG, "null session");
	const tg_config &c = s->m->cfg;
	if (layer < 0 || layer >= c.n_layers) return tg_fail(TG_ERR_BAD_ARG, "no such layer");
	TG_HIP(hipStreamSynchronize(g_stream));
	if (int rc = fused_check(s)) return rc;
	const size_t bytes = sizeof(float) * (size_t)s->max_pos[(size_t)layer] * c.head_dim;
	if (keys) TG_HIP(hipMemcpy(keys, s->kc[(size_t)layer], bytes, hipMemcpyDeviceToHost));
	if (values) TG_HIP(hipMemcpy(values, s->vc[(size_t)layer], bytes, hipMemcpyDeviceToHost));
	if (position_ptr) *position_ptr = s->pos;
	if (buffer_ptr) *buffer_ptr = s->m->L[(size_t)layer].is_sw ? s->bp_local : s->bp_global;
	if (max_pos) *max_pos = s->max_pos[(size_t)layer];
	return TG_OK;
}

}  // extern "C"
