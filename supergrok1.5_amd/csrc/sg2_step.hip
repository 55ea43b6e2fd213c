// C-ABI entry points of the SuperGrok v2 batched step: validation, workspace
// carving, the small per-call table upload and the launch sequence
//   keys -> 4 radix passes -> sharpness gather -> coefficient composition
//   -> chunk summaries -> chunk prefix -> scan output
//   -> per-element GRU/PEER/expert/Adam,
// and of the scan part of the bilevel pass (the same sort + scan with the
// tile-start states kept, and its adjoint).
// Stands behind supergrok2_mamba_peer_batched_step (csrc/ops.cpp:815-877 of
// the reference) in place of launch_mamba3_peer_batched_step
// (csrc/supergrok2_mamba_peer_kernels.cu:1754-2117).
#include <atomic>
#include <map>
#include <mutex>
#include <vector>

#include "sg2_internal.hpp"

namespace sg2 {
namespace {

// process-wide settings (atomic: a call reads each once; changing them while other threads are inside a call only
// affects calls that start later)
std::atomic<int> g_chunk_len{0};      // 0: chosen per call from the amount of work, see auto_chunk_len
std::atomic<int> g_window{SG2_DEFAULT_SCAN_WINDOW};

// What the forward call of the bilevel pass laid out in a workspace, so that the backward call addresses it the same
// way whatever the settings are by then.  Keyed by the workspace address.
struct BilevelRecord { int chunk_len, window, P, total; uint64_t seq; };
uint64_t g_bilevel_seq = 0;
constexpr size_t MAX_BILEVEL_RECORDS = 64;
std::mutex g_bilevel_mutex;
std::map<const void*, BilevelRecord> g_bilevel_records;

// Longer chunks mean fewer summaries (less work in the first scan pass and the prefix), shorter chunks
// mean more workgroups.  The replay runs one wave per chunk and direction, 2048 of them resident on 256 CUs:
// take the longest of 4096 / 2048 / 1024 that still gives two full rounds of them, else 512 (on the 14-tensor set
// of 0.42 M elements: 0.31 ms per step with 512, 0.36 with 1024, 0.33 with 256, whose summaries cost more than
// the extra waves gain).
// tensor sizes of a call, either as a plain array (the *_bytes queries) or read from the tensor records (no copy)
struct Numels {
    const int64_t* plain;
    const Sg2Tensor* tensors;
    int64_t operator[](int i) const { return plain ? plain[i] : tensors[i].numel; }
};

int auto_chunk_len(int P, Numels numels) {
    for (int L = 4096; L > 512; L >>= 1) {
        int64_t wgs = 0;
        for (int i = 0; i < P; i++) wgs += 2 * ((numels[i] + L - 1) / L);
        if (wgs >= 4096) return L;
    }
    return 512;
}
int effective_chunk_len(int P, Numels numels) {
    const int set = g_chunk_len.load();
    return set > 0 ? set : auto_chunk_len(P, numels);
}

// ---- optional per-stage timing with HIP events on the step's stream
constexpr int PROF_MARKS = SG2_PROF_STAGES + 1;
struct Prof {
    bool on = false;
    int calls = 0;
    std::vector<hipEvent_t> ev;     // [SG2_PROF_MAX_CALLS][PROF_MARKS], created on first enable
} g_prof;

struct Layout {
    int P, total, elem_tiles, sort_tiles, chunks, wchunks, nb;
    size_t off_tables, off_keys[2], off_vals[2], off_ssorted, off_spine, off_blocksums, off_summ, off_hstart, off_comp, off_flags, off_padw, off_ctx, off_htile, off_adj_summ, off_adj_lam, off_adj_part, off_adj_blk, bytes;
    size_t tables_bytes;
};

// Floats of the 20 scan weight tensors (input_proj W, b; 9 per direction) at a kernel geometry, each rounded up to
// a multiple of 4 floats so that every tensor starts 16-byte aligned.
inline size_t scan_weight_floats(const GeoInfo& gi, int k) {
    const size_t dm = gi.dm, ds = gi.ds, di = gi.di;
    const size_t block[9] = {2 * di * dm, di * di, di, ds * di, ds * di, di * ds, di, di * (ds / 2), dm * di};
    const size_t n = k == 0 ? 2 * dm : (k == 1 ? dm : block[(k - 2) % 9]);
    return (n + 3) / 4 * 4;
}
inline size_t padded_weight_floats(const GeoInfo& gi) {
    size_t n = 0;
    for (int k = 0; k < 20; k++) n += scan_weight_floats(gi, k);
    return n;
}

// A scan block smaller than the kernel geometry, embedded in it so that it computes the same function:
//   * rows / columns beyond the true d_model, d_inner, d_state of input_proj, in_proj, dt_W, B_proj, C_proj, D, rope
//     and out_proj are zero: the extra columns see a zero x-branch and gate, the extra states receive no input and
//     contribute nothing to y, the extra context entries are +0;
//   * every fma chain only gains terms with a zero factor, so the real entries keep their bits;
//   * the extra poles copy real ones (A_log[j][0] for extra states of a real column, column 0 for extra columns) and
//     the extra columns take dt_b[0]: their (never used) states contract like real ones, so the decisions that look
//     at all lanes (summary contraction, first-block length, polynomial limits) see nothing new.
struct PadArgs {
    const float* src[20];
    float* dst[20];
    int dm, ds, di;        // true dimensions
    int DM, DS, DI;        // kernel geometry
};
__global__ __launch_bounds__(256) void k_pad_weights(PadArgs a) {
    const int k = blockIdx.y;
    const int dm = a.dm, ds = a.ds, di = a.di, hp = ds / 2, DM = a.DM, DS = a.DS, DI = a.DI, HP = DS / 2;
    const int slot = k < 2 ? k : 2 + (k - 2) % 9;
    const int count = k == 0 ? 2 * DM : k == 1 ? DM : slot == 2 ? 2 * DI * DM : slot == 3 ? DI * DI : (slot == 4 || slot == 8) ? DI
                    : (slot == 5 || slot == 6) ? DS * DI : slot == 7 ? DI * DS : slot == 9 ? DI * HP : DM * DI;
    const float* __restrict__ src = a.src[k];
    float* __restrict__ dst = a.dst[k];
    for (int i = blockIdx.x * 256 + threadIdx.x; i < count; i += gridDim.x * 256) {
        float v = 0.0f;
        if (k == 0) { const int r = i / 2, c = i % 2; if (r < dm) v = src[r * 2 + c]; }                    // input_proj W [dm][2]
        else if (k == 1) { if (i < dm) v = src[i]; }                                                          // input_proj b
        else if (slot == 2) {                                                                                 // in_proj [2 di][dm]: x rows, then z rows
            const int r = i / DM, c = i % DM, part = r / DI, j = r % DI;
            if (j < di && c < dm) v = src[(part * di + j) * dm + c];
        } else if (slot == 3) { const int r = i / DI, c = i % DI; if (r < di && c < di) v = src[r * di + c]; } // dt_W [di][di]
        else if (slot == 4) v = src[i < di ? i : 0];                                                           // dt_b
        else if (slot == 5 || slot == 6) { const int r = i / DI, c = i % DI; if (r < ds && c < di) v = src[r * di + c]; }   // B_proj, C_proj [ds][di]
        else if (slot == 7) { const int j = i / DS, st = i % DS; v = src[(j < di ? j : 0) * ds + (st < ds ? st : 0)]; }     // A_log [di][ds]
        else if (slot == 8) { if (i < di) v = src[i]; }                                                        // D
        else if (slot == 9) { const int j = i / HP, q = i % HP; if (j < di && q < hp) v = src[j * hp + q]; }   // rope [di][ds/2]
        else { const int r = i / DI, c = i % DI; if (r < dm && c < di) v = src[r * di + c]; }                  // out_proj [dm][di]
        dst[i] = v;
    }
}

int make_layout(int geo, int P, Numels numels, int chunk_len, Layout* L, bool bilevel = false) {
    const GeoInfo gi = geo_info(geo);
    int64_t total = 0, et = 0, stl = 0, ch = 0, wch = 0;
    for (int i = 0; i < P; i++) {
        const int64_t n = numels[i];
        if (n < 0) return sg::fail("tensor %d: negative numel", i);
        if (n > 0x7fffffff) return sg::fail("tensor %d: numel %lld exceeds 2^31-1", i, (long long)n);
        total += n;
        et += (n + ELEM_TILE - 1) / ELEM_TILE;
        stl += (n + SORT_TILE - 1) / SORT_TILE;
        const int64_t nc = (n + chunk_len - 1) / chunk_len;
        ch += nc;
        wch += nc > 0 ? nc - 1 : 0;
    }
    if (total > 0x7ffffff0) return sg::fail("total element count %lld exceeds the 2^31 indexing limit", (long long)total);
    L->P = P; L->total = (int)total; L->elem_tiles = (int)et; L->sort_tiles = (int)stl;
    L->chunks = (int)ch; L->wchunks = (int)wch;
    L->nb = (int)((256 * stl + SCAN_BLOCK_ITEMS - 1) / SCAN_BLOCK_ITEMS);
    size_t o = 0;
    auto take = [&](size_t bytes) { size_t r = o; o = sg::align_up(o + bytes, 256); return r; };
    L->tables_bytes = sizeof(TensorDev) * (size_t)P + 4 * sizeof(int) * (size_t)(P + 1);
    L->off_tables = take(L->tables_bytes);
    for (int k = 0; k < 2; k++) L->off_keys[k] = take(4 * (size_t)total);
    for (int k = 0; k < 2; k++) L->off_vals[k] = take(4 * (size_t)total);
    L->off_ssorted = take(4 * (size_t)total);
    L->off_spine = take(4 * 256 * (size_t)stl);
    L->off_blocksums = take(4 * (size_t)(L->nb + 1));
    L->off_summ = take(4 * 2 * (size_t)wch * 6 * gi.threads);
    L->off_hstart = take(4 * 2 * (size_t)ch * 2 * gi.threads);
    L->off_comp = take(4 * (2 * 5 * (size_t)gi.rows * 3 + 2 * 2 * (size_t)gi.rows * 4 + 12));      // composed triples, Taylor polynomials, coefficient maxima and polynomial limits
    L->off_flags = take(4 * (2 * (size_t)P + 3));    // apart from the tensor records: it is written while those are being read
    L->off_padw = take(4 * (size_t)padded_weight_floats(gi));   // scan weights embedded in the kernel geometry (used when the caller's block is smaller)
    L->off_ctx = take(4 * 2 * (size_t)total * gi.dm);
    // bilevel only: state entering every HT_STEP-th step, both directions
    L->off_htile = take(bilevel ? 4 * 2 * (size_t)htile_count((int)total, P) * 2 * SCAN_THREADS : 0);
    L->off_adj_summ = take(bilevel ? 4 * 2 * (size_t)L->chunks * SCAN_THREADS * 6 : 0);
    L->off_adj_lam = take(bilevel ? 4 * 2 * (size_t)L->chunks * SCAN_THREADS * 2 : 0);
    L->off_adj_part = take(bilevel ? 4 * 2 * (size_t)ADJ_GROUPS * SG2_BWD_STRIDE : 0);
    L->off_adj_blk = take(bilevel ? 4 * 2 * (size_t)SG2_BWD_STRIDE : 0);
    L->bytes = o;
    return 0;
}


// Per-call tables travel as kernel arguments: UPLOAD_RECS tensor records and their entries of the four prefix
// tables (tiles of the elementwise kernels, sort tiles, scan chunks, chunks with a summary) per launch.
constexpr int UPLOAD_RECS = 24;
struct TableChunk {
    TensorDev rec[UPLOAD_RECS];
    int pre[4][UPLOAD_RECS];       // prefix table q, entries i0+1 .. i0+cnt
    TensorDev* dst_rec;
    int* dst_pre;                  // four tables of P+1 ints, back to back
    int* flags;                    // per-tensor "sharpness is not all zero" flags to clear, or NULL to keep them
    int* state_bad;                // with flags: per tensor, 1 when one of its carried Mamba states holds a non-finite entry
    int i0, cnt, P, state_floats;  // state_floats: d_inner * d_state of the caller's states
};
static_assert(sizeof(TableChunk) <= 3600, "kernel arguments stay well below 4 KB");

// Workgroup 0 writes the records and tables; workgroup 1 + k looks at the carried states of tensor i0 + k.
__global__ __launch_bounds__(256) void k_tables(TableChunk c) {
    if (blockIdx.x > 0) {
        // A tensor whose carried state is not finite (a diverged run) must come out non-finite as a whole, as it does in
        // the reference, which multiplies every chunk's start state through: the scan only lets contracted summaries
        // forget what came before them while every carried state of the call is finite (k_compose reads these flags).
        const int k = blockIdx.x - 1;
        const TensorDev& t = c.rec[k];
        bool bad = false;
        if (t.numel > 0)
            for (int r = threadIdx.x; r < 2 * c.state_floats; r += 256)
                bad = bad || !sg_isfinite((r < c.state_floats ? t.mfwd : t.mbwd)[r % c.state_floats]);
        const int any = __syncthreads_or(bad ? 1 : 0);
        if (threadIdx.x == 0) c.state_bad[c.i0 + k] = any ? 1 : 0;
        return;
    }
    constexpr int WORDS = sizeof(TensorDev) / 4;
    const int* src = reinterpret_cast<const int*>(c.rec);
    int* dst = reinterpret_cast<int*>(c.dst_rec + c.i0);
    for (int w = threadIdx.x; w < c.cnt * WORDS; w += 256) dst[w] = src[w];
    for (int w = threadIdx.x; w < 4 * c.cnt; w += 256) {
        const int q = w / c.cnt, k = w % c.cnt;
        c.dst_pre[q * (c.P + 1) + c.i0 + 1 + k] = c.pre[q][k];
    }
    if (c.i0 == 0 && threadIdx.x < 4) c.dst_pre[threadIdx.x * (c.P + 1)] = 0;
    if (c.flags != nullptr)
        for (int k = threadIdx.x; k < c.cnt; k += 256) c.flags[c.i0 + k] = 0;
}

}  // namespace

int geo_of(const SgDims* d) {
    if (!d) return sg::fail("dims is NULL"), -1;
    // the limits the reference enforces (csrc/supergrok2_mamba_peer_kernels.cu:1796-1801)
    if (d->d_state % 2) return sg::fail("d_state must be even for paired RoPE (got %d)", d->d_state), -1;
    if (d->d_state > 32) return sg::fail("d_state exceeds MAX_D_STATE (%d > 32)", d->d_state), -1;
    if (d->d_model > 16) return sg::fail("d_model exceeds MAX_D_MODEL (%d > 16)", d->d_model), -1;
    if (d->gru_hidden > 8) return sg::fail("gru_hidden exceeds MAX_GRU_HIDDEN (%d > 8)", d->gru_hidden), -1;
    if (d->d_inner > 32) return sg::fail("d_inner exceeds MAX_D_INNER (%d > 32)", d->d_inner), -1;
    if (d->d_inner % 4) return sg::fail("d_inner must be a multiple of 4 (got %d)", d->d_inner), -1;
    // what the reference takes for granted (its kernels index with these and would read out of bounds otherwise)
    if (d->d_model < 1 || d->d_state < 2 || d->d_inner < 4 || d->gru_hidden < 1 || d->num_heads < 1 || d->pk_dim < 1 ||
        d->expert_hidden < 1 || d->num_experts < 1)
        return sg::fail("meta-net dimensions must be positive (d_model %d, d_state %d, d_inner %d, gru_hidden %d, num_heads %d, pk_dim %d, "
                        "expert_hidden %d, num_experts %d)", d->d_model, d->d_state, d->d_inner, d->gru_hidden, d->num_heads, d->pk_dim,
                        d->expert_hidden, d->num_experts), -1;
    if (d->d_model % 2)
        return sg::fail("d_model must be even (got %d): a query is split into two halves of d_model/2 entries, one per product-key table "
                        "(grokking_optimizers/mamba3_peer_metanet.py:69,337-338)", d->d_model), -1;
    if ((int64_t)d->num_experts > (int64_t)d->pk_dim * d->pk_dim)
        return sg::fail("num_experts (%d) exceeds pk_dim^2 (%d): the product-key index a * pk_dim + b (csrc/supergrok2_mamba_peer_kernels.cu:1048) "
                        "cannot reach every expert", d->num_experts, d->pk_dim * d->pk_dim), -1;
    for (int geo = 0; geo < GEO_COUNT; geo++) {       // the smallest compiled geometry that holds the scan block
        const GeoInfo gi = geo_info(geo);
        if (d->d_model <= gi.dm && d->d_state <= gi.ds && d->d_inner <= gi.di) return geo;
    }
    return sg::fail("no scan geometry holds d_model %d, d_state %d, d_inner %d", d->d_model, d->d_state, d->d_inner), -1;
}

bool scan_exact(const SgDims* d, int geo) {
    const GeoInfo gi = geo_info(geo);
    return d->d_model == gi.dm && d->d_state == gi.ds && d->d_inner == gi.di;
}

int elem_kind_of(const SgDims* d, int geo) {
    if (!scan_exact(d, geo) || d->gru_hidden != GH || d->num_heads != NH || d->pk_dim != PK || d->num_experts != NE) return ELEM_ANY;
    if (d->expert_hidden == EH) return ELEM_FAST16;
    if (d->expert_hidden == 4 && geo == GEO_DEFAULT) return ELEM_FAST4;
    return ELEM_ANY;
}

int check_dims(const SgDims* d, bool per_element) {
    const int geo = geo_of(d);
    if (geo < 0) return 1;
    if (per_element && (d->gru_hidden != GH || d->num_heads != NH || d->pk_dim != PK || d->expert_hidden != EH || d->num_experts != NE ||
                        d->d_model != GeoDefault::DM))
        return sg::fail("the per-element kernel of the bilevel pass is built for d_model=%d gru_hidden=%d num_heads=%d pk_dim=%d expert_hidden=%d "
                        "num_experts=%d (got %d, %d, %d, %d, %d, %d); smaller d_model, gru_hidden and expert_hidden run embedded in these "
                        "(zero rows and columns)", GeoDefault::DM, GH, NH, PK, EH, NE, d->d_model, d->gru_hidden, d->num_heads, d->pk_dim,
                        d->expert_hidden, d->num_experts);
    if (geo != GEO_DEFAULT)
        return sg::fail("the scan kernels of the bilevel pass are built for blocks up to d_model=%d d_state=%d d_inner=%d (got %d, %d, %d)",
                        GeoDefault::DM, GeoDefault::DS, GeoDefault::DI, d->d_model, d->d_state, d->d_inner);
    return 0;
}

namespace {

}  // namespace

void prof_mark(int idx, hipStream_t st) {
    if (!g_prof.on || g_prof.calls >= SG2_PROF_MAX_CALLS) return;
    (void)hipEventRecord(g_prof.ev[(size_t)g_prof.calls * PROF_MARKS + idx], st);
}
}  // namespace sg2

extern "C" {

int sg2_profile_enable(int on) {
    using namespace sg2;
    if (on && g_prof.ev.empty()) {
        g_prof.ev.resize((size_t)SG2_PROF_MAX_CALLS * PROF_MARKS);
        for (auto& e : g_prof.ev) SG_HIP_CHECK(hipEventCreate(&e));
    }
    g_prof.on = on != 0;
    g_prof.calls = 0;
    return 0;
}

int sg2_profile_read(float* ms, int* calls) {
    using namespace sg2;
    if (!ms || !calls) return sg::fail("NULL argument");
    for (int k = 0; k < SG2_PROF_STAGES; k++) ms[k] = 0.0f;
    *calls = g_prof.calls;
    for (int c = 0; c < g_prof.calls; c++) {
        hipEvent_t* e = &g_prof.ev[(size_t)c * PROF_MARKS];
        SG_HIP_CHECK(hipEventSynchronize(e[PROF_MARKS - 1]));
        for (int k = 0; k < SG2_PROF_STAGES; k++) {
            float t = 0.0f;
            SG_HIP_CHECK(hipEventElapsedTime(&t, e[k], e[k + 1]));
            ms[k] += t;
        }
    }
    g_prof.calls = 0;
    return 0;
}

const char* sg_last_error(void) { return sg::last_error().c_str(); }

int sg2_set_chunk_len(int chunk_len) {
    if (chunk_len < 0 || chunk_len % sg2::SCAN_TT) return sg::fail("chunk_len must be 0 (automatic) or a positive multiple of %d", sg2::SCAN_TT);
    sg2::g_chunk_len = chunk_len;
    return 0;
}
int sg2_get_chunk_len(void) { return sg2::g_chunk_len.load(); }
int sg2_chunk_len_for(int num_tensors, const int64_t* numels) {
    if (num_tensors < 0 || (num_tensors > 0 && !numels)) return 0;
    return sg2::effective_chunk_len(num_tensors, sg2::Numels{numels, nullptr});
}

int sg2_set_scan_window(int window) {
    if (window < 0) window = SG2_DEFAULT_SCAN_WINDOW;
    if (window % sg2::SCAN_TT) return sg::fail("scan window must be a multiple of %d (0 disables it)", sg2::SCAN_TT);
    sg2::g_window = window;
    return 0;
}
int sg2_get_scan_window(void) { return sg2::g_window.load(); }

size_t sg2_workspace_bytes(const SgDims* dims, int num_tensors, const int64_t* numels) {
    const int geo = sg2::geo_of(dims);
    if (geo < 0 || num_tensors < 0 || (num_tensors > 0 && !numels)) return 0;
    sg2::Layout L;
    if (sg2::make_layout(geo, num_tensors, sg2::Numels{numels, nullptr}, sg2::effective_chunk_len(num_tensors, sg2::Numels{numels, nullptr}), &L)) return 0;
    return L.bytes;
}

}  // extern "C"

namespace sg2 {
// Validates the call, lays out the workspace, uploads the per-tensor records and fills the Plan.  full_step:
// the optimizer-state pointers of every tensor are required; otherwise only grad, sharpness and the two Mamba
// states (bilevel forward/backward).  Returns 0 with pl->total == 0 when there is nothing to do.
int build_plan(const SgDims* dims, const Sg2Weights* weights, int num_tensors, const Sg2Tensor* tensors, const Sg2Scalars* scalars,
               void* workspace, size_t workspace_bytes, bool full_step, bool bilevel, bool keep_flags, hipStream_t st, Plan* plp, Layout* Lp,
               int chunk_override = 0, int window_override = -1) {
    Plan& pl = *plp;
    Layout& L = *Lp;
    pl.total = 0;
    const int geo = geo_of(dims);
    if (geo < 0 || (bilevel && check_dims(dims))) return 1;
    pl.geo = geo;
    pl.elem_kind = elem_kind_of(dims, geo);
    pl.st_di = dims->d_inner;
    pl.st_ds = dims->d_state;
    pl.dims = *dims;
    if (num_tensors == 0) return 0;
    if (num_tensors < 0 || !tensors || !weights || !scalars) return sg::fail("NULL argument");
    for (int k = 0; k < SG2_NUM_WEIGHTS; k++)
        if (!weights->w[k]) return sg::fail("weight pointer %d is NULL", k);
    const int P = num_tensors;

    const Numels numels = {nullptr, tensors};
    for (int i = 0; i < P; i++) {
        const Sg2Tensor& t = tensors[i];
        if (t.numel > 0) {
            if (!t.grad || !t.sharpness || !t.mamba_fwd_state || !t.mamba_bwd_state) return sg::fail("tensor %d: NULL pointer", i);
            if (full_step && (!t.param || !t.exp_avg || !t.exp_avg_sq || !t.mu || !t.gru_state)) return sg::fail("tensor %d: NULL pointer", i);
            if (t.dtype != SG_F32 && t.dtype != SG_F16 && t.dtype != SG_BF16) return sg::fail("tensor %d: bad dtype %d", i, t.dtype);
            if (full_step && ((uintptr_t)t.gru_state & 15u) != 0) return sg::fail("tensor %d: gru_state must be 16-byte aligned", i);
        }
    }
    const int chunk_len = chunk_override > 0 ? chunk_override : effective_chunk_len(P, numels);
    if (make_layout(geo, P, numels, chunk_len, &L, bilevel)) return 1;
    if (L.total == 0) return 0;
    if (!workspace || workspace_bytes < L.bytes)
        return sg::fail("workspace too small: need %zu bytes, got %zu", L.bytes, workspace_bytes);
    if (((uintptr_t)workspace & 255u) != 0) return sg::fail("workspace must be 256-byte aligned");
    // ---- per-tensor records and the four prefix tables: written by k_tables from kernel arguments, UPLOAD_RECS
    // tensors per launch (no host-to-device copy: nothing here blocks the host or depends on the lifetime of host
    // memory, and the call can be recorded into a graph)
    unsigned char* ws = static_cast<unsigned char*>(workspace);
    {
        TensorDev* d_rec = reinterpret_cast<TensorDev*>(ws + L.off_tables);
        int* d_pre = reinterpret_cast<int*>(ws + L.off_tables + sizeof(TensorDev) * (size_t)P);
        int* d_flags = keep_flags ? nullptr : reinterpret_cast<int*>(ws + L.off_flags);
        int off = 0, run[4] = {0, 0, 0, 0};
        for (int i0 = 0; i0 < P; i0 += UPLOAD_RECS) {
            TableChunk c;
            c.dst_rec = d_rec; c.dst_pre = d_pre; c.flags = d_flags;
            c.state_bad = reinterpret_cast<int*>(ws + L.off_flags) + P + 3;
            c.state_floats = dims->d_inner * dims->d_state;
            c.i0 = i0; c.cnt = P - i0 < UPLOAD_RECS ? P - i0 : UPLOAD_RECS; c.P = P;
            for (int k = 0; k < c.cnt; k++) {
                const Sg2Tensor& t = tensors[i0 + k];
                const int n = (int)t.numel;
                const int nc = (n + chunk_len - 1) / chunk_len;
                TensorDev& d = c.rec[k];
                d.param = t.param; d.grad = t.grad; d.sharp = t.sharpness;
                d.ea = t.exp_avg; d.easq = t.exp_avg_sq; d.mu = t.mu; d.gru = t.gru_state;
                d.mfwd = t.mamba_fwd_state; d.mbwd = t.mamba_bwd_state;
                d.off = off; d.numel = n; d.dtype = t.dtype; d.nchunks = nc;
                d.alpha = t.alpha_mu; d.lamb = t.lamb_eff; d.beta1 = t.beta1; d.bc2 = t.bc2;
                d.step_size = full_step ? scalars->lr / t.bc1 : 0.0f;
                for (int q = 0; q < 5; q++) d.pad_[q] = 0;
                off += n;
                run[0] += (n + ELEM_TILE - 1) / ELEM_TILE;
                run[1] += (n + SORT_TILE - 1) / SORT_TILE;
                run[2] += nc;
                run[3] += nc > 0 ? nc - 1 : 0;
                for (int q = 0; q < 4; q++) c.pre[q][k] = run[q];
            }
            hipLaunchKernelGGL(k_tables, dim3(d_flags ? 1 + c.cnt : 1), dim3(256), 0, st, c);
            SG_LAUNCH_CHECK("k_tables");
        }
    }

    pl.tensors = reinterpret_cast<const TensorDev*>(ws + L.off_tables);
    const int* dpre = reinterpret_cast<const int*>(ws + L.off_tables + sizeof(TensorDev) * (size_t)P);
    pl.elem_tile_prefix = dpre;
    pl.sort_tile_prefix = dpre + (P + 1);
    pl.chunk_prefix = dpre + 2 * (P + 1);
    pl.wchunk_prefix = dpre + 3 * (P + 1);
    pl.P = P; pl.total = L.total; pl.elem_tiles = L.elem_tiles; pl.sort_tiles = L.sort_tiles;
    pl.chunks = L.chunks; pl.wchunks = L.wchunks; pl.chunk_len = chunk_len; pl.window = window_override >= 0 ? window_override : g_window.load();
    for (int k = 0; k < 2; k++) {
        pl.keys[k] = reinterpret_cast<uint32_t*>(ws + L.off_keys[k]);
        pl.vals[k] = reinterpret_cast<int32_t*>(ws + L.off_vals[k]);
    }
    pl.ssorted = reinterpret_cast<float*>(ws + L.off_ssorted);
    pl.spine = reinterpret_cast<uint32_t*>(ws + L.off_spine);
    pl.blocksums = reinterpret_cast<uint32_t*>(ws + L.off_blocksums);
    pl.summaries = reinterpret_cast<float*>(ws + L.off_summ);
    pl.hstart = reinterpret_cast<float*>(ws + L.off_hstart);
    pl.comp = reinterpret_cast<float*>(ws + L.off_comp);
    pl.sharp_nonzero = reinterpret_cast<int*>(ws + L.off_flags);
    pl.contracted = pl.sharp_nonzero + P;
    pl.state_bad = pl.contracted + 3;
    pl.ctx = reinterpret_cast<float*>(ws + L.off_ctx);
    pl.decay = 1.0f - scalars->lr * scalars->wd_eff;
    pl.beta2 = scalars->beta2; pl.eps = scalars->eps; pl.rescale = scalars->rescale;
    pl.W = *weights;
    if (!scan_exact(dims, geo)) {
        // the caller's scan block is smaller than the kernel geometry: embed its 20 weight tensors (every call: the
        // caller may have changed them) and let the sort / scan kernels read the embedded copies
        const GeoInfo gi = geo_info(geo);
        PadArgs a;
        float* at = reinterpret_cast<float*>(ws + L.off_padw);
        for (int k = 0; k < 20; k++) {
            a.src[k] = weights->w[k];
            a.dst[k] = at;
            pl.W.w[k] = at;
            at += scan_weight_floats(gi, k);
        }
        a.dm = dims->d_model; a.ds = dims->d_state; a.di = dims->d_inner;
        a.DM = gi.dm; a.DS = gi.ds; a.DI = gi.di;
        hipLaunchKernelGGL(k_pad_weights, dim3(4, 20), dim3(256), 0, st, a);
        SG_LAUNCH_CHECK("k_pad_weights");
    }

    pl.htile = bilevel ? reinterpret_cast<float*>(ws + L.off_htile) : nullptr;
    pl.scan_out[0] = pl.scan_out[1] = nullptr;
    pl.adj_summ = bilevel ? reinterpret_cast<float*>(ws + L.off_adj_summ) : nullptr;
    pl.adj_lam = bilevel ? reinterpret_cast<float*>(ws + L.off_adj_lam) : nullptr;
    pl.adj_part = bilevel ? reinterpret_cast<float*>(ws + L.off_adj_part) : nullptr;
    pl.adj_blk = bilevel ? reinterpret_cast<float*>(ws + L.off_adj_blk) : nullptr;
    return 0;
}

// per-call options -> the override arguments of build_plan (0 / -1: the process-wide settings)
int resolve_options(const Sg2Options* o, int P, Numels numels, int* chunk_len, int* window) {
    *chunk_len = 0;
    *window = -1;
    if (!o) return 0;
    if (o->chunk_len < 0 || o->chunk_len % SCAN_TT) return sg::fail("options: chunk_len must be 0 (automatic) or a positive multiple of %d", SCAN_TT);
    if (o->scan_window > 0 && o->scan_window % SCAN_TT) return sg::fail("options: scan_window must be a multiple of %d (0 disables it, negative = default)", SCAN_TT);
    *chunk_len = o->chunk_len > 0 ? o->chunk_len : auto_chunk_len(P, numels);
    *window = o->scan_window < 0 ? SG2_DEFAULT_SCAN_WINDOW : o->scan_window;
    return 0;
}

int run_step(const SgDims* dims, const Sg2Weights* weights, int num_tensors, const Sg2Tensor* tensors, const Sg2Scalars* scalars,
             int32_t* expert_counts, void* workspace, size_t workspace_bytes, const Sg2Debug* debug, hipStream_t st,
             const Sg2Options* options = nullptr) {
    Plan pl;
    Layout L;
    int chunk_override = 0, window_override = -1;
    if (options && num_tensors > 0 && tensors && resolve_options(options, num_tensors, Numels{nullptr, tensors}, &chunk_override, &window_override)) return 1;
    if (build_plan(dims, weights, num_tensors, tensors, scalars, workspace, workspace_bytes, true, false, false, st, &pl, &L, chunk_override,
                   window_override))
        return 1;
    if (pl.total == 0) return 0;
    prof_mark(0, st);
    if (launch_sort(pl, debug ? debug->perm : nullptr, st)) return 1;
    prof_mark(1, st);
    if (launch_scan(pl, st)) return 1;
    if (debug && debug->ctx) {    // [2][total][d_model] for the caller; the kernels' rows are d_model of the kernel geometry wide
        if (dims->d_model == geo_info(pl.geo).dm)
            SG_HIP_CHECK(hipMemcpyAsync(debug->ctx, pl.ctx, 4 * 2 * (size_t)L.total * dims->d_model, hipMemcpyDeviceToDevice, st));
        else
            SG_HIP_CHECK(hipMemcpy2DAsync(debug->ctx, 4 * (size_t)dims->d_model, pl.ctx, 4 * (size_t)geo_info(pl.geo).dm,
                                          4 * (size_t)dims->d_model, 2 * (size_t)L.total, hipMemcpyDeviceToDevice, st));
    }
    if (launch_elem(pl, expert_counts, debug ? debug->expert_idx : nullptr, st)) return 1;
    prof_mark(5, st);
    if (g_prof.on && g_prof.calls < SG2_PROF_MAX_CALLS) g_prof.calls++;
    return 0;
}

// Scratch of sg2_batched_step_static: one array per GPU the library runs on, held until the process ends.  The
// array's name is only a handle in host code; its device address is looked up once per device.
static __device__ __align__(256) unsigned char scratch[SG2_STATIC_SCRATCH_BYTES];
constexpr int MAX_DEVICES = 64;
void* g_scratch_ptr[MAX_DEVICES] = {};
std::mutex g_scratch_mutex;

int static_scratch_address(void** out) {
    int dev = -1;
    SG_HIP_CHECK(hipGetDevice(&dev));
    if (dev < 0 || dev >= MAX_DEVICES) return sg::fail("device index %d outside 0..%d", dev, MAX_DEVICES - 1);
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (g_scratch_ptr[dev] == nullptr) {
        void* p = nullptr;
        SG_HIP_CHECK(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
        if (p == nullptr) return sg::fail("hipGetSymbolAddress returned NULL for the static scratch buffer");
        g_scratch_ptr[dev] = p;
    }
    *out = g_scratch_ptr[dev];
    return 0;
}
}  // namespace sg2

extern "C" {

int sg2_batched_step(const SgDims* dims, const Sg2Weights* weights, int num_tensors, const Sg2Tensor* tensors,
                     const Sg2Scalars* scalars, int32_t* expert_counts, void* workspace, size_t workspace_bytes,
                     const Sg2Debug* debug, void* stream) {
    return sg2::run_step(dims, weights, num_tensors, tensors, scalars, expert_counts, workspace, workspace_bytes, debug,
                         (hipStream_t)stream);
}

size_t sg2_workspace_bytes_opt(const SgDims* dims, int num_tensors, const int64_t* numels, const Sg2Options* options) {
    if (!options) return sg2_workspace_bytes(dims, num_tensors, numels);
    const int geo = sg2::geo_of(dims);
    if (geo < 0 || num_tensors < 0 || (num_tensors > 0 && !numels)) return 0;
    int chunk_len = 0, window = -1;
    if (sg2::resolve_options(options, num_tensors, sg2::Numels{numels, nullptr}, &chunk_len, &window)) return 0;
    sg2::Layout L;
    if (sg2::make_layout(geo, num_tensors, sg2::Numels{numels, nullptr}, chunk_len, &L)) return 0;
    return L.bytes;
}

int sg2_batched_step_opt(const SgDims* dims, const Sg2Weights* weights, int num_tensors, const Sg2Tensor* tensors,
                         const Sg2Scalars* scalars, int32_t* expert_counts, void* workspace, size_t workspace_bytes,
                         const Sg2Debug* debug, const Sg2Options* options, void* stream) {
    return sg2::run_step(dims, weights, num_tensors, tensors, scalars, expert_counts, workspace, workspace_bytes, debug,
                         (hipStream_t)stream, options);
}

size_t sg2_static_scratch_bytes(void) { return SG2_STATIC_SCRATCH_BYTES; }

int sg2_batched_step_static(const SgDims* dims, const Sg2Weights* weights, int num_tensors, const Sg2Tensor* tensors,
                            const Sg2Scalars* scalars, int32_t* expert_counts, const Sg2Debug* debug, void* stream) {
    using namespace sg2;
    const int geo = geo_of(dims);
    if (geo < 0) return 1;
    if (num_tensors < 0 || (num_tensors > 0 && !tensors)) return sg::fail("NULL argument");
    Layout L;
    const Numels numels = {nullptr, tensors};
    if (make_layout(geo, num_tensors, numels, effective_chunk_len(num_tensors, numels), &L)) return 1;
    if (L.bytes > SG2_STATIC_SCRATCH_BYTES)
        return sg::fail("sg2_batched_step_static: these tensors need %zu bytes of scratch, the library's static buffer holds %zu "
                        "(about 700 000 elements per call); use sg2_batched_step with a caller-provided workspace",
                        L.bytes, (size_t)SG2_STATIC_SCRATCH_BYTES);
    void* ws = nullptr;
    if (static_scratch_address(&ws)) return 1;
    return run_step(dims, weights, num_tensors, tensors, scalars, expert_counts, ws, SG2_STATIC_SCRATCH_BYTES, debug,
                    (hipStream_t)stream);
}

int sg2_meta_forward(const SgDims* dims, const Sg2Weights* weights, int num_tensors, const Sg2Tensor* tensors, float rescale,
                     float* smart_out, float* gru_out, int32_t* expert_counts, void* workspace, size_t workspace_bytes, void* stream) {
    using namespace sg2;
    hipStream_t st = (hipStream_t)stream;
    Plan pl;
    Layout L;
    const Sg2Scalars none = {rescale, 0.0f, 0.0f, 0.0f, 0.0f};
    if (num_tensors > 0 && tensors)
        for (int i = 0; i < num_tensors; i++)
            if (tensors[i].numel > 0 && !tensors[i].gru_state) return sg::fail("tensor %d: gru_state is NULL", i);
    if (build_plan(dims, weights, num_tensors, tensors, &none, workspace, workspace_bytes, false, false, false, st, &pl, &L)) return 1;
    if (pl.total == 0) return 0;
    if (!smart_out || !gru_out) return sg::fail("smart_out / gru_out is NULL");
    if (launch_sort(pl, nullptr, st)) return 1;
    if (launch_scan(pl, st)) return 1;
    return launch_elem_forward(pl, expert_counts, smart_out, gru_out, st);
}

size_t sg2_bilevel_workspace_bytes(const SgDims* dims, int num_tensors, const int64_t* numels) {
    if (sg2::check_dims(dims) || num_tensors < 0 || (num_tensors > 0 && !numels)) return 0;
    sg2::Layout L;
    if (sg2::make_layout(sg2::GEO_DEFAULT, num_tensors, sg2::Numels{numels, nullptr}, sg2::effective_chunk_len(num_tensors, sg2::Numels{numels, nullptr}), &L, true)) return 0;
    return L.bytes;
}

int sg2_bilevel_forward_ex(const SgDims* dims, const Sg2Weights* weights, int num_tensors, const Sg2Tensor* tensors, float* ctx_out,
                           const Sg2BilevelExtra* extra, void* workspace, size_t workspace_bytes, void* stream) {
    using namespace sg2;
    hipStream_t st = (hipStream_t)stream;
    Plan pl;
    Layout L;
    const Sg2Scalars none = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
    if (build_plan(dims, weights, num_tensors, tensors, &none, workspace, workspace_bytes, false, true, false, st, &pl, &L)) return 1;
    {
        std::lock_guard<std::mutex> lock(g_bilevel_mutex);
        // bounded memory: a workspace whose forward call is the oldest on record is forgotten first (a live pair of
        // forward and backward calls is only ever separated by the calls of other workspaces still in use)
        while (g_bilevel_records.size() >= MAX_BILEVEL_RECORDS && g_bilevel_records.find(workspace) == g_bilevel_records.end()) {
            auto oldest = g_bilevel_records.begin();
            for (auto it = g_bilevel_records.begin(); it != g_bilevel_records.end(); ++it)
                if (it->second.seq < oldest->second.seq) oldest = it;
            g_bilevel_records.erase(oldest);
        }
        g_bilevel_records[workspace] = BilevelRecord{pl.total > 0 ? pl.chunk_len : 0, pl.total > 0 ? pl.window : 0, num_tensors, pl.total, ++g_bilevel_seq};
    }
    if (pl.total == 0) return 0;
    if (extra && !scan_exact(dims, pl.geo))
        return sg::fail("sg2_bilevel_forward_ex: the extra outputs are laid out for d_model=%d d_state=%d d_inner=%d only", GeoDefault::DM,
                        GeoDefault::DS, GeoDefault::DI);
    if (ctx_out) pl.ctx = ctx_out;                 // else the contexts stay in the workspace
    if (extra) { pl.scan_out[0] = extra->scan_out_fwd; pl.scan_out[1] = extra->scan_out_bwd; }
    if (launch_sort(pl, extra ? extra->perm : nullptr, st)) return 1;
    if (launch_scan(pl, st)) return 1;
    if (extra && launch_saved_intermediates(pl, *extra, st)) return 1;
    if (extra && extra->x_sorted) return launch_x_sorted(pl, extra->x_sorted, st);
    return 0;
}

int sg2_bilevel_forward(const SgDims* dims, const Sg2Weights* weights, int num_tensors, const Sg2Tensor* tensors, float* ctx_out,
                        void* workspace, size_t workspace_bytes, void* stream) {
    if (!ctx_out && num_tensors > 0) return sg::fail("ctx_out is NULL");
    return sg2_bilevel_forward_ex(dims, weights, num_tensors, tensors, ctx_out, nullptr, workspace, workspace_bytes, stream);
}

int sg2_bilevel_backward_ex(const SgDims* dims, const Sg2Weights* weights, int num_tensors, const Sg2Tensor* tensors, const float* d_ctx,
                            const float* d_scan_out_fwd, const float* d_scan_out_bwd, const float* row_dx, float* dx_out, float* grads_out,
                            void* workspace, size_t workspace_bytes, void* stream) {
    using namespace sg2;
    hipStream_t st = (hipStream_t)stream;
    Plan pl;
    Layout L;
    const Sg2Scalars none = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
    if (!grads_out) return sg::fail("grads_out is NULL");
    BilevelRecord rec;
    {
        std::lock_guard<std::mutex> lock(g_bilevel_mutex);
        const auto it = g_bilevel_records.find(workspace);
        if (it == g_bilevel_records.end())
            return sg::fail("sg2_bilevel_backward: no forward call has been made on this workspace");
        rec = it->second;
    }
    // the layout of the forward call (its chunk length and window, whatever the settings are now): sorted keys /
    // payloads / sharpness, the sharpness flags, coefficients and tile states are still in place
    if (build_plan(dims, weights, num_tensors, tensors, &none, workspace, workspace_bytes, false, true, true, st, &pl, &L, rec.chunk_len,
                   rec.window))
        return 1;
    if (num_tensors != rec.P || pl.total != rec.total)
        return sg::fail("sg2_bilevel_backward: %d tensors / %d elements, but the forward call on this workspace had %d / %d", num_tensors,
                        pl.total, rec.P, rec.total);
    if ((d_scan_out_fwd != nullptr) != (d_scan_out_bwd != nullptr)) return sg::fail("d_scan_out: both directions or neither");
    if (pl.total > 0 && ((d_ctx != nullptr) == (d_scan_out_fwd != nullptr))) return sg::fail("exactly one of d_ctx and d_scan_out must be given");
    if (dx_out != nullptr && row_dx == nullptr) return sg::fail("dx_out needs row_dx");
    if ((d_scan_out_fwd != nullptr || row_dx != nullptr) && !scan_exact(dims, pl.geo))
        return sg::fail("sg2_bilevel_backward_ex: d_scan_out / row_dx are laid out for d_model=%d d_state=%d d_inner=%d only", GeoDefault::DM,
                        GeoDefault::DS, GeoDefault::DI);
    const float* const d_scan[2] = {d_scan_out_fwd, d_scan_out_bwd};
    return launch_bilevel_backward(pl, d_ctx, d_scan, row_dx, dx_out, grads_out, st);
}

int sg2_bilevel_backward(const SgDims* dims, const Sg2Weights* weights, int num_tensors, const Sg2Tensor* tensors, const float* d_ctx,
                         float* grads_out, void* workspace, size_t workspace_bytes, void* stream) {
    if (num_tensors > 0 && !d_ctx) return sg::fail("d_ctx is NULL");
    return sg2_bilevel_backward_ex(dims, weights, num_tensors, tensors, d_ctx, nullptr, nullptr, nullptr, nullptr, grads_out, workspace,
                                   workspace_bytes, stream);
}

}  // extern "C"
