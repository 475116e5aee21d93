// Lifecycle of a drafter between speculation cycles: prefix, pending token and transactions.
//
// Mirrors the state machine of Gemma3DraftPlan (include/local_gguf_engine/engine/gemma3_draft.hpp:56-82;
// src/engine/gemma3_draft.mm:1300-1490; lifecycle cases tests/engine/gemma3_draft_tests.cpp:206-277):
//
//   position       tokens the plan knows, a pending one included
//   materialized   tokens whose K/V rows exist; a pending token (the drafter's last emission, or one restored
//                  by the caller) gets its rows only when the next input needs them
//   transaction    begin .. commit_prefix(p) | abort: rows written in between can be taken back
//
// The reference keeps a transaction's rows in a private arena that attention reads beside the ring.  Here a
// transaction's rows go to the rings at once, where the ring attention of guffin_hip_forward_rows sees them,
// and the ring rows they overwrite (a local layer's slot (position & mask) held position - window) are first
// saved per position in a backup arena per layer (the plan's transaction capacity, a constructor argument as in
// the reference, rounded up to a power of two); abort, truncate and a commit of a shorter prefix copy them back.
// The final normalised row of every position a transaction runs is kept as well (the reference's private_norm,
// gemma3_draft.mm:966-968, 984-992), so that logits can be projected at a frontier a truncate or a shorter commit
// went back to.  Same observable behaviour: an aborted or truncated suffix leaves every ring row as it was, and
// logits after a commit equal those of a plain replay of the kept tokens.
//
// Every call is host-synchronous (it returns when its device work is done); the path that is timed is
// guffin_hip_h1_step, which needs none of this.
#include <algorithm>
#include <cstring>
#include <vector>

#include "common.hpp"

#define GUFFIN_TRY(expr) do { if (int rc_ = (expr)) return rc_; } while (0)

namespace guffin {
namespace {

constexpr uint32_t kDefaultTransactionRows = 32;   // when the caller names none (the reference's callers use 96 or 256)
constexpr uint32_t kMaxHorizon = 23;        // external_speculation_max_horizon
constexpr uint64_t kLawBytes = 8 + 256 * 4 + 257 * 8;
struct Draws { uint32_t word, pad; double u_accept, u_residual, u_next; };

struct Carve {
    uint8_t* base; uint64_t used;
    template <typename T> T* take(uint64_t count) {
        used = (used + 255) & ~uint64_t{255};
        T* p = base ? reinterpret_cast<T*>(base + used) : nullptr;
        used += count * sizeof(T);
        return p;
    }
};

struct Buffers {
    uint8_t* forward; uint64_t forward_bytes;
    uint16_t *priv_k, *priv_v, *backup_k, *backup_v;
    float *hidden, *hidden_sums, *hidden_saved, *sums_saved, *txn_hidden, *logits, *parts, *scores;
    uint32_t *tokens, *drafted, *history, *status, *proposal;
    Draws* draws;
    uint8_t *law_ws, *law;
    uint64_t* cdf;
    void **ring_k_table, **ring_v_table;
};

uint32_t arena_rows(uint32_t transaction_rows) {
    uint32_t rows = 1;
    while (rows < transaction_rows) rows <<= 1;
    return rows;
}

Buffers carve(const guffin_model_desc& m, uint32_t arena, void* workspace, uint64_t* total) {
    Carve c {static_cast<uint8_t*>(workspace), 0};
    Buffers b {};
    const uint64_t kvw = uint64_t(m.kv_heads) * m.head_dim;
    b.forward_bytes = guffin_hip_forward_scratch_bytes(&m, 2, m.ring_global - 2);
    b.forward = c.take<uint8_t>(b.forward_bytes);
    b.priv_k = c.take<uint16_t>(uint64_t(m.layer_count) * 2 * kvw);
    b.priv_v = c.take<uint16_t>(uint64_t(m.layer_count) * 2 * kvw);
    b.backup_k = c.take<uint16_t>(uint64_t(m.layer_count) * arena * kvw);
    b.backup_v = c.take<uint16_t>(uint64_t(m.layer_count) * arena * kvw);
    b.hidden = c.take<float>(2 * uint64_t(m.hidden));
    b.hidden_sums = c.take<float>(guffin_hip_receipt_bytes(2, m.hidden) / 4);
    b.hidden_saved = c.take<float>(2 * uint64_t(m.hidden));
    b.sums_saved = c.take<float>(guffin_hip_receipt_bytes(2, m.hidden) / 4);
    b.txn_hidden = c.take<float>(uint64_t(arena) * m.hidden);
    b.logits = c.take<float>(2 * uint64_t(m.vocab));
    b.parts = c.take<float>(uint64_t(std::max(1u, guffin_hip_gemv_packed_slices(m.head_dtype, m.hidden, m.vocab))) * 2 * m.vocab);
    b.scores = c.take<float>(m.vocab);
    b.tokens = c.take<uint32_t>(2);
    b.drafted = c.take<uint32_t>(kMaxHorizon + 1);
    b.history = c.take<uint32_t>(64);
    b.status = c.take<uint32_t>(1);
    b.proposal = c.take<uint32_t>(1);
    b.draws = c.take<Draws>(kMaxHorizon);
    b.law_ws = c.take<uint8_t>(guffin_hip_draft_law_any_workspace_bytes(m.vocab));
    b.law = c.take<uint8_t>(kLawBytes);
    b.cdf = c.take<uint64_t>(uint64_t(m.vocab) + 1);
    b.ring_k_table = c.take<void*>(m.layer_count);
    b.ring_v_table = c.take<void*>(m.layer_count);
    if (total) *total = (c.used + 255) & ~uint64_t{255};
    return b;
}

Buffers carve(const guffin_draft_plan* p) { return carve(*p->model, p->transaction_arena, p->workspace, nullptr); }

int usable(const guffin_draft_plan* p, const char* what) {
    if (!p || !p->model || !p->workspace) return fail(GUFFIN_E_ARG, what);
    if (p->poisoned) return fail(GUFFIN_E_STATE, "draft_plan: the plan is poisoned (a device status was raised); reset it");
    return GUFFIN_OK;
}

int poison(guffin_draft_plan* p, int code, const char* what) {
    p->poisoned = 1;
    return fail(code, what);
}

// ring rows [first, end) of every layer to the backup arena (save) or back (restore)
int move_rows(hipStream_t s, const guffin_draft_plan* p, const Buffers& b, uint32_t first, uint32_t end, bool save) {
    const guffin_model_desc& m = *p->model;
    if (end <= first) return GUFFIN_OK;
    const uint64_t kvw = uint64_t(m.kv_heads) * m.head_dim;
    for (uint32_t l = 0; l < m.layer_count; ++l) {
        const uint32_t ring_mask = (layer_is_local(m.global_period, l) ? m.ring_local : m.ring_global) - 1;
        const uint32_t arena = p->transaction_arena;
        void* bk = b.backup_k + uint64_t(l) * arena * kvw;
        void* bv = b.backup_v + uint64_t(l) * arena * kvw;
        void* rk = m.layers[l].ring_k;
        void* rv = m.layers[l].ring_v;
        const int rc = save ? guffin_hip_kv_cache_copy(s, rk, rv, bk, bv, first, end - first, ring_mask, arena - 1, kvw)
                            : guffin_hip_kv_cache_copy(s, bk, bv, rk, rv, first, end - first, arena - 1, ring_mask, kvw);
        if (rc) return rc;
    }
    return GUFFIN_OK;
}

// one pass of `rows` tokens (already in b.tokens) at the materialized frontier, published to the rings
int forward(hipStream_t s, guffin_draft_plan* p, const Buffers& b, uint32_t rows) {
    const guffin_model_desc& m = *p->model;
    const uint32_t at = p->materialized;
    if (p->transaction_active && at + rows > p->backup_end) {   // rows below backup_end already hold the originals
        const uint32_t first = std::max(at, p->backup_end);
        GUFFIN_TRY(move_rows(s, p, b, first, at + rows, true));
        p->backup_end = at + rows;
    }
    // The resident pass can give up a wait (a device shared with other work): its rows, and whatever else it
    // raised in the status word, are then not to be trusted.  These calls are host-synchronous anyway: the status
    // word is read before and after such a pass and, if the bit came up, put back, the resident form is switched
    // off for the process and the pass runs again, one launch per operator.
    const bool watched = resident_chosen(m, rows) && g_forward_mode == 0;
    uint32_t before = 0, after = 0;
    if (watched && (hipStreamSynchronize(s) != hipSuccess || hipMemcpy(&before, b.status, 4, hipMemcpyDeviceToHost) != hipSuccess))
        return fail(GUFFIN_E_HIP, "draft_plan: the stream failed");
    GUFFIN_TRY(guffin_hip_forward_rows(s, &m, b.tokens, rows, at, b.forward, b.forward_bytes, b.priv_k, b.priv_v, b.hidden,
                                       b.hidden_sums, b.status));
    if (watched) {
        if (hipStreamSynchronize(s) != hipSuccess || hipMemcpy(&after, b.status, 4, hipMemcpyDeviceToHost) != hipSuccess)
            return fail(GUFFIN_E_HIP, "draft_plan: the pass failed");
        if ((after & GUFFIN_STATUS_SYNC) && !(before & GUFFIN_STATUS_SYNC)) {
            resident_note_status(after);
            if (hipMemcpy(b.status, &before, 4, hipMemcpyHostToDevice) != hipSuccess) return fail(GUFFIN_E_HIP, "draft_plan: the pass failed");
            GUFFIN_TRY(guffin_hip_forward_rows(s, &m, b.tokens, rows, at, b.forward, b.forward_bytes, b.priv_k, b.priv_v, b.hidden,
                                               b.hidden_sums, b.status));
        }
    }
    GUFFIN_TRY(guffin_hip_commit_rows(s, &m, b.priv_k, b.priv_v, b.ring_k_table, b.ring_v_table, nullptr, at, rows));
    if (p->transaction_active   // the rows' final normalised states, by their place in the transaction
        && hipMemcpyAsync(b.txn_hidden + uint64_t(at - p->checkpoint_materialized) * m.hidden, b.hidden, uint64_t(rows) * m.hidden * 4,
                          hipMemcpyDeviceToDevice, s) != hipSuccess)
        return fail(GUFFIN_E_HIP, "draft_plan: keeping the rows' final states failed");
    p->materialized = at + rows;
    p->last_rows = rows;
    p->logits_valid = 0;
    p->hidden_valid = 1;
    return GUFFIN_OK;
}

int finish(hipStream_t s, guffin_draft_plan* p, const Buffers& b, const char* what) {
    uint32_t status = 0;
    if (hipStreamSynchronize(s) != hipSuccess || hipMemcpy(&status, b.status, 4, hipMemcpyDeviceToHost) != hipSuccess)
        return poison(p, GUFFIN_E_HIP, what);
    if (status != 0) return poison(p, GUFFIN_E_NUMERIC, what);
    return GUFFIN_OK;
}

// host tokens through the blocks one row per pass, a pending token first: a token's rows and logits then do
// not depend on how the caller grouped its appends (a two-row pass sums attention partitions and norms in
// another order than two one-row passes), which is what lets a commit be compared with a replay bit for bit
int ingest(hipStream_t s, guffin_draft_plan* p, const Buffers& b, const uint32_t* tokens, uint32_t count) {
    std::vector<uint32_t> input;
    if (p->has_pending) input.push_back(p->pending_token);
    input.insert(input.end(), tokens, tokens + count);
    for (size_t i = 0; i < input.size(); ++i) {
        if (hipMemcpyWithStream(b.tokens, input.data() + i, 4, hipMemcpyHostToDevice, s) != hipSuccess)
            return poison(p, GUFFIN_E_HIP, "draft_plan: token upload failed");
        if (int rc = forward(s, p, b, 1)) { p->poisoned = 1; return rc; }
    }
    p->has_pending = 0;
    p->position = p->materialized;
    return GUFFIN_OK;
}

// logits of the rows of the last pass (the head GEMV runs only when somebody asks)
int ensure_logits(hipStream_t s, guffin_draft_plan* p, const Buffers& b) {
    if (p->logits_valid) return GUFFIN_OK;
    if (!p->hidden_valid) return fail(GUFFIN_E_STATE, "draft_plan: no pass stands at the current frontier (append a token first)");
    const guffin_model_desc& m = *p->model;
    GUFFIN_TRY(guffin_hip_gemv_packed(s, m.head_dtype, m.head_tiles, b.hidden, b.hidden_sums, b.parts, b.logits, p->last_rows,
                                      m.hidden, m.vocab));
    p->logits_valid = 1;
    return GUFFIN_OK;
}

int capacity_check(const guffin_draft_plan* p, uint32_t new_rows, const char* what) {
    const guffin_model_desc& m = *p->model;
    if (uint64_t(p->materialized) + new_rows > m.ring_global) return fail(GUFFIN_E_CAPACITY, what);
    if (p->transaction_active && uint64_t(p->materialized) + new_rows - p->checkpoint_materialized > p->transaction_rows)
        return fail(GUFFIN_E_CAPACITY, "draft_plan: the transaction would write more rows than the plan was prepared for");
    return GUFFIN_OK;
}

}  // namespace
}  // namespace guffin

using namespace guffin;

// transaction_rows: 0 = 32; otherwise at least the largest horizon + 2 (gemma3_draft.mm:654-655) and no more than a ring holds
static bool transaction_rows_fit(const guffin_model_desc& m, uint32_t& transaction_rows) {
    if (transaction_rows == 0) transaction_rows = kDefaultTransactionRows;
    return transaction_rows >= kMaxHorizon + 2 && arena_rows(transaction_rows) <= m.ring_local && arena_rows(transaction_rows) <= m.ring_global;
}

extern "C" uint64_t guffin_hip_draft_plan_bytes(const guffin_model_desc* model, uint32_t transaction_rows) {
    if (!model || !model->layers || !model->head_tiles || model->ring_global < 4 || !transaction_rows_fit(*model, transaction_rows)) return 0;
    uint64_t total = 0;
    carve(*model, arena_rows(transaction_rows), nullptr, &total);
    return total;
}

extern "C" int guffin_hip_draft_plan_init(void* stream, guffin_draft_plan* plan, const guffin_model_desc* model, void* workspace,
                                          uint64_t workspace_bytes, uint32_t transaction_rows) {
    if (!plan || !model || !model->layers || !workspace) return fail(GUFFIN_E_ARG, "draft_plan_init: null pointer");
    if (!model->head_tiles) return fail(GUFFIN_E_ARG, "draft_plan_init: the model needs its head tiles");
    if (model->vocab % 256 != 0) return fail(GUFFIN_E_SHAPE, "draft_plan_init: the law kernels need a vocabulary that is a multiple of 256");
    if (!transaction_rows_fit(*model, transaction_rows))
        return fail(GUFFIN_E_SHAPE, "draft_plan_init: a transaction holds at least 25 rows (the largest horizon + 2) and, rounded up to a power of two, no more than the smallest ring");
    const uint64_t need = guffin_hip_draft_plan_bytes(model, transaction_rows);
    if (need == 0 || workspace_bytes < need) return fail(GUFFIN_E_CAPACITY, "draft_plan_init: workspace below guffin_hip_draft_plan_bytes");
    if (reinterpret_cast<uintptr_t>(workspace) & 255u) return fail(GUFFIN_E_ALIGN, "draft_plan_init: workspace must be 256-byte aligned");
    std::memset(plan, 0, sizeof(*plan));
    plan->model = model;
    plan->workspace = workspace;
    plan->workspace_bytes = workspace_bytes;
    plan->transaction_rows = transaction_rows;
    plan->transaction_arena = arena_rows(transaction_rows);
    const Buffers b = carve(plan);
    std::vector<void*> rk(model->layer_count), rv(model->layer_count);
    for (uint32_t l = 0; l < model->layer_count; ++l) {
        if (!model->layers[l].ring_k || !model->layers[l].ring_v) return fail(GUFFIN_E_ARG, "draft_plan_init: every layer needs its rings");
        rk[l] = model->layers[l].ring_k;
        rv[l] = model->layers[l].ring_v;
    }
    hipStream_t s = as_stream(stream);
    if (hipMemcpyAsync(b.ring_k_table, rk.data(), rk.size() * sizeof(void*), hipMemcpyHostToDevice, s) != hipSuccess
        || hipMemcpyAsync(b.ring_v_table, rv.data(), rv.size() * sizeof(void*), hipMemcpyHostToDevice, s) != hipSuccess
        || hipMemsetAsync(b.status, 0, 4, s) != hipSuccess || hipStreamSynchronize(s) != hipSuccess)
        return fail(GUFFIN_E_HIP, "draft_plan_init: upload failed");
    return GUFFIN_OK;
}

// Forgets the prefix (reset(), gemma3_draft.hpp:63): ring contents stay but no row of them is referenced.
extern "C" int guffin_hip_draft_plan_reset(void* stream, guffin_draft_plan* plan) {
    if (!plan || !plan->model || !plan->workspace) return fail(GUFFIN_E_ARG, "draft_plan_reset: null pointer");
    const Buffers b = carve(plan);
    hipStream_t s = as_stream(stream);
    if (hipMemsetAsync(b.status, 0, 4, s) != hipSuccess || hipStreamSynchronize(s) != hipSuccess)
        return fail(GUFFIN_E_HIP, "draft_plan_reset: clearing the status failed");
    const guffin_model_desc* model = plan->model;
    void* workspace = plan->workspace;
    const uint64_t bytes = plan->workspace_bytes;
    const uint32_t rows = plan->transaction_rows, arena = plan->transaction_arena;
    std::memset(plan, 0, sizeof(*plan));
    plan->model = model; plan->workspace = workspace; plan->workspace_bytes = bytes;
    plan->transaction_rows = rows; plan->transaction_arena = arena;
    return GUFFIN_OK;
}

// the output rows of the pass at the frontier, kept across a transaction so that an abort leaves the plan able to
// draft from (or read the logits of) the prefix it returns to
static int copy_frontier(hipStream_t s, const guffin_model_desc& m, const Buffers& b, bool save) {
    const size_t hidden_bytes = 2 * size_t(m.hidden) * 4, sums_bytes = guffin_hip_receipt_bytes(2, m.hidden);
    if (hipMemcpyAsync(save ? b.hidden_saved : b.hidden, save ? b.hidden : b.hidden_saved, hidden_bytes, hipMemcpyDeviceToDevice, s) != hipSuccess
        || hipMemcpyAsync(save ? b.sums_saved : b.hidden_sums, save ? b.hidden_sums : b.sums_saved, sums_bytes, hipMemcpyDeviceToDevice, s) != hipSuccess)
        return fail(GUFFIN_E_HIP, "draft_plan: copying the frontier rows failed");
    return GUFFIN_OK;
}

extern "C" int guffin_hip_draft_plan_begin_transaction(void* stream, guffin_draft_plan* plan) {
    GUFFIN_TRY(usable(plan, "draft_plan_begin_transaction: null pointer"));
    if (plan->transaction_active) return fail(GUFFIN_E_STATE, "draft_plan_begin_transaction: a transaction is already open");
    if (plan->hidden_valid) GUFFIN_TRY(copy_frontier(as_stream(stream), *plan->model, carve(plan), true));
    plan->checkpoint_hidden_valid = plan->hidden_valid;
    plan->checkpoint_last_rows = plan->last_rows;
    plan->checkpoint_position = plan->position;
    plan->checkpoint_materialized = plan->materialized;
    plan->checkpoint_pending = plan->pending_token;
    plan->checkpoint_has_pending = plan->has_pending;
    plan->backup_end = plan->materialized;
    plan->transaction_active = 1;
    return GUFFIN_OK;
}

extern "C" int guffin_hip_draft_plan_abort_transaction(void* stream, guffin_draft_plan* plan) {
    GUFFIN_TRY(usable(plan, "draft_plan_abort_transaction: null pointer"));
    // outside a transaction the reference's abort poisons the plan (gemma3_draft.mm:1305-1312): there is nothing to
    // go back to, and the caller's ledger is out of step with the plan's
    if (!plan->transaction_active) { plan->poisoned = 1; return fail(GUFFIN_E_STATE, "draft_plan_abort_transaction: no transaction is open; the plan is poisoned"); }
    const Buffers b = carve(plan);
    hipStream_t s = as_stream(stream);
    if (int rc = move_rows(s, plan, b, plan->checkpoint_materialized, plan->backup_end, false)) { plan->poisoned = 1; return rc; }
    GUFFIN_TRY(finish(s, plan, b, "draft_plan_abort_transaction: restoring the ring rows failed"));
    plan->position = plan->checkpoint_position;
    plan->materialized = plan->checkpoint_materialized;
    plan->pending_token = plan->checkpoint_pending;
    plan->has_pending = plan->checkpoint_has_pending;
    plan->transaction_active = 0;
    plan->hidden_valid = plan->logits_valid = 0;
    if (plan->checkpoint_hidden_valid) {
        if (int rc = copy_frontier(s, *plan->model, b, false)) { plan->poisoned = 1; return rc; }
        plan->hidden_valid = 1;
        plan->last_rows = plan->checkpoint_last_rows;
    }
    return GUFFIN_OK;
}

// 1 if truncate(position) would be admitted: the current position always (nothing changes), and inside a transaction
// any position down to where it began (gemma3_draft.mm:1283-1288)
extern "C" int guffin_hip_draft_plan_can_truncate(const guffin_draft_plan* plan, uint32_t position) {
    if (!plan || !plan->model || plan->poisoned || position > plan->position) return 0;
    return position == plan->position || (plan->transaction_active && position >= plan->checkpoint_position);
}

extern "C" int guffin_hip_draft_plan_truncate(void* stream, guffin_draft_plan* plan, uint32_t position) {
    GUFFIN_TRY(usable(plan, "draft_plan_truncate: null pointer"));
    if (!guffin_hip_draft_plan_can_truncate(plan, position))
        return fail(GUFFIN_E_STATE, "draft_plan_truncate: only rows written inside the open transaction can be dropped");
    if (position == plan->position) return GUFFIN_OK;
    if (position < plan->materialized) {
        const Buffers b = carve(plan);
        hipStream_t s = as_stream(stream);
        if (int rc = move_rows(s, plan, b, position, plan->backup_end, false)) { plan->poisoned = 1; return rc; }
        GUFFIN_TRY(finish(s, plan, b, "draft_plan_truncate: restoring the ring rows failed"));
        plan->backup_end = std::min(plan->backup_end, position);
        plan->materialized = position;
        plan->hidden_valid = plan->logits_valid = 0;
        // the frontier's final state: a row this transaction ran, or the one the transaction began on
        const guffin_model_desc& m = *plan->model;
        if (position > plan->checkpoint_materialized) {
            const float* kept = b.txn_hidden + uint64_t(position - 1 - plan->checkpoint_materialized) * m.hidden;
            if (hipMemcpyAsync(b.hidden, kept, uint64_t(m.hidden) * 4, hipMemcpyDeviceToDevice, s) != hipSuccess)
                return poison(plan, GUFFIN_E_HIP, "draft_plan_truncate: restoring the frontier's state failed");
            if (int rc = guffin_hip_group_sums(s, b.hidden, b.hidden_sums, 1, m.hidden)) { plan->poisoned = 1; return rc; }
            plan->last_rows = 1;
            plan->hidden_valid = 1;
        } else if (plan->checkpoint_hidden_valid) {
            if (int rc = copy_frontier(s, m, b, false)) { plan->poisoned = 1; return rc; }
            plan->last_rows = plan->checkpoint_last_rows;
            plan->hidden_valid = 1;
        }
        GUFFIN_TRY(finish(s, plan, b, "draft_plan_truncate: restoring the frontier's state failed"));
    }
    plan->has_pending = 0;    // position <= materialized now: whatever was pending lay beyond it
    plan->position = position;
    return GUFFIN_OK;
}

// Keeps the first `position` tokens and closes the transaction.  The prefix may end in the pending token.
extern "C" int guffin_hip_draft_plan_commit_prefix(void* stream, guffin_draft_plan* plan, uint32_t position) {
    GUFFIN_TRY(usable(plan, "draft_plan_commit_prefix: null pointer"));
    if (!plan->transaction_active) return fail(GUFFIN_E_STATE, "draft_plan_commit_prefix: no transaction is open");
    if (position < plan->checkpoint_position || position > plan->position)
        return fail(GUFFIN_E_ARG, "draft_plan_commit_prefix: the prefix must end inside the transaction");
    if (position < plan->position) GUFFIN_TRY(guffin_hip_draft_plan_truncate(stream, plan, position));
    plan->transaction_active = 0;
    return GUFFIN_OK;
}

extern "C" int guffin_hip_draft_plan_append(void* stream, guffin_draft_plan* plan, const uint32_t* tokens, uint32_t count) {
    GUFFIN_TRY(usable(plan, "draft_plan_append: null pointer"));
    if (count == 0) return GUFFIN_OK;
    if (!tokens) return fail(GUFFIN_E_ARG, "draft_plan_append: null pointer");
    for (uint32_t i = 0; i < count; ++i)
        if (tokens[i] >= plan->model->vocab) return fail(GUFFIN_E_ARG, "draft_plan_append: token outside the vocabulary");
    GUFFIN_TRY(capacity_check(plan, count + (plan->has_pending ? 1u : 0u), "draft_plan_append: the context is full"));
    const Buffers b = carve(plan);
    hipStream_t s = as_stream(stream);
    GUFFIN_TRY(ingest(s, plan, b, tokens, count));
    return finish(s, plan, b, "draft_plan_append: the pass raised the device status");
}

// A saved emission of this drafter put back after its prefix was replayed: known, but not run (:75-77).
extern "C" int guffin_hip_draft_plan_restore_pending_token(guffin_draft_plan* plan, uint32_t token) {
    GUFFIN_TRY(usable(plan, "draft_plan_restore_pending_token: null pointer"));
    if (plan->transaction_active) return fail(GUFFIN_E_STATE, "draft_plan_restore_pending_token: not inside a transaction");
    if (plan->has_pending) return fail(GUFFIN_E_STATE, "draft_plan_restore_pending_token: a token is already pending");
    if (plan->materialized == 0) return fail(GUFFIN_E_STATE, "draft_plan_restore_pending_token: no prefix to follow");
    if (token >= plan->model->vocab) return fail(GUFFIN_E_ARG, "draft_plan_restore_pending_token: token outside the vocabulary");
    if (uint64_t(plan->position) + 1 > plan->model->ring_global) return fail(GUFFIN_E_CAPACITY, "draft_plan_restore_pending_token: the context is full");
    plan->pending_token = token;
    plan->has_pending = 1;
    plan->position += 1;
    return GUFFIN_OK;
}

// Drafts `horizon` tokens inside the open transaction from the given 32-bit words: token i comes from the
// law of the logits after token i-1 (the last appended token for i = 0); all but the last are run through the
// blocks, the last one stays pending (propose, gemma3_draft.mm:1430-1486).  history: the sampler's window in
// chronological order (host), extended by the drafted tokens as the chain grows; used when the options carry
// a repetition penalty.
extern "C" int guffin_hip_draft_plan_propose(void* stream, guffin_draft_plan* plan, const uint32_t* words, uint32_t horizon,
                                             const void* options, const uint32_t* history, uint32_t history_count,
                                             uint32_t* drafted) {
    GUFFIN_TRY(usable(plan, "draft_plan_propose: null pointer"));
    if (!words || !options || !drafted) return fail(GUFFIN_E_ARG, "draft_plan_propose: null pointer");
    if (!plan->transaction_active) return fail(GUFFIN_E_STATE, "draft_plan_propose: proposals are drafted inside a transaction");
    if (horizon == 0 || horizon > kMaxHorizon) return fail(GUFFIN_E_CAPACITY, "draft_plan_propose: the horizon must be in [1, 23]");
    if (history_count > 64 || (history_count && !history)) return fail(GUFFIN_E_ARG, "draft_plan_propose: at most 64 history tokens");
    if (plan->materialized == 0) return fail(GUFFIN_E_STATE, "draft_plan_propose: no prefix to draft from");
    if (!plan->has_pending && !plan->hidden_valid && !plan->logits_valid)   // a state error, not a fault: nothing is poisoned
        return fail(GUFFIN_E_STATE, "draft_plan_propose: no pass stands at the current frontier (append a token first)");
    GUFFIN_TRY(capacity_check(plan, horizon - 1 + (plan->has_pending ? 1u : 0u), "draft_plan_propose: the context is full"));
    struct Options { float temperature; uint32_t top_k; float top_p, min_p, repetition_penalty; };
    Options opt;
    std::memcpy(&opt, options, sizeof(opt));
    const guffin_model_desc& m = *plan->model;
    const Buffers b = carve(plan);
    hipStream_t s = as_stream(stream);
    if (plan->has_pending) GUFFIN_TRY(ingest(s, plan, b, nullptr, 0));
    std::vector<Draws> draws(horizon);
    for (uint32_t i = 0; i < horizon; ++i) draws[i] = {words[i], 0, 0.5, 0.5, 0.5};
    if (hipMemcpyWithStream(b.draws, draws.data(), horizon * sizeof(Draws), hipMemcpyHostToDevice, s) != hipSuccess)
        return poison(plan, GUFFIN_E_HIP, "draft_plan_propose: upload failed");
    std::vector<uint32_t> window(history, history + history_count);
    const bool penalise = opt.repetition_penalty != 1.0f;
    Options law_options = opt;
    law_options.repetition_penalty = 1.0f;   // applied to the scores below, as gd_process does before the law
    for (uint32_t i = 0; i < horizon; ++i) {
        if (int rc = ensure_logits(s, plan, b)) { plan->poisoned = 1; return rc; }
        const float* logits = b.logits + uint64_t(plan->last_rows - 1) * m.vocab;
        if (penalise && !window.empty()) {
            if (hipMemcpyWithStream(b.history, window.data(), window.size() * 4, hipMemcpyHostToDevice, s) != hipSuccess)
                return poison(plan, GUFFIN_E_HIP, "draft_plan_propose: upload failed");
            if (int rc = guffin_hip_draft_process(s, logits, m.vocab, b.history, static_cast<uint32_t>(window.size()),
                                                  opt.repetition_penalty, b.scores)) { plan->poisoned = 1; return rc; }
            logits = b.scores;
        }
        if (int rc = guffin_hip_draft_law_any(s, logits, m.vocab, &law_options, 0, 0, b.draws + i, b.law_ws, b.law, b.cdf,
                                              b.tokens, b.status)) { plan->poisoned = 1; return rc; }
        GUFFIN_TRY(finish(s, plan, b, "draft_plan_propose: the law raised the device status"));
        if (hipMemcpy(&drafted[i], b.tokens, 4, hipMemcpyDeviceToHost) != hipSuccess)
            return poison(plan, GUFFIN_E_HIP, "draft_plan_propose: read-back failed");
        if (window.size() == 64) window.erase(window.begin());
        window.push_back(drafted[i]);
        if (i + 1 < horizon) {           // b.tokens[0] holds the drafted token: run it
            if (int rc = forward(s, plan, b, 1)) { plan->poisoned = 1; return rc; }
            plan->position = plan->materialized;
        }
    }
    GUFFIN_TRY(finish(s, plan, b, "draft_plan_propose: the pass raised the device status"));
    plan->pending_token = drafted[horizon - 1];
    plan->has_pending = 1;
    plan->position = plan->materialized + 1;
    return GUFFIN_OK;
}

// Logits after the last materialized token (read_logits, :94), to host memory.
extern "C" int guffin_hip_draft_plan_read_logits(void* stream, guffin_draft_plan* plan, float* logits_host) {
    GUFFIN_TRY(usable(plan, "draft_plan_read_logits: null pointer"));
    if (!logits_host) return fail(GUFFIN_E_ARG, "draft_plan_read_logits: null pointer");
    const Buffers b = carve(plan);
    hipStream_t s = as_stream(stream);
    GUFFIN_TRY(ensure_logits(s, plan, b));
    GUFFIN_TRY(finish(s, plan, b, "draft_plan_read_logits: the head raised the device status"));
    const uint64_t V = plan->model->vocab;
    if (hipMemcpy(logits_host, b.logits + uint64_t(plan->last_rows - 1) * V, V * 4, hipMemcpyDeviceToHost) != hipSuccess)
        return poison(plan, GUFFIN_E_HIP, "draft_plan_read_logits: read-back failed");
    return GUFFIN_OK;
}

// fp16 K and V rows of `count` materialized positions of one layer, in position order (read_cache, :95-98).
// Rows a local layer no longer holds (older than its ring) are refused, never made up.
extern "C" int guffin_hip_draft_plan_read_cache(void* stream, const guffin_draft_plan* plan, uint32_t layer, uint32_t first_position,
                                                uint32_t count, void* keys_host, void* values_host) {
    if (!plan || !plan->model || !keys_host || !values_host) return fail(GUFFIN_E_ARG, "draft_plan_read_cache: null pointer");
    const guffin_model_desc& m = *plan->model;
    if (layer >= m.layer_count) return fail(GUFFIN_E_ARG, "draft_plan_read_cache: no such layer");
    if (uint64_t(first_position) + count > plan->materialized) return fail(GUFFIN_E_ARG, "draft_plan_read_cache: rows beyond the materialized prefix");
    const uint32_t capacity = layer_is_local(m.global_period, layer) ? m.ring_local : m.ring_global;
    if (plan->materialized - first_position > capacity) return fail(GUFFIN_E_ARG, "draft_plan_read_cache: rows older than the layer's ring");
    if (hipStreamSynchronize(as_stream(stream)) != hipSuccess) return fail(GUFFIN_E_HIP, "draft_plan_read_cache: the stream failed");
    const uint64_t row_bytes = uint64_t(m.kv_heads) * m.head_dim * 2;
    for (uint32_t i = 0; i < count; ++i) {
        const uint64_t slot = (first_position + i) & (capacity - 1);
        if (hipMemcpy(static_cast<uint8_t*>(keys_host) + i * row_bytes, static_cast<const uint8_t*>(m.layers[layer].ring_k) + slot * row_bytes,
                      row_bytes, hipMemcpyDeviceToHost) != hipSuccess
            || hipMemcpy(static_cast<uint8_t*>(values_host) + i * row_bytes, static_cast<const uint8_t*>(m.layers[layer].ring_v) + slot * row_bytes,
                         row_bytes, hipMemcpyDeviceToHost) != hipSuccess)
            return fail(GUFFIN_E_HIP, "draft_plan_read_cache: read-back failed");
    }
    return GUFFIN_OK;
}
