// Host-side transaction of one target verify pass: encode -> submit -> complete ->
// provisional commit -> finalize, with discard and release.
//
// Mirrors TargetVerificationTicket and its free functions
//   encode_gemma2_metal_target_verifier                src/engine/target_verifier_runtime.cpp:349-445
//   submit_ / complete_                                 :447-533
//   provisionally_commit_gemma2_metal_target_verifier   :535-609
//   finalize_ / discard_                                :611-688
//   ~TargetVerificationTicket                           :315-335
// with the states of VerifierTransactionState (include/local_gguf_engine/engine/gemma2_metal_plan.hpp:
// 208-215).  The pass keeps its K/V in private rows; a provisional commit first copies the ring rows
// it is about to overwrite into the backup rows, then scatters the selected private rows into the
// rings; finalize keeps a prefix of them and restores the rest.  The rows of a pass are a chain of 1 or
// 2 rows (one launch sequence of the block graph) or a tree of up to 4 rows in topological order (row r's
// parent is any earlier row), which runs in passes of 2 rows whose attention reads the earlier rows'
// private K/V; a provisional commit takes any root-to-node path.  Nothing is allocated: every buffer is
// the caller's.
#include <cstddef>
#include "common.hpp"
#include "receipt.hpp"

#include <algorithm>

#define GUFFIN_TRY(expr) do { if (int rc_ = (expr)) return rc_; } while (0)

namespace guffin {
namespace {

constexpr uint32_t kMaxTicketRows = GUFFIN_TICKET_MAX_ROWS;
constexpr uint64_t kAlign = 256;
uint64_t aligned(uint64_t n) { return (n + kAlign - 1) & ~(kAlign - 1); }

struct Arena {
    uint64_t forward, hidden, parts, pass_receipt, logits, select, total;
    uint64_t hidden_receipt;  // floats from the hidden rows to their receipt
};

Arena arena_of(const guffin_model_desc& m, uint32_t position, uint32_t retain) {
    Arena a {};
    const uint32_t rows = kMaxTicketRows;
    uint64_t off = 0;
    // a pass has at most 2 rows; a tree pass sizes its arena at the deepest position a row can take
    a.forward = off; off += aligned(std::max({guffin_hip_forward_scratch_bytes(&m, 2, position),
                                              guffin_hip_forward_scratch_bytes(&m, 2, position + kMaxTicketRows),
                                              guffin_hip_forward_scratch_bytes(&m, 1, position + kMaxTicketRows)}));
    a.hidden_receipt = (uint64_t(rows) * m.hidden + 63) & ~uint64_t{63};
    a.hidden = off; off += aligned(a.hidden_receipt * 4 + receipt_layout(rows, m.hidden).bytes);
    const uint32_t slices = guffin_hip_gemv_packed_slices(m.head_dtype, m.hidden, m.vocab);
    a.parts = off; off += aligned(uint64_t(slices) * rows * m.vocab * 4);
    a.pass_receipt = off; off += aligned(receipt_layout(2, m.hidden).bytes);
    a.logits = off; off += aligned(uint64_t(rows) * m.vocab * 4);
    a.select = off; off += aligned(guffin_hip_select_workspace_bytes(rows, m.vocab, retain));
    a.total = off;
    return a;
}

int ticket_ready(const guffin_verify_ticket* t, const char* what) {
    if (!t || !t->target || !t->scratch || !t->priv_k || !t->priv_v || !t->backup_k || !t->backup_v || !t->tokens
        || !t->selected || !t->candidates || !t->status)
        return fail(GUFFIN_E_ARG, what);
    return GUFFIN_OK;
}

void clear_transaction(guffin_verify_ticket* t) {
    t->state = GUFFIN_TXN_IDLE;
    t->rows = 0;
    t->provisional_count = 0;
}

struct LayerRing { void* k; void* v; uint32_t mask; };
LayerRing ring_of(const guffin_model_desc& m, uint32_t layer) {
    const bool local = layer_is_local(m.global_period, layer);  // the same rule as the forward pass it commits for
    return {m.layers[layer].ring_k, m.layers[layer].ring_v, (local ? m.ring_local : m.ring_global) - 1u};
}

// restores ring rows [position + first, position + first + count) of every layer from the backup rows
int restore_rows(hipStream_t s, const guffin_verify_ticket* t, uint32_t first, uint32_t count) {
    const guffin_model_desc& m = *t->target;
    const uint32_t kvw = m.kv_heads * m.head_dim;
    for (uint32_t l = 0; l < m.layer_count; ++l) {
        const LayerRing r = ring_of(m, l);
        const uint16_t* bk = static_cast<const uint16_t*>(t->backup_k) + size_t(l) * kMaxTicketRows * kvw;
        const uint16_t* bv = static_cast<const uint16_t*>(t->backup_v) + size_t(l) * kMaxTicketRows * kvw;
        GUFFIN_TRY(guffin_hip_kv_cache_copy(s, bk, bv, r.k, r.v, t->position + first, count, kMaxTicketRows - 1u, r.mask, kvw));
    }
    return GUFFIN_OK;
}

}  // namespace
}  // namespace guffin

using namespace guffin;

extern "C" uint64_t guffin_hip_ticket_scratch_bytes(const guffin_verify_ticket* t, uint32_t last_position) {
    if (!t || !t->target || t->retain == 0) return 0;
    return arena_of(*t->target, last_position, t->retain).total;
}

namespace {
int encode(guffin_verify_ticket* t, const uint32_t* row_tokens, const uint32_t* parents, uint32_t rows, uint32_t position,
           uint32_t max_rows, const char* too_many) {
    GUFFIN_TRY(ticket_ready(t, "ticket_encode: null pointer"));
    if (!row_tokens) return fail(GUFFIN_E_ARG, "ticket_encode: null pointer");
    if (t->state == GUFFIN_TXN_POISONED) return fail(GUFFIN_E_STATE, "ticket_encode: the ticket is poisoned");
    if (t->state != GUFFIN_TXN_IDLE) return fail(GUFFIN_E_STATE, "ticket_encode: a verify pass is already pending");
    const guffin_model_desc& m = *t->target;
    if (rows == 0 || rows > max_rows) return fail(GUFFIN_E_SHAPE, too_many);
    if (!m.head_tiles || !m.layers) return fail(GUFFIN_E_ARG, "ticket_encode: the target needs its head tiles and layers");
    if (reinterpret_cast<uintptr_t>(t->scratch) & 255u) return fail(GUFFIN_E_ALIGN, "ticket_encode: the arena must be 256-byte aligned");
    // the selection keeps at most 320 candidates per row (guffin_hip_select_candidates)
    if (t->retain == 0 || t->retain > 320) return fail(GUFFIN_E_CAPACITY, "ticket_encode: retain must be 1..320 candidates per row");
    uint32_t depths[kMaxTicketRows] = {}, deepest = 0;
    for (uint32_t r = 0; r < rows; ++r) {
        const uint32_t parent = parents ? parents[r] : (r == 0 ? GUFFIN_TICKET_ROOT : r - 1);
        if ((r == 0) != (parent == GUFFIN_TICKET_ROOT) || (r > 0 && parent >= r))
            return fail(GUFFIN_E_ARG, "ticket_encode: rows come in topological order under one root");
        depths[r] = r == 0 ? 0u : depths[parent] + 1;
        deepest = std::max(deepest, depths[r]);
    }
    if (uint64_t(position) + deepest + 1 > m.ring_global) return fail(GUFFIN_E_CAPACITY, "ticket_encode: the rows do not fit the global rings");
    if (t->scratch_bytes < arena_of(m, position, t->retain).total) return fail(GUFFIN_E_CAPACITY, "ticket_encode: scratch arena too small");
    t->rows = rows;
    t->position = position;
    t->provisional_count = 0;
    for (uint32_t r = 0; r < kMaxTicketRows; ++r) {
        t->row_tokens[r] = r < rows ? row_tokens[r] : 0u;
        t->parents[r] = r < rows ? (parents ? parents[r] : (r == 0 ? GUFFIN_TICKET_ROOT : r - 1)) : 0u;
        t->depths[r] = r < rows ? depths[r] : 0u;
    }
    t->state = GUFFIN_TXN_ENCODED;
    return GUFFIN_OK;
}

bool is_chain(const guffin_verify_ticket* t) {
    for (uint32_t r = 1; r < t->rows; ++r)
        if (t->parents[r] != r - 1) return false;
    return true;
}
}  // namespace

extern "C" int guffin_hip_ticket_encode(guffin_verify_ticket* t, const uint32_t* row_tokens, uint32_t rows, uint32_t position) {
    return encode(t, row_tokens, nullptr, rows, position, 2, "ticket_encode: a pass has 1 or 2 rows");
}

extern "C" int guffin_hip_ticket_encode_tree(guffin_verify_ticket* t, const uint32_t* row_tokens, const uint32_t* parents,
                                             uint32_t rows, uint32_t position) {
    if (!parents) return fail(GUFFIN_E_ARG, "ticket_encode_tree: null pointer");
    return encode(t, row_tokens, parents, rows, position, kMaxTicketRows, "ticket_encode_tree: a tree has 1 to 4 rows");
}

extern "C" int guffin_hip_ticket_submit(void* stream, guffin_verify_ticket* t) {
    GUFFIN_TRY(ticket_ready(t, "ticket_submit: null pointer"));
    if (t->state != GUFFIN_TXN_ENCODED) return fail(GUFFIN_E_STATE, "ticket_submit: requires an encoded ticket");
    const guffin_model_desc& m = *t->target;
    const Arena a = arena_of(m, t->position, t->retain);
    uint8_t* base = static_cast<uint8_t*>(t->scratch);
    float* hidden = reinterpret_cast<float*>(base + a.hidden);
    float* hidden_sums = hidden + a.hidden_receipt;
    float* parts = reinterpret_cast<float*>(base + a.parts);
    float* logits = reinterpret_cast<float*>(base + a.logits);
    hipStream_t hs = as_stream(stream);
    static const uint32_t kZero[1 + kMaxTicketRows] = {};
    int rc = GUFFIN_OK;
    // the row tokens live in the ticket, which outlives the copy
    if (hipMemcpyAsync(t->tokens, t->row_tokens, t->rows * sizeof(uint32_t), hipMemcpyHostToDevice, hs) != hipSuccess
        || hipMemcpyAsync(t->status, kZero, sizeof(kZero), hipMemcpyHostToDevice, hs) != hipSuccess)
        rc = fail(GUFFIN_E_HIP, "ticket_submit: upload failed");
    if (t->rows <= 2 && is_chain(t)) {
        if (rc == GUFFIN_OK)
            rc = guffin_hip_forward_rows(stream, &m, t->tokens, t->rows, t->position, base + a.forward, a.hidden - a.forward, t->priv_k,
                                         t->priv_v, hidden, hidden_sums, t->status);
        if (rc == GUFFIN_OK)
            rc = guffin_hip_gemv_packed(stream, m.head_dtype, m.head_tiles, hidden, hidden_sums, parts, logits, t->rows, m.hidden, m.vocab);
    } else {
        // passes of two rows in row order; a row's ancestor list is its path from the root, itself last
        float* pass_receipt = reinterpret_cast<float*>(base + a.pass_receipt);
        for (uint32_t first = 0; rc == GUFFIN_OK && first < t->rows; first += 2) {
            const uint32_t n = std::min(2u, t->rows - first);
            uint32_t lists[2 * kMaxTicketRows], counts[2], used = 0;
            for (uint32_t r = 0; r < n; ++r) {
                uint32_t path[kMaxTicketRows], len = 0;
                for (uint32_t node = first + r; node != GUFFIN_TICKET_ROOT; node = t->parents[node]) path[len++] = node;
                for (uint32_t i = 0; i < len; ++i) lists[used + i] = path[len - 1 - i];
                counts[r] = len;
                used += len;
            }
            rc = guffin_hip_forward_tree_rows(stream, &m, t->tokens + first, n, t->position, t->depths + first, lists, counts, first,
                                              t->rows, base + a.forward, a.hidden - a.forward, t->priv_k, t->priv_v,
                                              hidden + size_t(first) * m.hidden, pass_receipt, t->status);
            if (rc == GUFFIN_OK)
                rc = guffin_hip_gemv_packed(stream, m.head_dtype, m.head_tiles, hidden + size_t(first) * m.hidden, pass_receipt, parts,
                                            logits + size_t(first) * m.vocab, n, m.hidden, m.vocab);
        }
    }
    if (rc == GUFFIN_OK)
        rc = guffin_hip_select_candidates(stream, logits, t->rows, m.vocab, t->retain, nullptr, nullptr, base + a.select,
                                          t->candidates, t->status + 1);
    if (rc != GUFFIN_OK) {
        // the rings are untouched by anything enqueued so far: the transaction is dropped (:447-463)
        clear_transaction(t);
        return rc;
    }
    t->state = GUFFIN_TXN_SUBMITTED;
    return GUFFIN_OK;
}

extern "C" int guffin_hip_ticket_complete(void* stream, guffin_verify_ticket* t, uint32_t* device_status) {
    GUFFIN_TRY(ticket_ready(t, "ticket_complete: null pointer"));
    if (t->state != GUFFIN_TXN_SUBMITTED) return fail(GUFFIN_E_STATE, "ticket_complete: requires a submitted ticket");
    uint32_t status[1 + kMaxTicketRows] = {};
    if (hipStreamSynchronize(as_stream(stream)) != hipSuccess
        || hipMemcpy(status, t->status, sizeof(status), hipMemcpyDeviceToHost) != hipSuccess) {
        t->state = GUFFIN_TXN_POISONED;  // the pass may still be running over the private rows
        return fail(GUFFIN_E_HIP, "ticket_complete: wait or read-back failed, the ticket is poisoned");
    }
    resident_note_status(status[0]);
    uint32_t raised = status[0];
    for (uint32_t r = 0; r < t->rows; ++r) raised |= status[1 + r];
    if (device_status) *device_status = raised;
    if (raised != 0) {
        // the pass wrote private rows only: the transaction is dropped, the caches are as before (:483-509)
        clear_transaction(t);
        return fail(GUFFIN_E_NUMERIC, (raised & GUFFIN_STATUS_KV_NONFINITE)
                                          ? "ticket_complete: F16 KV storage produced nonfinite values"
                                          : "ticket_complete: the verify pass rejected malformed device input");
    }
    t->state = GUFFIN_TXN_COMPLETED;
    return GUFFIN_OK;
}

extern "C" int guffin_hip_ticket_provisional_commit(void* stream, guffin_verify_ticket* t, const uint32_t* path, uint32_t count) {
    GUFFIN_TRY(ticket_ready(t, "ticket_provisional_commit: null pointer"));
    if (t->state != GUFFIN_TXN_COMPLETED) return fail(GUFFIN_E_STATE, "ticket_provisional_commit: requires completion");
    if (!path || count == 0 || count > t->rows) return fail(GUFFIN_E_ARG, "ticket_provisional_commit: selected path extent is invalid");
    for (uint32_t i = 0; i < count; ++i) {
        // row 0 is the root of the pass; every further node is a child of the one before it
        if (path[i] >= t->rows || (i == 0 && path[i] != 0) || (i > 0 && t->parents[path[i]] != path[i - 1]))
            return fail(GUFFIN_E_ARG, "ticket_provisional_commit: selected nodes are not one causal path");
    }
    const guffin_model_desc& m = *t->target;
    const uint32_t kvw = m.kv_heads * m.head_dim;
    hipStream_t hs = as_stream(stream);
    for (uint32_t i = 0; i < kMaxTicketRows; ++i) t->provisional_path[i] = i < count ? path[i] : 0u;
    int rc = GUFFIN_OK;
    if (hipMemcpyAsync(t->selected, t->provisional_path, count * sizeof(uint32_t), hipMemcpyHostToDevice, hs) != hipSuccess)
        rc = fail(GUFFIN_E_HIP, "ticket_provisional_commit: upload failed");
    // backups read the durable rows of every layer before any selected private row is published
    for (uint32_t l = 0; rc == GUFFIN_OK && l < m.layer_count; ++l) {
        const LayerRing r = ring_of(m, l);
        uint16_t* bk = static_cast<uint16_t*>(t->backup_k) + size_t(l) * kMaxTicketRows * kvw;
        uint16_t* bv = static_cast<uint16_t*>(t->backup_v) + size_t(l) * kMaxTicketRows * kvw;
        rc = guffin_hip_kv_cache_copy(stream, r.k, r.v, bk, bv, t->position, count, r.mask, kMaxTicketRows - 1u, kvw);
    }
    const bool rings_touched = rc == GUFFIN_OK;
    for (uint32_t l = 0; rc == GUFFIN_OK && l < m.layer_count; ++l) {
        const LayerRing r = ring_of(m, l);
        const uint16_t* pk = static_cast<const uint16_t*>(t->priv_k) + size_t(l) * t->rows * kvw;
        const uint16_t* pv = static_cast<const uint16_t*>(t->priv_v) + size_t(l) * t->rows * kvw;
        rc = guffin_hip_kv_scatter(stream, pk, pv, t->selected, r.k, r.v, t->position, count, kvw, r.mask);
    }
    if (rc == GUFFIN_OK && hipStreamSynchronize(hs) != hipSuccess) rc = fail(GUFFIN_E_HIP, "ticket_provisional_commit: wait failed");
    if (rc != GUFFIN_OK) {
        // some rings may hold the pass's rows and some not (:586-590); before the first scatter
        // nothing durable has changed and the ticket stays completed
        if (rings_touched) t->state = GUFFIN_TXN_POISONED;
        return rc;
    }
    t->provisional_count = count;
    t->state = GUFFIN_TXN_PROVISIONAL;
    return GUFFIN_OK;
}

extern "C" int guffin_hip_ticket_finalize(void* stream, guffin_verify_ticket* t, uint32_t retained) {
    GUFFIN_TRY(ticket_ready(t, "ticket_finalize: null pointer"));
    if (t->state != GUFFIN_TXN_PROVISIONAL) return fail(GUFFIN_E_STATE, "ticket_finalize: requires a provisional commit");
    if (retained > t->provisional_count) return fail(GUFFIN_E_ARG, "ticket_finalize: cannot retain an uncommitted row");
    if (retained < t->provisional_count) {
        int rc = restore_rows(as_stream(stream), t, retained, t->provisional_count - retained);
        if (rc == GUFFIN_OK && hipStreamSynchronize(as_stream(stream)) != hipSuccess) rc = fail(GUFFIN_E_HIP, "ticket_finalize: wait failed");
        if (rc != GUFFIN_OK) {
            t->state = GUFFIN_TXN_POISONED;  // a rejected suffix may still be in the rings
            return rc;
        }
    }
    clear_transaction(t);
    return GUFFIN_OK;
}

extern "C" int guffin_hip_ticket_discard(void* stream, guffin_verify_ticket* t) {
    if (!t) return fail(GUFFIN_E_ARG, "ticket_discard: null pointer");
    if (t->state == GUFFIN_TXN_IDLE) return GUFFIN_OK;
    if (t->state == GUFFIN_TXN_PROVISIONAL) return guffin_hip_ticket_finalize(stream, t, 0);
    if (t->state == GUFFIN_TXN_ENCODED || t->state == GUFFIN_TXN_COMPLETED) {
        clear_transaction(t);
        return GUFFIN_OK;
    }
    return fail(GUFFIN_E_STATE, "ticket_discard: a submitted or poisoned verify pass cannot be discarded safely");
}

extern "C" int guffin_hip_ticket_release(void* stream, guffin_verify_ticket* t) {
    if (!t) return fail(GUFFIN_E_ARG, "ticket_release: null pointer");
    if (t->state == GUFFIN_TXN_IDLE || t->state == GUFFIN_TXN_POISONED) return GUFFIN_OK;
    if (t->state == GUFFIN_TXN_ENCODED || t->state == GUFFIN_TXN_COMPLETED) {
        clear_transaction(t);
        return GUFFIN_OK;
    }
    if (t->state == GUFFIN_TXN_PROVISIONAL) {
        if (guffin_hip_ticket_finalize(stream, t, 0) != GUFFIN_OK) t->state = GUFFIN_TXN_POISONED;
        return GUFFIN_OK;
    }
    t->state = GUFFIN_TXN_POISONED;  // submitted: work on the private rows is still in flight
    return GUFFIN_OK;
}
