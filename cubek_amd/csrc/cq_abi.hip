// C ABI of the library: argument validation, path selection, launches.
// Mirrors the host side of the reference's launch functions
// (crates/cubek-quant/src/quantize.rs:174-326, src/dequantize.rs:171-332):
// the reference's panics become status codes, its JIT launch becomes a
// precompiled gfx950 kernel launch on the caller's stream.
#include <hip/hip_runtime.h>

#include <atomic>
#include <cstring>
#include <utility>

#include "../../include/cubek_quant.h"
#include "cq_internal.hpp"

namespace {

thread_local int g_last_hip_error = 0;

// cq_plan_kind() runs an entry point's planning with launches switched off and notes which kernel family
// each launch would have used: the family that moves the value tensors, or, for calls that only produce
// scales, the family that reads the floats.
struct PlanProbe {
    bool on = false;
    uint32_t main = CQ_FAMILY_NONE, aux = CQ_FAMILY_NONE;
};
thread_local PlanProbe g_probe;
// true: probing, the launch is to be skipped
bool probing(uint32_t family, bool aux) {
    if (!g_probe.on) return false;
    uint32_t& slot = aux ? g_probe.aux : g_probe.main;
    if (slot == CQ_FAMILY_NONE) slot = family;
    return true;
}
#define CQ_RUN(family, call) (probing(family, false) ? CQ_OK : hip_status(call))
#define CQ_RUN_AUX(family, call) (probing(family, true) ? CQ_OK : hip_status(call))

void drop_stale_hip_error() {
    if (!g_probe.on) (void)hipGetLastError();
}

cq_status hip_status(hipError_t e) {
    if (e == hipSuccess) return CQ_OK;
    g_last_hip_error = static_cast<int>(e);
    return CQ_ERR_HIP;
}

// The launchers read hipGetLastError() after each launch.  An error left on the calling thread by earlier
// HIP calls of the caller would be taken for a failed launch, so every entry point that launches kernels
// clears it first (as any hipGetLastError() does).
void drop_stale_hip_error();

uint32_t dtype_size(int dtype) { return dtype == CQ_F32 ? 4u : 2u; }
bool valid_dtype(int dtype) { return dtype == CQ_F32 || dtype == CQ_F16 || dtype == CQ_BF16; }
int param_to_dtype(uint8_t p) { return p == CQ_PARAM_F32 ? CQ_F32 : (p == CQ_PARAM_F16 ? CQ_F16 : CQ_BF16); }

uint32_t value_bits(uint8_t v) {
    switch (v) {
        case CQ_VALUE_Q8F: case CQ_VALUE_Q8S: case CQ_VALUE_E4M3: case CQ_VALUE_E5M2: return 8;
        case CQ_VALUE_Q4F: case CQ_VALUE_Q4S: case CQ_VALUE_E2M1: case CQ_VALUE_E2M1_OCP: return 4;
        case CQ_VALUE_Q2F: case CQ_VALUE_Q2S: return 2;
        default: return 0;
    }
}

cq_status check_scheme(const cq_scheme* s) {
    if (!s) return CQ_ERR_INVALID_ARGUMENT;
    if (value_bits(s->value) == 0 || s->param > CQ_PARAM_BF16 || s->store > CQ_STORE_NATIVE ||
        s->level > CQ_LEVEL_BLOCK || s->reserved != 0)
        return CQ_ERR_INVALID_ARGUMENT;
    if (s->mode != CQ_MODE_SYMMETRIC) return CQ_ERR_UNSUPPORTED_SCHEME;
    if (s->level == CQ_LEVEL_BLOCK) {
        if (s->block_rank < 1 || s->block_rank > CQ_MAX_BLOCK_DIMS) return CQ_ERR_INVALID_ARGUMENT;
        for (uint32_t i = 0; i < s->block_rank; i++)
            if (s->block[i] == 0) return CQ_ERR_INVALID_ARGUMENT;
    }
    if (s->store == CQ_STORE_NATIVE) {
        // the native arm of launch_ref accepts only these values (src/quantize.rs:192-219)
        switch (s->value) {
            case CQ_VALUE_Q8F: case CQ_VALUE_Q8S: case CQ_VALUE_E4M3: case CQ_VALUE_E5M2:
            case CQ_VALUE_E2M1: case CQ_VALUE_E2M1_OCP: break;
            default: return CQ_ERR_UNSUPPORTED_SCHEME;
        }
    }
    return CQ_OK;
}

bool tensor_ok(const cq_tensor* t) {
    return t && t->ptr && t->shape && t->strides && t->rank >= 1 && t->rank <= CQ_MAX_RANK;
}

uint64_t numel(const cq_tensor* t) {
    uint64_t n = 1;
    for (uint32_t i = 0; i < t->rank; i++) n *= t->shape[i];
    return n;
}

bool is_contiguous(const cq_tensor* t) {
    uint64_t expect = 1;
    for (int d = static_cast<int>(t->rank) - 1; d >= 0; d--) {
        if (t->shape[d] != 1 && t->strides[d] != expect) return false;
        expect *= t->shape[d];
    }
    return true;
}

bool aligned(const void* p, uintptr_t a) { return (reinterpret_cast<uintptr_t>(p) & (a - 1)) == 0; }

// Everything the launches need to know about one (values, scales) pair.
struct Plan {
    uint32_t rank;
    uint64_t shape[CQ_MAX_RANK];  // unpacked shape
    uint64_t n;                   // elements
    uint32_t bits, nq;            // bits per value; values per stored element
    cq::Range range;
    cq::Layout layout;
    cq::ValueStrides vs;    // vs.on: a value tensor is not contiguous row-major
    bool tensor_level;
    bool last_dim_blocks;   // block extents are 1 everywhere but the last dimension
    uint32_t block_last;
    uint64_t num_blocks;
    bool block_splits_words;  // U32 store: the last block extent is not a multiple of the values per word
};

uint32_t stored_nq(const cq_scheme* s) {
    if (s->store == CQ_STORE_U32) return 32u / value_bits(s->value);
    return (s->value == CQ_VALUE_E2M1 || s->value == CQ_VALUE_E2M1_OCP) ? 2u : 1u;
}

// Line size the reference would pick for the native quantize kernel (src/quantize.rs:234-240,
// cubecl's tensor_line_size_parallel over the line sizes of at most 16 bytes): 1 when the last
// dimension is not contiguous, else the widest power of two up to 16 bytes / elem_size that divides
// the last dimension and the smallest stride above 1.  Only used for its block-size assertion.
uint32_t native_line_size(const cq_tensor* t) {
    const uint32_t last = t->rank - 1;
    if (t->strides[last] != 1) return 1;
    uint64_t next_stride = 0;
    for (uint32_t d = 0; d < t->rank; d++)
        if (t->strides[d] > 1 && (next_stride == 0 || t->strides[d] < next_stride)) next_stride = t->strides[d];
    uint32_t l = 16u / t->elem_size;
    while (l > 1 && (t->shape[last] % l || next_stride % l)) l /= 2;
    return l;
}

// `values` is the stored tensor, `floats` the float tensor (input of quantize,
// output of dequantize); they must agree in shape and may have any strides.
// `quantizing`: the call is one the reference guards with check_block_size_compat (its quantize launchers
// only: src/quantize.rs:260,305; dequantize_packed and dequantize_native do not call it).
cq_status make_plan(const cq_scheme* s, const cq_tensor* floats, int dtype, const cq_tensor* values,
                    const cq_tensor* scale_a, uint32_t scale_a_size, const cq_tensor* scale_b,
                    uint32_t scale_b_size, bool quantizing, Plan* p) {
    if (!tensor_ok(floats) || !tensor_ok(values) || !tensor_ok(scale_a) || (scale_b && !tensor_ok(scale_b)))
        return CQ_ERR_INVALID_ARGUMENT;
    if (!valid_dtype(dtype)) return CQ_ERR_INVALID_ARGUMENT;
    p->bits = value_bits(s->value);
    p->nq = stored_nq(s);
    if (cq_value_range(s->value, &p->range.lo, &p->range.hi) != CQ_OK) return CQ_ERR_INVALID_ARGUMENT;
    p->range.unrounded = s->value == CQ_VALUE_E2M1_OCP ? 1u : 0u;
    if (floats->elem_size != dtype_size(dtype)) return CQ_ERR_SHAPE_MISMATCH;
    if (values->elem_size != (s->store == CQ_STORE_U32 ? 4u : 1u)) return CQ_ERR_SHAPE_MISMATCH;
    if (scale_a->elem_size != scale_a_size || (scale_b && scale_b->elem_size != scale_b_size))
        return CQ_ERR_SHAPE_MISMATCH;
    if (floats->rank != values->rank) return CQ_ERR_SHAPE_MISMATCH;
    p->rank = floats->rank;
    for (uint32_t d = 0; d < p->rank; d++) {
        p->shape[d] = floats->shape[d];
        uint64_t want = d + 1 == p->rank ? values->shape[d] * p->nq : values->shape[d];
        if (floats->shape[d] != want) return CQ_ERR_SHAPE_MISMATCH;
        if (floats->shape[d] > 0xffffffffull) return CQ_ERR_TOO_LARGE;
    }
    p->n = 1;
    for (uint32_t d = 0; d < p->rank; d++)
        if (p->shape[d] == 0) p->n = 0;
    for (uint32_t d = 0; d < p->rank && p->n != 0; d++) {
        if (p->n > (1ull << 48) / p->shape[d]) return CQ_ERR_TOO_LARGE;  // far beyond any HBM; keeps products in 64 bits
        p->n *= p->shape[d];
    }
    if (p->n == 0) return CQ_OK;  // an empty tensor: the callers launch nothing
    std::memset(&p->vs, 0, sizeof(p->vs));
    p->vs.on = !is_contiguous(floats) || !is_contiguous(values);
    p->vs.rank = p->rank;
    for (uint32_t d = 0; d < p->rank; d++) {
        p->vs.shape[d] = static_cast<uint32_t>(p->shape[d]);
        p->vs.floats[d] = floats->strides[d];
        p->vs.stored[d] = values->strides[d];
    }

    std::memset(&p->layout, 0, sizeof(p->layout));
    p->tensor_level = s->level == CQ_LEVEL_TENSOR;
    p->last_dim_blocks = false;
    p->block_last = 0;
    p->num_blocks = 1;
    p->block_splits_words = false;
    if (p->tensor_level) {
        if (numel(scale_a) < 1 || (scale_b && numel(scale_b) < 1)) return CQ_ERR_SHAPE_MISMATCH;
        return CQ_OK;
    }
    if (s->block_rank > p->rank) return CQ_ERR_SHAPE_MISMATCH;
    // check_block_size_compat (src/lib.rs:20-33): the last block extent must be a multiple of num_quants
    // (packed) or of the line size (native), asserted where the reference quantizes.  Its dequantize
    // launchers accept any block: the packed kernel then gives a whole word the scale of the word's first
    // element (src/dequantize.rs:70-76), which the per-element kernel here reproduces; the native kernel gives
    // every element the scale of its own block (the reference: of its line's first element, with a line
    // size that differs between its runtimes; the two agree whenever the block is a multiple of the line).
    uint32_t last_block = s->block[s->block_rank - 1];
    p->block_splits_words = s->store == CQ_STORE_U32 && last_block % p->nq != 0;
    if (quantizing && last_block % (s->store == CQ_STORE_U32 ? p->nq : native_line_size(floats)) != 0)
        return CQ_ERR_BLOCK_NOT_DIVISIBLE;
    if (scale_a->rank != p->rank || (scale_b && scale_b->rank != p->rank)) return CQ_ERR_SHAPE_MISMATCH;
    p->layout.rank = p->rank;
    p->last_dim_blocks = true;
    uint32_t pad = p->rank - s->block_rank;
    for (uint32_t d = 0; d < p->rank; d++) {
        uint32_t b = d < pad ? 1u : s->block[d - pad];
        if (p->shape[d] % b) return CQ_ERR_SHAPE_MISMATCH;
        uint64_t nb = p->shape[d] / b;
        if (scale_a->shape[d] != nb || (scale_b && scale_b->shape[d] != nb)) return CQ_ERR_SHAPE_MISMATCH;
        p->layout.shape[d] = static_cast<uint32_t>(p->shape[d]);
        p->layout.block[d] = b;
        p->layout.stride_a[d] = scale_a->strides[d];
        p->layout.stride_b[d] = scale_b ? scale_b->strides[d] : scale_a->strides[d];
        p->num_blocks *= nb;
        if (d + 1 < p->rank && b != 1) p->last_dim_blocks = false;
    }
    p->block_last = last_block;
    return CQ_OK;
}

// Can the flat kernels take this launch?  (contiguous scales, 1-D blocks along
// the last axis that map onto lane groups, 16-byte aligned float tensor)
// `reads_scales`: the launch reads its scales (given, stored, dequantize): blocks of any whole number of chunks;
// a fused abs-max takes a power of two of them
bool flat_ok(const Plan& p, int dtype, const cq_tensor* floats, const cq_tensor* values,
             const cq_tensor* scale_a, const cq_tensor* scale_b, bool reads_scales) {
    if (p.vs.on || !aligned(floats->ptr, 16) || !aligned(values->ptr, 8)) return false;
    if (p.tensor_level) return true;
    if (!p.last_dim_blocks) return false;
    if (!is_contiguous(scale_a) || (scale_b && !is_contiguous(scale_b))) return false;
    return reads_scales ? cq::flat_block_supported_with_scales(dtype, p.block_last) : cq::flat_block_supported(dtype, p.block_last);
}

// Rows of a tensor as the flat kernels take them: the last dimension contiguous, the rows in front of
// it as groups of `inner_rows` rows, `inner` elements between the rows of a group and `outer` between
// groups (pitched rows; a slice along the second to last dimension, a batch of pitched matrices).
// levels = 0 (a single row), 1 (one uniform run: inner_rows = all rows) or 2.
struct RowLevels {
    int levels;
    uint64_t rows, inner_rows, inner, outer;
};
bool row_levels(const cq_tensor* t, RowLevels* l) {
    const uint32_t last = t->rank - 1;
    if (t->shape[last] != 1 && t->strides[last] != 1) return false;
    *l = RowLevels{0, 1, 1, 0, 0};
    uint64_t expect = 0;
    for (int d = static_cast<int>(last) - 1; d >= 0; d--) {
        if (t->shape[d] == 1) continue;
        if (t->strides[d] == 0) return false;  // broadcast rows: not for these kernels
        if (l->levels == 0) {
            l->levels = 1;
            l->inner = t->strides[d];
        } else if (t->strides[d] != expect) {
            if (l->levels == 2) return false;
            l->levels = 2;
            l->inner_rows = l->rows;
            l->outer = t->strides[d];
        }
        expect = t->strides[d] * t->shape[d];
        l->rows *= t->shape[d];
    }
    if (l->levels < 2) l->inner_rows = l->rows;
    return true;
}

bool scales_rows_ok(const Plan& p);

// Can the flat kernels take this launch over the steps of its rows?  (value tensors with a contiguous last
// dimension whose rows form one uniform run or groups with a pitch of their own, rows of at least a step
// of 256 whole chunks, 1-D blocks that map onto lane groups (given scales: also blocks of rows), scales
// with a contiguous last dimension.)  Fills the row fields of `a` and a.num_chunks = chunks per row.
bool flat_rows_ok(const Plan& p, const cq_scheme* s, int dtype, const cq_tensor* floats, const cq_tensor* values,
                  const cq_tensor* scale_a, uint32_t scale_a_size, const cq_tensor* scale_b, uint32_t scale_b_size,
                  bool given_scales, cq::FlatArgs* a) {
    if (p.rank < 2) return false;
    const uint32_t last = p.rank - 1;
    const uint32_t elem = dtype_size(dtype), per_chunk = 16u / elem;
    const uint32_t stored = s->store == CQ_STORE_U32 ? 4u : 1u;
    RowLevels lf, lv, la{}, lb{};
    if (!row_levels(floats, &lf) || !row_levels(values, &lv) || lf.rows != lv.rows) return false;
    const uint64_t rows_f = lf.rows;
    const uint64_t cols = p.shape[last];
    // whole chunks and whole 32-bit words of codes (lanes that share a word store it together)
    const uint64_t chunk_elems = per_chunk > 32u / p.bits ? per_chunk : 32u / p.bits;
    if (cols == 0 || cols % chunk_elems) return false;
    const uint64_t row_chunks = cols / per_chunk;
    // steps of 256 chunks, a row's last one with idle lanes where 256 does not divide the row.  Measured on
    // pitched bf16 rows against the row kernels: ahead or level down to rows of 320 chunks (idle lanes 60 % of
    // the row: quantize 21 against 29 us, dequantize 21.5 against 21.7 us); shorter ragged rows stay there.
    if (row_chunks < 256) return false;
    const uint64_t row_steps = (row_chunks + 255) / 256;
    if ((row_steps * 256 - row_chunks) * 10 > row_chunks * 6) return false;
    if (rows_f * row_steps >= (1ull << 31)) return false;
    a->scale_rows = 1;
    if (!p.tensor_level) {
        // blocks along the last dimension, or (where the scales are given) over the last two: a block of
        // br rows is br rows of the launch that read the same row of scales
        const uint32_t br = p.layout.block[last - 1];
        if (!cq::flat_block_supported(dtype, p.block_last) || !scales_rows_ok(p) || (br != 1 && !given_scales)) return false;
        if (!row_levels(scale_a, &la) || la.rows * br != rows_f) return false;
        if (scale_b && (!row_levels(scale_b, &lb) || lb.rows * br != rows_f)) return false;
        a->scale_rows = br;
    }
    // one split into groups of rows must serve all tensors; uniform ones fit any
    uint64_t inner_rows = 0;
    for (const RowLevels* l : {&lf, &lv, &la, &lb}) {
        if (l->levels != 2) continue;
        if (inner_rows != 0 && inner_rows != l->inner_rows) return false;
        inner_rows = l->inner_rows;
    }
    if (inner_rows == 0) inner_rows = rows_f;
    if (inner_rows != rows_f && a->scale_rows != 1) return false;  // blocks of rows: uniform rows only
    const auto outer_of = [&](const RowLevels& l) { return l.levels == 2 ? l.outer : l.inner * inner_rows; };
    if (!aligned(floats->ptr, 16) || !aligned(values->ptr, 8) || (lf.inner * elem) % 16 || (outer_of(lf) * elem) % 16 ||
        (lv.inner * stored) % 8 || (outer_of(lv) * stored) % 8)
        return false;
    a->rows = rows_f;
    a->inner_rows = inner_rows;
    a->num_chunks = row_chunks;
    a->in_pitch = lf.inner * elem;  // quantize: floats in, stored out; dequantize swaps them
    a->in_outer = outer_of(lf) * elem;
    a->out_pitch = lv.inner * stored;
    a->out_outer = outer_of(lv) * stored;
    a->scale_in_pitch = la.inner * scale_a_size;
    a->scale_in_outer = outer_of(la) * scale_a_size;
    a->scale_out_pitch = lb.inner * scale_b_size;
    a->scale_out_outer = outer_of(lb) * scale_b_size;
    return true;
}

// Can the flat kernels take this launch with every lane finding its own row?  (Every tensor with a
// contiguous last dimension, rows of whole chunks, aligned strides, one scale per tensor or 1-D blocks that
// map onto lane groups.)  Fills a.rows, a.num_chunks = chunks per row and a.lanes: the leading dimensions
// innermost first, neighbours merged where all four tensors step uniformly through them.
bool lane_rows_ok(const Plan& p, const cq_scheme* s, int dtype, const cq_tensor* floats, const cq_tensor* values,
                  const cq_tensor* scale_a, uint32_t scale_a_size, const cq_tensor* scale_b, uint32_t scale_b_size,
                  bool given_scales, cq::FlatArgs* a) {
    if (p.rank < 2) return false;
    const uint32_t last = p.rank - 1;
    const uint32_t elem = dtype_size(dtype), per_chunk = 16u / elem;
    const uint32_t stored = s->store == CQ_STORE_U32 ? 4u : 1u;
    const auto rows_contiguous = [&](const cq_tensor* t) { return t->shape[last] == 1 || t->strides[last] == 1; };
    // 16-byte accesses to the floats at any multiple of their element size (rows that start on odd multiples of
    // 2 bytes included), 8-byte stores of codes at any multiple of 4 bytes: global memory takes unaligned accesses,
    // at some cost in cache lines crossed, and whole-chunk alignment is what the other flat launches are for
    if (!rows_contiguous(floats) || !aligned(floats->ptr, elem)) return false;
    if (values && (!rows_contiguous(values) || !aligned(values->ptr, 4))) return false;  // NULL: scales only
    const uint64_t cols = p.shape[last];
    // whole chunks and whole 32-bit words of codes (lanes that share a word store it together)
    const uint64_t chunk_elems = per_chunk > 32u / p.bits ? per_chunk : 32u / p.bits;
    if (cols == 0 || cols % chunk_elems) return false;
    const bool scales = !p.tensor_level;
    // blocks along the last dimension, or (where the scales are given) over the last two: the rows of a block
    // read the same row of scales
    const uint32_t br = scales ? p.layout.block[last - 1] : 1;
    if (scales && (!(p.last_dim_blocks || (given_scales && scales_rows_ok(p))) ||
                   !(given_scales ? cq::flat_block_supported_with_scales(dtype, p.block_last) : cq::flat_block_supported(dtype, p.block_last)) ||
                   !rows_contiguous(scale_a) || (scale_b && !rows_contiguous(scale_b))))
        return false;
    a->scale_rows = br;
    cq::LaneLevels& l = a->lanes;
    l = cq::LaneLevels{};
    uint64_t rows = 1;
    for (int d = static_cast<int>(last) - 1; d >= 0; d--) {
        const uint64_t n = p.shape[d];
        if (n == 1) continue;
        const uint64_t in = floats->strides[d] * elem, out = values ? values->strides[d] * stored : in;
        const uint64_t scale_in = scales ? scale_a->strides[d] * scale_a_size : 0;
        const uint64_t scale_out = scales && scale_b ? scale_b->strides[d] * scale_b_size : 0;
        if (in == 0 || out == 0 || out % 4) return false;  // broadcast rows, or codes off their words
        const uint32_t k = l.levels;
        // entries of the level inside this one as the scales count them: blocks of rows at the innermost level
        const uint64_t scale_count = k == 1 && br > 1 ? l.count[0] / br : (k > 0 ? l.count[k - 1] : 0);
        if (k > 0 && in == l.in[k - 1] * l.count[k - 1] && out == l.out[k - 1] * l.count[k - 1] &&
            scale_in == l.scale_in[k - 1] * scale_count && scale_out == l.scale_out[k - 1] * scale_count &&
            l.count[k - 1] * n < (1ull << 31)) {
            l.count[k - 1] *= static_cast<uint32_t>(n);
        } else {
            if (k == static_cast<uint32_t>(cq::kMaxLaneLevels)) return false;  // too many levels: the row kernels' layout
            l.count[k] = static_cast<uint32_t>(n);
            l.in[k] = in;
            l.out[k] = out;
            l.scale_in[k] = scale_in;
            l.scale_out[k] = scale_out;
            l.levels = k + 1;
        }
        rows *= n;
    }
    if (l.levels == 0) {  // a single row
        l.levels = 1;
        l.count[0] = 1;
    }
    const uint64_t row_chunks = cols / per_chunk;
    if (rows * row_chunks >= (1ull << 31)) return false;
    a->rows = rows;
    a->num_chunks = row_chunks;
    return true;
}

// The float tensor is the output (dequantize): the planners fill `in` with it.
void swap_value_roles(cq::FlatArgs* a) {
    std::swap(a->in_pitch, a->out_pitch);
    std::swap(a->in_outer, a->out_outer);
    for (uint32_t l = 0; l < a->lanes.levels; l++) std::swap(a->lanes.in[l], a->lanes.out[l]);
}
// The only scale tensor of the call is an output (fused abs-max): the planners fill `scale_in` with it.
void scale_in_to_out(cq::FlatArgs* a) {
    a->scale_out_pitch = a->scale_in_pitch;
    a->scale_out_outer = a->scale_in_outer;
    a->scale_in_pitch = a->scale_in_outer = 0;
    for (uint32_t l = 0; l < a->lanes.levels; l++) {
        a->lanes.scale_out[l] = a->lanes.scale_in[l];
        a->lanes.scale_in[l] = 0;
    }
}

// E4M3 / E5M2 in the U32 store: the reference sends every U32 scheme to quantize_packed (src/quantize.rs:185-191),
// which packs the rounded integer (up to +-448 / +-57344) into an 8-bit field with `i32 & mask` (src/quantize.rs:75),
// so most codes wrap.  The flat launches take them lane by lane (the one geometry compiled with wrapping fields);
// the row, block, tile and transposed kernels do not, and such layouts run per element.
bool wraps_its_field(const cq_scheme* s) {
    return s->store == CQ_STORE_U32 && (s->value == CQ_VALUE_E4M3 || s->value == CQ_VALUE_E5M2);
}

// Stored encoding of the flat kernels (cq::Encoding) and the field width they see.
int flat_encoding(const cq_scheme* s) {
    // the extension value holds e2m1 nibbles in both stores; eight of them in a word lie as the native store's bytes do
    if (s->value == CQ_VALUE_E2M1_OCP) return 3;
    if (s->store == CQ_STORE_U32) return 0;
    switch (s->value) {
        case CQ_VALUE_E4M3: return 1;
        case CQ_VALUE_E5M2: return 2;
        case CQ_VALUE_E2M1: return 3;
        default: return 0;  // native i8: the bytes of 8-bit two's-complement fields
    }
}

// Row kernels: last dimension contiguous on both sides and everything a multiple of a
// unit (see cq_kernels_rows.hip).  `values` may be NULL when only the float tensor
// takes part (scale production).  Fills `r` except the data pointers and dtypes.
bool rows_args(const Plan& p, const cq_scheme* s, int dtype, const cq_tensor* floats, const cq_tensor* values,
               cq::RowArgs* r) {
    const uint32_t last = p.rank - 1;
    const uint32_t per_chunk = 16u / dtype_size(dtype);
    const uint32_t unit = values ? cq::rows_unit_values(dtype, static_cast<int>(p.bits)) : per_chunk;
    const uint64_t cols = p.shape[last];
    if (cols == 0 || cols % unit || cols > (1ull << 26)) return false;
    if (!p.tensor_level && p.layout.block[last] % unit) return false;
    if (floats->strides[last] != 1 || !aligned(floats->ptr, 16)) return false;
    const bool native = s->store == CQ_STORE_NATIVE;
    if (values && (values->strides[last] != 1 || !aligned(values->ptr, 4))) return false;
    std::memset(r, 0, sizeof(*r));
    r->rank = p.rank;
    r->tensor_level = p.tensor_level ? 1u : 0u;
    r->rows = 1;
    for (uint32_t d = 0; d < p.rank; d++) {
        r->shape[d] = static_cast<uint32_t>(p.shape[d]);
        r->block[d] = p.tensor_level ? 1u : p.layout.block[d];
        r->sa[d] = p.layout.stride_a[d];
        r->sb[d] = p.layout.stride_b[d];
        if (d == last) continue;
        r->rows *= p.shape[d];
        if (p.shape[d] == 1) continue;  // its stride never contributes
        if (floats->strides[d] % per_chunk) return false;
        r->fstride[d] = floats->strides[d];
        if (values) {
            if (native && values->strides[d] % 4) return false;
            r->vstride[d] = native ? values->strides[d] / 4 : values->strides[d];
        }
    }
    if (r->rows >= (1ull << 31)) return false;
    r->fstride[last] = 1;
    r->vstride[last] = 1;
    const uint32_t bc = r->block[last];
    r->bc_shift = -1;
    if ((bc & (bc - 1)) == 0)
        for (int k = 0; k < 9; k++)
            if ((1u << k) == bc) r->bc_shift = k;
    r->param_dtype = param_to_dtype(s->param);
    r->encoding = flat_encoding(s);
    r->range = p.range;
    return true;
}

// Transposed float tensor (stride 1 on the second to last dimension), stored tensor with a
// contiguous last dimension, blocks along the last dimension only (see cq_kernels_transposed.hip).
// Fills `t` except the data pointers and scale_in_dtype; `values` may be NULL for a launch that only
// reads the floats (scale production).
bool transposed_args(const Plan& p, const cq_scheme* s, int dtype, const cq_tensor* floats, const cq_tensor* values,
                     cq::TransposedArgs* t) {
    if (p.rank < 2) return false;
    const uint32_t last = p.rank - 1, rdim = p.rank - 2;
    if (floats->strides[rdim] != 1 || p.shape[rdim] < 2) return false;
    if (values && (values->strides[last] != 1 || !aligned(values->ptr, 4))) return false;
    const bool native = values && s->store == CQ_STORE_NATIVE;
    const uint32_t unit = cq::rows_unit_values(dtype, static_cast<int>(p.bits));
    const uint64_t cols = p.shape[last];
    std::memset(t, 0, sizeof(*t));
    if (p.tensor_level) {
        t->segment = cols % 32 == 0 ? 32u : unit;
    } else {
        for (uint32_t d = 0; d < last; d++)
            if (p.layout.block[d] != 1) return false;
        t->segment = p.layout.block[last];
    }
    if (t->segment % unit || cols % t->segment || cols == 0) return false;
    if (native && values->strides[rdim] % 4) return false;
    t->tensor_level = p.tensor_level ? 1u : 0u;
    t->rows = static_cast<uint32_t>(p.shape[rdim]);
    t->segments = static_cast<uint32_t>(cols / t->segment);
    t->pitch_f = floats->strides[last];
    if (values) t->vrow = native ? values->strides[rdim] / 4 : values->strides[rdim];
    t->sa_row = p.layout.stride_a[rdim];
    t->sa_col = p.layout.stride_a[last];
    t->sb_row = p.layout.stride_b[rdim];
    t->sb_col = p.layout.stride_b[last];
    uint64_t batches = 1;
    for (uint32_t d = 0; d < rdim; d++) {
        if (p.shape[d] == 1) continue;
        if (native && values->strides[d] % 4) return false;
        const uint32_t k = t->num_batch_dims++;
        t->batch_shape[k] = static_cast<uint32_t>(p.shape[d]);
        t->batch_f[k] = floats->strides[d];
        if (values) t->batch_v[k] = native ? values->strides[d] / 4 : values->strides[d];
        t->batch_sa[k] = p.layout.stride_a[d];
        t->batch_sb[k] = p.layout.stride_b[d];
        batches *= p.shape[d];
    }
    if (batches > 65535 || (t->segments + 3) / 4 > 65535) return false;
    t->batches = static_cast<uint32_t>(batches);
    t->param_dtype = param_to_dtype(s->param);
    t->encoding = flat_encoding(s);
    t->range = p.range;
    return true;
}

// Blocks that are not a power-of-two number of lanes, fused abs-max (or given scales): contiguous tensors and
// scales, one run of blocks (see cq_kernels_staged.hip).  Fills `a` except the data pointers.
bool pieces_ok(const Plan& p, const cq_scheme* s, int dtype, const cq_tensor* floats, const cq_tensor* values,
               const cq_tensor* scale_a, const cq_tensor* scale_b, cq::PiecesArgs* a) {
    if (p.vs.on || p.tensor_level || !p.last_dim_blocks) return false;
    if (!aligned(floats->ptr, 16) || !aligned(values->ptr, 4)) return false;
    if (!is_contiguous(scale_a) || (scale_b && !is_contiguous(scale_b))) return false;
    *a = cq::PiecesArgs{};
    if (!cq::pieces_supported(dtype, static_cast<int>(p.bits), p.block_last, &a->per, &a->group_log2)) return false;
    const uint64_t per_chunk = 16 / dtype_size(dtype);
    a->num_chunks = p.n / per_chunk;
    if ((p.n * p.bits) % 32 != 0) return false;  // whole words of codes
    a->param_dtype = param_to_dtype(s->param);
    a->encoding = flat_encoding(s);
    a->range = p.range;
    return true;
}

// The leading dimensions of a scale tensor as one dimension of rows with a stride of its own (any stride along
// the last dimension).  False where they do not step uniformly.
bool scale_rows_and_columns(const cq_tensor* t, uint64_t* row_stride, uint64_t* col_stride) {
    const uint32_t last = t->rank - 1;
    *col_stride = t->strides[last];
    *row_stride = 0;
    uint64_t expect = 0;
    bool any = false;
    for (int d = static_cast<int>(last) - 1; d >= 0; d--) {
        if (t->shape[d] == 1) continue;
        if (!any) {
            any = true;
            *row_stride = t->strides[d];
        } else if (t->strides[d] != expect) {
            return false;
        }
        expect = t->strides[d] * t->shape[d];
    }
    return true;
}

// Rows of whole chunks with one pitch per value tensor, 1-D blocks of a power-of-two number of lanes, and scale
// tensors with a stride along the rows and another along the block columns, neither of which need be 1 (stored
// column by column, say): the tile kernels that move the scales through LDS (cq_kernels_staged.hip).  The launches
// before this one have taken the scale tensors whose last dimension is contiguous.  Fills `t` except the data
// pointers and scale_in_dtype.
bool scale_tiles_ok(const Plan& p, const cq_scheme* s, int dtype, const cq_tensor* floats, const cq_tensor* values,
                    const cq_tensor* scale_a, const cq_tensor* scale_b, cq::ScaleTileArgs* t) {
    if (p.tensor_level || !p.last_dim_blocks || !cq::flat_block_supported(dtype, p.block_last)) return false;
    const uint32_t last = p.rank - 1;
    const uint32_t elem = dtype_size(dtype), per_chunk = 16u / elem;
    const uint32_t stored = s->store == CQ_STORE_U32 ? 4u : 1u;
    RowLevels lf, lv;
    if (!row_levels(floats, &lf) || lf.levels > 1) return false;
    // the stored tensor: rows with one pitch, or (words of the U32 store) a stride along the last dimension as well,
    // in which case the codes of a tile pass through LDS like its scales
    uint64_t stored_col = 1;
    if (row_levels(values, &lv)) {
        if (lv.levels > 1 || lf.rows != lv.rows) return false;
    } else {
        uint64_t v_row = 0;
        // (two's-complement fields only: the kernels that stage codes are not compiled for the float encodings)
        if (s->store != CQ_STORE_U32 || flat_encoding(s) != 0 || !scale_rows_and_columns(values, &v_row, &stored_col) || stored_col == 0) return false;
        lv = RowLevels{1, lf.rows, lf.rows, v_row, 0};
    }
    const uint64_t cols = p.shape[last];
    const uint64_t chunk_elems = per_chunk > 32u / p.bits ? per_chunk : 32u / p.bits;  // whole chunks and whole words of codes
    if (cols == 0 || cols % chunk_elems || cols / per_chunk >= (1ull << 31) || lf.rows >= (1ull << 31)) return false;
    const uint32_t chunk_bytes = per_chunk * p.bits / 8;
    const uint32_t stored_align = chunk_bytes >= 8 && stored_col == 1 ? 8u : 4u;  // (staged codes leave word by word)
    if (!aligned(floats->ptr, 16) || (lf.inner * elem) % 16 || !aligned(values->ptr, stored_align) || (lv.inner * stored) % stored_align)
        return false;
    *t = cq::ScaleTileArgs{};
    if (!scale_rows_and_columns(scale_a, &t->sa_row, &t->sa_col)) return false;
    if (scale_b && !scale_rows_and_columns(scale_b, &t->sb_row, &t->sb_col)) return false;
    t->rows = static_cast<uint32_t>(lf.rows);
    t->row_chunks = static_cast<uint32_t>(cols / per_chunk);
    const uint32_t group = p.block_last / per_chunk;
    while ((1u << t->group_log2) < group) t->group_log2++;
    t->float_pitch = lf.inner * elem;
    t->stored_pitch = lv.inner * stored;
    t->stored_col = stored_col;
    t->param_dtype = param_to_dtype(s->param);
    t->encoding = flat_encoding(s);
    t->range = p.range;
    return true;
}

// A tensor whose elements fill a buffer without gaps or overlap (a permutation of a contiguous
// layout): order-free reductions may read the buffer front to back.
bool is_dense_permutation(const cq_tensor* t) {
    uint32_t order[CQ_MAX_RANK], n = 0;
    for (uint32_t d = 0; d < t->rank; d++)
        if (t->shape[d] != 1) order[n++] = d;
    for (uint32_t i = 1; i < n; i++)  // insertion sort by stride
        for (uint32_t j = i; j > 0 && t->strides[order[j]] < t->strides[order[j - 1]]; j--) {
            const uint32_t tmp = order[j];
            order[j] = order[j - 1];
            order[j - 1] = tmp;
        }
    uint64_t expect = 1;
    for (uint32_t i = 0; i < n; i++) {
        if (t->strides[order[i]] != expect) return false;
        expect *= t->shape[order[i]];
    }
    return true;
}

// Block abs-max by the row kernels: blocks over the last two dimensions only.
bool scales_rows_ok(const Plan& p) {
    if (p.tensor_level) return false;
    for (uint32_t d = 0; d + 2 < p.rank; d++)
        if (p.layout.block[d] != 1) return false;
    return true;
}

cq::GenericArgs generic_args(const Plan& p, const cq_scheme* s) {
    cq::GenericArgs g;
    std::memset(&g, 0, sizeof(g));
    g.param_dtype = param_to_dtype(s->param);
    g.value = s->value;
    g.range = p.range;
    g.layout = p.layout;
    g.vs = p.vs;
    return g;
}

// Scratch of cq_quantize_dynamic_static: the abs-max partials of the per-tensor grid reduction.  Every GPU
// holds its own copy of the array at its own address until the process ends.  In host code the array's name
// is only a handle for hipGetSymbolAddress, never a device address: kernels get the resolved pointer.
static __device__ __align__(256) unsigned char scratch[CQ_STATIC_SCRATCH_BYTES];
static_assert(CQ_STATIC_SCRATCH_BYTES >= cq::kMaxPartials * sizeof(float), "the partials of one reduction must fit");
constexpr int kMaxDevices = 64;
std::atomic<void*> g_scratch_ptr[kMaxDevices];

// Device address of `scratch` on the device the launches will run on, resolved on the first call per device
// (threads that race here resolve the same address).  hipGetSymbolAddress answers for the current device, so a
// stream that lives on another device is refused: its kernels would be handed this device's address.
cq_status static_scratch(hipStream_t stream, void** ptr) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return hip_status(e);
    if (dev < 0 || dev >= kMaxDevices) return CQ_ERR_INVALID_ARGUMENT;
    if (stream != nullptr) {  // the null stream is the current device's
        hipDevice_t stream_dev = -1;
        e = hipStreamGetDevice(stream, &stream_dev);
        if (e != hipSuccess) return hip_status(e);
        if (static_cast<int>(stream_dev) != dev) return CQ_ERR_INVALID_ARGUMENT;
    }
    void* p = g_scratch_ptr[dev].load(std::memory_order_acquire);
    if (p == nullptr) {
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return hip_status(e);
        if (p == nullptr) return CQ_ERR_HIP;
        g_scratch_ptr[dev].store(p, std::memory_order_release);
    }
    *ptr = p;
    return CQ_OK;
}

}  // namespace

extern "C" {

uint32_t cq_abi_version(void) { return CQ_ABI_VERSION; }

int cq_last_hip_error(void) { return g_last_hip_error; }

const char* cq_strerror(cq_status st) {
    switch (st) {
        case CQ_OK: return "success";
        case CQ_ERR_INVALID_ARGUMENT: return "invalid argument";
        case CQ_ERR_UNSUPPORTED_SCHEME: return "unsupported quantization scheme";
        case CQ_ERR_BLOCK_NOT_DIVISIBLE: return "block size must be divisible by the number of values per stored element";
        case CQ_ERR_SHAPE_MISMATCH: return "tensor shapes or element sizes do not agree with the scheme";
        case CQ_ERR_NON_CONTIGUOUS: return "tensor must be contiguous";
        case CQ_ERR_WORKSPACE_TOO_SMALL: return "workspace too small";
        case CQ_ERR_HIP: return "HIP runtime error";
        case CQ_ERR_TOO_LARGE: return "tensor too large";
        case CQ_ERR_INVALID_AXIS: return "the reduction axis must be smaller than the tensor rank";
        case CQ_ERR_SCRATCH_TOO_SMALL: return "the call needs more scratch memory than the library's built-in array holds; use the entry point that takes a workspace";
        default: return "unknown status";
    }
}

uint32_t cq_value_size_bits(uint8_t value) { return value_bits(value); }

uint32_t cq_scheme_num_quants(const cq_scheme* s) {
    if (!s || value_bits(s->value) == 0) return 0;
    return stored_nq(s);
}

cq_status cq_value_range(uint8_t value, float* lo, float* hi) {
    if (!lo || !hi) return CQ_ERR_INVALID_ARGUMENT;
    switch (value) {
        case CQ_VALUE_Q8F: *lo = -128.f; *hi = 127.f; break;
        case CQ_VALUE_Q8S: *lo = -127.f; *hi = 127.f; break;
        case CQ_VALUE_Q4F: *lo = -8.f; *hi = 7.f; break;
        case CQ_VALUE_Q4S: *lo = -7.f; *hi = 7.f; break;
        case CQ_VALUE_Q2F: *lo = -2.f; *hi = 1.f; break;
        case CQ_VALUE_Q2S: *lo = -1.f; *hi = 1.f; break;
        case CQ_VALUE_E2M1: case CQ_VALUE_E2M1_OCP: *lo = -6.f; *hi = 6.f; break;
        case CQ_VALUE_E4M3: *lo = -448.f; *hi = 448.f; break;
        case CQ_VALUE_E5M2: *lo = -57344.f; *hi = 57344.f; break;
        default: return CQ_ERR_INVALID_ARGUMENT;
    }
    return CQ_OK;
}

size_t cq_workspace_bytes(const cq_scheme* s, uint64_t /*num_elements*/) {
    if (!s || s->level != CQ_LEVEL_TENSOR) return 0;
    return cq::kMaxPartials * sizeof(float);  // abs-max partials of the grid reduction
}

cq_status cq_quantize(cq_stream_t stream, const cq_tensor* input, const cq_tensor* output,
                      const cq_tensor* scale, const cq_tensor* out_scale, const cq_scheme* scheme,
                      cq_dtype input_dtype) {
    drop_stale_hip_error();
    cq_status st = check_scheme(scheme);
    if (st != CQ_OK) return st;
    Plan p;
    int pd = param_to_dtype(scheme->param);
    st = make_plan(scheme, input, input_dtype, output, scale, dtype_size(input_dtype), out_scale,
                   dtype_size(pd), true, &p);
    if (st != CQ_OK) return st;
    if (!out_scale) return CQ_ERR_INVALID_ARGUMENT;
    if (p.n == 0) return CQ_OK;

    const bool native = scheme->store == CQ_STORE_NATIVE;
    const uint64_t per_chunk = 16 / dtype_size(input_dtype);
    uint64_t flat_words = 0;
    const bool wraps = wraps_its_field(scheme);  // the flat launches take such fields (lane by lane), the others do not
    const bool streaming = !wraps;
    // blocks that are not a power-of-two number of lanes on one contiguous run: the kernel of the fused quantize,
    // reading its scales (bf16 [28672, 8184], blocks of 24: 104 us against 114 us lane by lane)
    cq::PiecesArgs pc;
    if (streaming && pieces_ok(p, scheme, input_dtype, input, output, scale, out_scale, &pc)) {
        pc.input = input->ptr;
        pc.output = output->ptr;
        pc.scale_in = scale->ptr;
        pc.scale_out = out_scale->ptr;
        return CQ_RUN(CQ_FAMILY_STAGED, cq::launch_quantize_pieces(stream, input_dtype, static_cast<int>(p.bits), pc));
    }
    if (flat_ok(p, input_dtype, input, output, scale, out_scale, true)) {
        cq::FlatArgs a{};
        a.lanes_only = wraps;
        a.input = input->ptr;
        a.output = output->ptr;
        a.scale_in = scale->ptr;
        a.scale_in_dtype = input_dtype;
        a.scale_out = out_scale->ptr;
        // whole chunks that also end on a stored-element boundary
        uint64_t chunk_elems = per_chunk > 32u / p.bits ? per_chunk : 32u / p.bits;  // whole chunks and whole words of codes
        a.num_chunks = (p.n / chunk_elems) * chunk_elems / per_chunk;
        a.block = p.tensor_level ? 0 : p.block_last;
        a.param_dtype = pd;
        a.encoding = flat_encoding(scheme);
        a.range = p.range;
        st = CQ_RUN(cq::flat_family(a, input_dtype), cq::launch_quantize_flat(stream, input_dtype, p.bits, cq::ScaleSource::Given, a));
        if (st != CQ_OK) return st;
        flat_words = a.num_chunks * per_chunk / p.nq;
    }
    cq::FlatArgs fr{};
    if (flat_words == 0 && (flat_rows_ok(p, scheme, input_dtype, input, output, scale, dtype_size(input_dtype), out_scale,
                                         dtype_size(pd), true, &fr) ||
                            lane_rows_ok(p, scheme, input_dtype, input, output, scale, dtype_size(input_dtype), out_scale,
                                         dtype_size(pd), true, &fr))) {
        fr.lanes_only = wraps;
        fr.input = input->ptr;
        fr.output = output->ptr;
        fr.scale_in = scale->ptr;
        fr.scale_in_dtype = input_dtype;
        fr.scale_out = out_scale->ptr;
        fr.block = p.tensor_level ? 0 : p.block_last;
        fr.param_dtype = pd;
        fr.encoding = flat_encoding(scheme);
        fr.range = p.range;
        return CQ_RUN(cq::flat_family(fr, input_dtype), cq::launch_quantize_flat(stream, input_dtype, p.bits, cq::ScaleSource::Given, fr));
    }
    cq::ScaleTileArgs ts;
    if (streaming && flat_words == 0 && scale_tiles_ok(p, scheme, input_dtype, input, output, scale, out_scale, &ts)) {
        ts.input = input->ptr;
        ts.output = output->ptr;
        ts.scale_in = scale->ptr;
        ts.scale_in_dtype = input_dtype;
        ts.scale_out = out_scale->ptr;
        return CQ_RUN(CQ_FAMILY_STAGED, cq::launch_quantize_scale_tiles(stream, input_dtype, static_cast<int>(p.bits), ts));
    }
    cq::RowArgs r;
    if (streaming && flat_words == 0 && rows_args(p, scheme, input_dtype, input, output, &r)) {
        r.input = input->ptr;
        r.output = output->ptr;
        r.scale_in = scale->ptr;
        r.scale_in_dtype = input_dtype;
        r.scale_out = out_scale->ptr;
        return CQ_RUN(CQ_FAMILY_ROWS, cq::launch_quantize_rows(stream, input_dtype, static_cast<int>(p.bits), r));
    }
    cq::TransposedArgs tr;
    if (streaming && flat_words == 0 && transposed_args(p, scheme, input_dtype, input, output, &tr)) {
        tr.input = input->ptr;
        tr.output = output->ptr;
        tr.scale_in = scale->ptr;
        tr.scale_in_dtype = input_dtype;
        tr.scale_out = out_scale->ptr;
        return CQ_RUN(CQ_FAMILY_TRANSPOSED, cq::launch_quantize_transposed(stream, input_dtype, static_cast<int>(p.bits), false, tr));
    }
    if (flat_words < p.n / p.nq) {
        cq::GenericArgs g = generic_args(p, scheme);
        g.input = input->ptr;
        g.output = output->ptr;
        g.scale_in = scale->ptr;
        g.scale_in_dtype = input_dtype;
        g.scale_out = out_scale->ptr;
        g.word_begin = flat_words;
        g.word_end = p.n / p.nq;
        st = CQ_RUN(CQ_FAMILY_PER_ELEMENT, native ? cq::launch_quantize_native(stream, input_dtype, g)
                               : cq::launch_quantize_generic(stream, input_dtype, p.bits, g));
    }
    return st;
}

cq_status cq_dequantize(cq_stream_t stream, const cq_tensor* values, const cq_tensor* output,
                        const cq_tensor* params, const cq_scheme* scheme, cq_dtype output_dtype) {
    drop_stale_hip_error();
    cq_status st = check_scheme(scheme);
    if (st != CQ_OK) return st;
    Plan p;
    int pd = param_to_dtype(scheme->param);
    st = make_plan(scheme, output, output_dtype, values, params, dtype_size(pd), nullptr, 0, false, &p);
    if (st != CQ_OK) return st;
    if (p.n == 0) return CQ_OK;

    const bool native = scheme->store == CQ_STORE_NATIVE;
    const uint64_t per_chunk = 16 / dtype_size(output_dtype);
    uint64_t flat_words = 0;
    // blocks that split a word: only the per-element kernel scales a whole word by its first element's block
    const bool streaming = !p.block_splits_words;
    if (streaming && flat_ok(p, output_dtype, output, values, params, nullptr, true)) {
        cq::FlatArgs a{};
        a.input = values->ptr;
        a.output = output->ptr;
        a.scale_in = params->ptr;
        uint64_t chunk_elems = per_chunk > 32u / p.bits ? per_chunk : 32u / p.bits;  // whole chunks and whole words of codes
        a.num_chunks = (p.n / chunk_elems) * chunk_elems / per_chunk;
        a.block = p.tensor_level ? 0 : p.block_last;
        a.param_dtype = pd;
        a.encoding = flat_encoding(scheme);
        a.range = p.range;
        st = CQ_RUN(cq::flat_family(a, output_dtype), cq::launch_dequantize_flat(stream, output_dtype, p.bits, a));
        if (st != CQ_OK) return st;
        flat_words = a.num_chunks * per_chunk / p.nq;
    }
    cq::FlatArgs fr{};
    if (streaming && flat_words == 0 && (flat_rows_ok(p, scheme, output_dtype, output, values, params, dtype_size(pd), nullptr, 0, true, &fr) ||
                            lane_rows_ok(p, scheme, output_dtype, output, values, params, dtype_size(pd), nullptr, 0, true, &fr))) {
        fr.input = values->ptr;
        fr.output = output->ptr;
        fr.scale_in = params->ptr;
        swap_value_roles(&fr);
        fr.block = p.tensor_level ? 0 : p.block_last;
        fr.param_dtype = pd;
        fr.encoding = flat_encoding(scheme);
        fr.range = p.range;
        return CQ_RUN(cq::flat_family(fr, output_dtype), cq::launch_dequantize_flat(stream, output_dtype, p.bits, fr));
    }
    cq::ScaleTileArgs ts;
    if (streaming && flat_words == 0 && scale_tiles_ok(p, scheme, output_dtype, output, values, params, nullptr, &ts)) {
        ts.input = values->ptr;
        ts.output = output->ptr;
        ts.scale_in = params->ptr;
        return CQ_RUN(CQ_FAMILY_STAGED, cq::launch_dequantize_scale_tiles(stream, output_dtype, static_cast<int>(p.bits), ts));
    }
    cq::RowArgs r;
    if (streaming && flat_words == 0 && rows_args(p, scheme, output_dtype, output, values, &r)) {
        r.input = values->ptr;
        r.output = output->ptr;
        r.scale_in = params->ptr;
        return CQ_RUN(CQ_FAMILY_ROWS, cq::launch_dequantize_rows(stream, output_dtype, static_cast<int>(p.bits), r));
    }
    cq::TransposedArgs tr;
    if (streaming && flat_words == 0 && transposed_args(p, scheme, output_dtype, output, values, &tr)) {
        tr.input = values->ptr;
        tr.output = output->ptr;
        tr.scale_in = params->ptr;
        return CQ_RUN(CQ_FAMILY_TRANSPOSED, cq::launch_dequantize_transposed(stream, output_dtype, static_cast<int>(p.bits), tr));
    }
    if (flat_words < p.n / p.nq) {
        cq::GenericArgs g = generic_args(p, scheme);
        g.input = values->ptr;
        g.output = output->ptr;
        g.scale_in = params->ptr;
        g.word_begin = flat_words;
        g.word_end = p.n / p.nq;
        st = CQ_RUN(CQ_FAMILY_PER_ELEMENT, native ? cq::launch_dequantize_native(stream, output_dtype, g)
                               : cq::launch_dequantize_generic(stream, output_dtype, p.bits, g));
    }
    return st;
}

// Shared by cq_compute_scales and cq_quantize_dynamic: scale of every block (or
// of the tensor) as out_dtype(F(2*absmax/(hi-lo))), written into `scales`.
// Pass 1 of the per-tensor reduction for any layout of the float tensor: `*num_partials` f32
// abs-max partials in the workspace.
static cq_status absmax_partials(cq_stream_t stream, const Plan& p, const cq_scheme* scheme, const cq_tensor* input,
                                 int input_dtype, void* workspace, size_t workspace_bytes, uint32_t* num_partials) {
    if (!workspace || workspace_bytes < cq::kMaxPartials * sizeof(float)) return CQ_ERR_WORKSPACE_TOO_SMALL;
    if (!aligned(workspace, 4)) return CQ_ERR_INVALID_ARGUMENT;
    cq::RowArgs r;
    if (p.vs.on && is_dense_permutation(input)) {
        // the order does not matter for a maximum: read the buffer front to back
        return CQ_RUN_AUX(CQ_FAMILY_FLAT, cq::launch_absmax_partials(stream, input_dtype, input->ptr, p.n, static_cast<float*>(workspace),
                                                     num_partials));
    }
    if (p.vs.on && rows_args(p, scheme, input_dtype, input, nullptr, &r)) {
        r.input = input->ptr;
        return CQ_RUN_AUX(CQ_FAMILY_ROWS, cq::launch_absmax_partials_rows(stream, input_dtype, r, static_cast<float*>(workspace), num_partials));
    }
    if (p.vs.on) {
        cq::GenericArgs g = generic_args(p, scheme);
        g.input = input->ptr;
        return CQ_RUN_AUX(CQ_FAMILY_PER_ELEMENT, cq::launch_absmax_partials_strided(stream, input_dtype, g, p.n, static_cast<float*>(workspace),
                                                             num_partials));
    }
    return CQ_RUN_AUX(CQ_FAMILY_FLAT, cq::launch_absmax_partials(stream, input_dtype, input->ptr, p.n, static_cast<float*>(workspace),
                                                 num_partials));
}

static cq_status produce_scales(cq_stream_t stream, const Plan& p, const cq_scheme* scheme,
                                const cq_tensor* input, int input_dtype, const cq_tensor* scales,
                                int out_dtype, void* workspace, size_t workspace_bytes) {
    if (p.tensor_level) {
        uint32_t num_partials = 0;
        const cq_status st = absmax_partials(stream, p, scheme, input, input_dtype, workspace, workspace_bytes, &num_partials);
        if (st != CQ_OK) return st;
        return CQ_RUN_AUX(CQ_FAMILY_FLAT, cq::launch_tensor_scale(stream, input_dtype, out_dtype,
                                                  static_cast<const float*>(workspace), num_partials,
                                                  p.range, scales->ptr));
    }
    cq::RowArgs r;
    if (scales_rows_ok(p) && rows_args(p, scheme, input_dtype, input, nullptr, &r)) {
        r.input = input->ptr;
        r.scale_out = scales->ptr;
        return CQ_RUN_AUX(CQ_FAMILY_ROWS, cq::launch_scales_rows(stream, input_dtype, out_dtype, r));
    }
    cq::TransposedArgs tr;
    if (transposed_args(p, scheme, input_dtype, input, nullptr, &tr)) {
        tr.input = input->ptr;
        tr.scale_out = scales->ptr;
        return CQ_RUN_AUX(CQ_FAMILY_TRANSPOSED, cq::launch_scales_transposed(stream, input_dtype, out_dtype, tr));
    }
    cq::GenericArgs g = generic_args(p, scheme);
    g.input = input->ptr;
    g.scale_out = scales->ptr;
    return CQ_RUN_AUX(CQ_FAMILY_PER_ELEMENT, cq::launch_scales_generic(stream, input_dtype, out_dtype, g, p.num_blocks));
}

cq_status cq_compute_scales(cq_stream_t stream, const cq_tensor* input, const cq_tensor* scales,
                            const cq_scheme* scheme, cq_dtype input_dtype, void* workspace,
                            size_t workspace_bytes) {
    drop_stale_hip_error();
    cq_status st = check_scheme(scheme);
    if (st != CQ_OK) return st;
    if (!tensor_ok(input) || !tensor_ok(scales) || !valid_dtype(input_dtype)) return CQ_ERR_INVALID_ARGUMENT;
    // build the plan against a synthetic stored tensor of the right shape
    uint64_t vshape[CQ_MAX_RANK], vstrides[CQ_MAX_RANK];
    uint32_t nq = stored_nq(scheme);
    if (input->shape[input->rank - 1] % nq) return CQ_ERR_SHAPE_MISMATCH;
    uint64_t acc = 1;
    for (int d = static_cast<int>(input->rank) - 1; d >= 0; d--) {
        vshape[d] = d + 1 == static_cast<int>(input->rank) ? input->shape[d] / nq : input->shape[d];
        vstrides[d] = acc;
        acc *= vshape[d];
    }
    cq_tensor values{input->ptr, vshape, vstrides, input->rank, scheme->store == CQ_STORE_U32 ? 4u : 1u};
    Plan p;
    st = make_plan(scheme, input, input_dtype, &values, scales, dtype_size(input_dtype), nullptr, 0, false, &p);
    if (st != CQ_OK) return st;
    if (p.n == 0) return CQ_OK;

    if (!p.vs.on && !p.tensor_level && p.last_dim_blocks && is_contiguous(scales) && aligned(input->ptr, 16) &&
        cq::flat_block_supported(input_dtype, p.block_last)) {
        cq::FlatArgs a{};
        a.input = input->ptr;
        a.scale_out = scales->ptr;
        a.num_chunks = p.n / (16 / dtype_size(input_dtype));
        a.block = p.block_last;
        a.range = p.range;
        return CQ_RUN_AUX(cq::flat_family(a, input_dtype), cq::launch_scales_flat(stream, input_dtype, a));
    }
    // pitched rows of at least a step of 256 chunks, 1-D blocks: the same kernel over the rows' steps
    // (rows in one uniform run or in groups with a pitch of their own, as in flat_rows_ok())
    const uint32_t elem = dtype_size(input_dtype);
    const uint64_t row_chunks = input->shape[input->rank - 1] / (16 / elem);
    RowLevels lf, ls;
    if (!p.tensor_level && p.last_dim_blocks && p.rank >= 2 && cq::flat_block_supported(input_dtype, p.block_last) &&
        row_levels(input, &lf) && row_levels(scales, &ls) && lf.rows == ls.rows &&
        !(lf.levels == 2 && ls.levels == 2 && lf.inner_rows != ls.inner_rows) &&
        input->shape[input->rank - 1] % (16 / elem) == 0 && row_chunks >= 256 &&
        ((row_chunks + 255) / 256 * 256 - row_chunks) * 10 <= row_chunks * 6 &&
        lf.rows * ((row_chunks + 255) / 256) < (1ull << 31)) {
        const uint64_t inner_rows = lf.levels == 2 ? lf.inner_rows : (ls.levels == 2 ? ls.inner_rows : lf.rows);
        const auto outer_of = [&](const RowLevels& l) { return l.levels == 2 ? l.outer : l.inner * inner_rows; };
        if (aligned(input->ptr, 16) && (lf.inner * elem) % 16 == 0 && (outer_of(lf) * elem) % 16 == 0) {
            cq::FlatArgs a{};
            a.input = input->ptr;
            a.scale_out = scales->ptr;
            a.num_chunks = row_chunks;
            a.rows = lf.rows;
            a.inner_rows = inner_rows;
            a.in_pitch = lf.inner * elem;
            a.in_outer = outer_of(lf) * elem;
            a.scale_out_pitch = ls.inner * elem;
            a.scale_out_outer = outer_of(ls) * elem;
            a.block = p.block_last;
            a.range = p.range;
            return CQ_RUN_AUX(cq::flat_family(a, input_dtype), cq::launch_scales_flat(stream, input_dtype, a));
        }
    }
    // short rows, rows behind several levels of strides: every lane finds its row
    cq::FlatArgs fl{};
    if (!p.tensor_level && lane_rows_ok(p, scheme, input_dtype, input, nullptr, scales, elem, nullptr, 0, false, &fl)) {
        scale_in_to_out(&fl);
        fl.input = input->ptr;
        fl.scale_out = scales->ptr;
        fl.block = p.block_last;
        fl.range = p.range;
        return CQ_RUN_AUX(cq::flat_family(fl, input_dtype), cq::launch_scales_flat(stream, input_dtype, fl));
    }
    return produce_scales(stream, p, scheme, input, input_dtype, scales, input_dtype, workspace, workspace_bytes);
}

static cq_status quantize_dynamic(cq_stream_t stream, const cq_tensor* input, const cq_tensor* output,
                                  const cq_tensor* out_scale, const cq_scheme* scheme, cq_dtype input_dtype,
                                  void* workspace, size_t workspace_bytes) {
    drop_stale_hip_error();
    cq_status st = check_scheme(scheme);
    if (st != CQ_OK) return st;
    if (!out_scale) return CQ_ERR_INVALID_ARGUMENT;
    Plan p;
    int pd = param_to_dtype(scheme->param);
    st = make_plan(scheme, input, input_dtype, output, out_scale, dtype_size(pd), nullptr, 0, true, &p);
    if (st != CQ_OK) return st;
    if (p.n == 0) return CQ_OK;

    const uint64_t per_chunk = 16 / dtype_size(input_dtype);
    const bool native = scheme->store == CQ_STORE_NATIVE;
    const bool wraps = wraps_its_field(scheme);  // the flat launches take such fields (lane by lane), the others do not
    const bool flat = flat_ok(p, input_dtype, input, output, out_scale, nullptr, false);

    // fused single pass: abs-max, scale, quantize, pack in registers (whole 32-bit words of codes: lanes that
    // share a word store it together)
    const uint64_t word_elems = per_chunk > 32u / p.bits ? per_chunk : 32u / p.bits;
    if (flat && !p.tensor_level && p.n % word_elems == 0) {
        cq::FlatArgs a{};
        a.input = input->ptr;
        a.output = output->ptr;
        a.scale_out = out_scale->ptr;
        a.num_chunks = p.n / per_chunk;
        a.block = p.block_last;
        a.param_dtype = pd;
        a.encoding = flat_encoding(scheme);
        a.range = p.range;
        a.lanes_only = wraps;
        return CQ_RUN(cq::flat_family(a, input_dtype), cq::launch_quantize_flat(stream, input_dtype, p.bits, cq::ScaleSource::Dynamic, a));
    }

    // pitched rows with 1-D blocks: the same fused kernel over the rows' steps
    cq::FlatArgs fr{};
    if (!p.tensor_level && (flat_rows_ok(p, scheme, input_dtype, input, output, out_scale, dtype_size(pd), nullptr, 0, false, &fr) ||
                            lane_rows_ok(p, scheme, input_dtype, input, output, out_scale, dtype_size(pd), nullptr, 0, false, &fr))) {
        fr.input = input->ptr;
        fr.output = output->ptr;
        fr.scale_out = out_scale->ptr;
        scale_in_to_out(&fr);
        fr.lanes_only = wraps;
        fr.block = p.block_last;
        fr.param_dtype = pd;
        fr.encoding = flat_encoding(scheme);
        fr.range = p.range;
        return CQ_RUN(cq::flat_family(fr, input_dtype), cq::launch_quantize_flat(stream, input_dtype, p.bits, cq::ScaleSource::Dynamic, fr));
    }

    // 1-D blocks that are not a power-of-two number of lanes, on one contiguous run: a lane holds a whole piece of its block
    cq::PiecesArgs pc;
    if (!wraps && pieces_ok(p, scheme, input_dtype, input, output, out_scale, nullptr, &pc)) {
        pc.input = input->ptr;
        pc.output = output->ptr;
        pc.scale_out = out_scale->ptr;
        return CQ_RUN(CQ_FAMILY_STAGED, cq::launch_quantize_pieces(stream, input_dtype, static_cast<int>(p.bits), pc));
    }
    // scale tensors whose last dimension is not the contiguous one: the scales of a tile leave through LDS
    cq::ScaleTileArgs ts;
    if (!wraps && scale_tiles_ok(p, scheme, input_dtype, input, output, out_scale, out_scale, &ts)) {
        ts.input = input->ptr;
        ts.output = output->ptr;
        ts.scale_out = out_scale->ptr;
        return CQ_RUN(CQ_FAMILY_STAGED, cq::launch_quantize_scale_tiles(stream, input_dtype, static_cast<int>(p.bits), ts));
    }

    // blocks over the last two dimensions (or 1-D blocks on layouts the flat kernel refuses): one
    // launch that owns whole blocks
    // Blocks of 8 - 64 rows on rows of at most 1 KiB leave the fused block kernel too few lanes along the row
    // (18 - 35 % of HBM peak).  Two launches take half the time there: the blocks' scales as FS(F(scale)) into
    // out_scale, then the flat body, lane by lane, reading them back (the divisor F(FS(scale)) is the same either way).
    if (!p.tensor_level && p.rank >= 2 && scales_rows_ok(p) && p.layout.block[p.rank - 2] >= 8 && p.layout.block[p.rank - 2] <= 64 &&
        p.shape[p.rank - 1] * dtype_size(input_dtype) <= 1024) {
        cq::FlatArgs f2{};
        if (lane_rows_ok(p, scheme, input_dtype, input, output, out_scale, dtype_size(pd), nullptr, 0, true, &f2)) {
            st = produce_scales(stream, p, scheme, input, input_dtype, out_scale, pd, workspace, workspace_bytes);
            if (st != CQ_OK) return st;
            f2.input = input->ptr;
            f2.output = output->ptr;
            f2.scale_in = out_scale->ptr;
            f2.lanes_only = wraps;
            f2.block = p.block_last;
            f2.param_dtype = pd;
            f2.encoding = flat_encoding(scheme);
            f2.range = p.range;
            return CQ_RUN(cq::flat_family(f2, input_dtype), cq::launch_quantize_flat(stream, input_dtype, p.bits, cq::ScaleSource::Stored, f2));
        }
    }

    cq::RowArgs rb;
    if (!wraps && !p.tensor_level && scales_rows_ok(p) && rows_args(p, scheme, input_dtype, input, output, &rb) &&
        cq::blocks_dynamic_supported(input_dtype, static_cast<int>(p.bits), rb)) {
        rb.input = input->ptr;
        rb.output = output->ptr;
        rb.scale_out = out_scale->ptr;
        return CQ_RUN(CQ_FAMILY_BLOCKS, cq::launch_quantize_blocks_dynamic(stream, input_dtype, static_cast<int>(p.bits), rb));
    }

    cq::TransposedArgs tr;
    const bool transposed = !wraps && !flat && transposed_args(p, scheme, input_dtype, input, output, &tr);
    if (transposed && !p.tensor_level) {  // each thread owns whole blocks: one launch
        tr.input = input->ptr;
        tr.output = output->ptr;
        tr.scale_out = out_scale->ptr;
        return CQ_RUN(CQ_FAMILY_TRANSPOSED, cq::launch_quantize_transposed(stream, input_dtype, static_cast<int>(p.bits), true, tr));
    }

    uint64_t flat_words = 0;
    // whole chunks and whole 32-bit words of codes (lanes that share a word store it together)
    const uint64_t chunk_elems = per_chunk > 32u / p.bits ? per_chunk : 32u / p.bits;
    const uint64_t flat_chunks = flat ? (p.n / chunk_elems) * chunk_elems / per_chunk : 0;
    if (p.tensor_level && flat_chunks > 0) {
        // per tensor, two-pass grid reduction: pass 1 leaves one abs-max per workgroup in
        // the workspace; pass 2 (the quantize kernel) reduces those, derives the scale,
        // writes out_scale[0] and quantizes
        if (!workspace || workspace_bytes < cq::kMaxPartials * sizeof(float)) return CQ_ERR_WORKSPACE_TOO_SMALL;
        if (!aligned(workspace, 4)) return CQ_ERR_INVALID_ARGUMENT;
        uint32_t num_partials = 0;
        st = CQ_RUN_AUX(CQ_FAMILY_FLAT, cq::launch_absmax_partials(stream, input_dtype, input->ptr, p.n,
                                                   static_cast<float*>(workspace), &num_partials));
        if (st != CQ_OK) return st;
        cq::FlatArgs a{};
        a.input = input->ptr;
        a.output = output->ptr;
        a.scale_in = workspace;
        a.num_partials = num_partials;
        a.scale_out = out_scale->ptr;
        a.num_chunks = flat_chunks;
        a.lanes_only = wraps;
        a.block = 0;
        a.param_dtype = pd;
        a.encoding = flat_encoding(scheme);
        a.range = p.range;
        st = CQ_RUN(cq::flat_family(a, input_dtype), cq::launch_quantize_flat(stream, input_dtype, p.bits, cq::ScaleSource::Partials, a));
        if (st != CQ_OK) return st;
        flat_words = flat_chunks * per_chunk / p.nq;
    } else if (p.tensor_level && (flat_rows_ok(p, scheme, input_dtype, input, output, out_scale, dtype_size(pd), nullptr, 0, false, &fr) ||
                                  lane_rows_ok(p, scheme, input_dtype, input, output, out_scale, dtype_size(pd), nullptr, 0, false, &fr))) {
        // per tensor on pitched rows: the same two passes, the second one over the rows' steps
        uint32_t num_partials = 0;
        st = absmax_partials(stream, p, scheme, input, input_dtype, workspace, workspace_bytes, &num_partials);
        if (st != CQ_OK) return st;
        fr.input = input->ptr;
        fr.output = output->ptr;
        fr.scale_in = workspace;
        fr.num_partials = num_partials;
        fr.scale_out = out_scale->ptr;
        fr.lanes_only = wraps;
        fr.block = 0;
        fr.param_dtype = pd;
        fr.encoding = flat_encoding(scheme);
        fr.range = p.range;
        return CQ_RUN(cq::flat_family(fr, input_dtype), cq::launch_quantize_flat(stream, input_dtype, p.bits, cq::ScaleSource::Partials, fr));
    } else {
        // scales as FS(F(scale)) into out_scale first, then quantize reading them back
        // (the divisor F(FS(scale)) is the same either way)
        st = produce_scales(stream, p, scheme, input, input_dtype, out_scale, pd, workspace, workspace_bytes);
        if (st != CQ_OK) return st;
    }
    cq::RowArgs r;
    if (!wraps && flat_words == 0 && rows_args(p, scheme, input_dtype, input, output, &r)) {
        r.input = input->ptr;
        r.output = output->ptr;
        r.scale_in = out_scale->ptr;
        r.scale_in_dtype = pd;
        r.scale_out = nullptr;
        return CQ_RUN(CQ_FAMILY_ROWS, cq::launch_quantize_rows(stream, input_dtype, static_cast<int>(p.bits), r));
    }
    if (flat_words == 0 && transposed) {
        tr.input = input->ptr;
        tr.output = output->ptr;
        tr.scale_in = out_scale->ptr;
        tr.scale_in_dtype = pd;
        tr.scale_out = nullptr;
        return CQ_RUN(CQ_FAMILY_TRANSPOSED, cq::launch_quantize_transposed(stream, input_dtype, static_cast<int>(p.bits), false, tr));
    }
    if (flat_words < p.n / p.nq) {
        cq::GenericArgs g = generic_args(p, scheme);
        g.input = input->ptr;
        g.output = output->ptr;
        g.scale_in = out_scale->ptr;
        g.scale_in_dtype = pd;
        g.scale_out = nullptr;
        g.word_begin = flat_words;
        g.word_end = p.n / p.nq;
        st = CQ_RUN(CQ_FAMILY_PER_ELEMENT, native ? cq::launch_quantize_native(stream, input_dtype, g)
                               : cq::launch_quantize_generic(stream, input_dtype, p.bits, g));
    }
    return st;
}

cq_status cq_quantize_dynamic(cq_stream_t stream, const cq_tensor* input, const cq_tensor* output,
                              const cq_tensor* out_scale, const cq_scheme* scheme, cq_dtype input_dtype,
                              void* workspace, size_t workspace_bytes) {
    return quantize_dynamic(stream, input, output, out_scale, scheme, input_dtype, workspace, workspace_bytes);
}

cq_status cq_quantize_dynamic_static(cq_stream_t stream, const cq_tensor* input, const cq_tensor* output,
                                     const cq_tensor* out_scale, const cq_scheme* scheme, cq_dtype input_dtype) {
    cq_status st = check_scheme(scheme);
    if (st != CQ_OK) return st;
    if (!tensor_ok(input)) return CQ_ERR_INVALID_ARGUMENT;
    // what the call would ask of a caller's workspace must fit the array
    uint64_t n = 1;
    for (uint32_t d = 0; d < input->rank; d++) {
        if (input->shape[d] != 0 && n > (1ull << 48) / input->shape[d]) return CQ_ERR_TOO_LARGE;
        n *= input->shape[d];
    }
    if (cq_workspace_bytes(scheme, n) > CQ_STATIC_SCRATCH_BYTES) return CQ_ERR_SCRATCH_TOO_SMALL;
    void* ws = nullptr;
    st = static_scratch(stream, &ws);
    if (st != CQ_OK) return st;
    return quantize_dynamic(stream, input, output, out_scale, scheme, input_dtype, ws, CQ_STATIC_SCRATCH_BYTES);
}

cq_status cq_into_contiguous_packed(cq_stream_t stream, const cq_tensor* input, const cq_tensor* output,
                                    const uint64_t* shape, uint32_t rank, uint32_t packing) {
    drop_stale_hip_error();
    if (!tensor_ok(input) || !tensor_ok(output) || !shape) return CQ_ERR_INVALID_ARGUMENT;
    if (input->rank != rank || output->rank != rank) return CQ_ERR_SHAPE_MISMATCH;
    const uint32_t elem = input->elem_size;
    if ((elem != 4 && elem != 1) || output->elem_size != elem) return CQ_ERR_SHAPE_MISMATCH;
    if (packing == 0 || (8 * elem) % packing) return CQ_ERR_INVALID_ARGUMENT;
    cq::RepackArgs a;
    std::memset(&a, 0, sizeof(a));
    // packed along the rightmost dimension of stride 1
    a.packed_dim = rank - 1;
    for (int d = static_cast<int>(rank) - 1; d >= 0; d--)
        if (input->strides[d] == 1) {
            a.packed_dim = static_cast<uint32_t>(d);
            break;
        }
    if (shape[rank - 1] % packing || shape[a.packed_dim] % packing) return CQ_ERR_SHAPE_MISMATCH;
    a.num_out = 1;
    for (uint32_t d = 0; d < rank; d++) {
        if (shape[d] > 0xffffffffull) return CQ_ERR_TOO_LARGE;
        if (input->shape[d] != (d == a.packed_dim ? shape[d] / packing : shape[d])) return CQ_ERR_SHAPE_MISMATCH;
        if (output->shape[d] != (d + 1 == rank ? shape[d] / packing : shape[d])) return CQ_ERR_SHAPE_MISMATCH;
        a.shape[d] = static_cast<uint32_t>(shape[d]);
        a.strides[d] = input->strides[d];
        a.num_out *= output->shape[d];
    }
    if (!is_contiguous(output)) return CQ_ERR_NON_CONTIGUOUS;
    a.input = input->ptr;
    a.output = output->ptr;
    a.elem_bytes = elem;
    a.packing = packing;
    a.bits = 8 * elem / packing;
    a.rank = rank;
    return hip_status(cq::launch_repack(stream, a));
}

cq_status cq_gemv_quantized(cq_stream_t stream, const cq_tensor* values, const cq_tensor* params, const cq_scheme* scheme,
                            const cq_tensor* x, const cq_tensor* y, cq_dtype dtype, cq_dtype y_dtype) {
    drop_stale_hip_error();
    cq_status st = check_scheme(scheme);
    if (st != CQ_OK) return st;
    const bool native = scheme->store == CQ_STORE_NATIVE;
    // the native store holds i8, e4m3, e5m2 bytes or e2m1 pairs (src/quantize.rs:196-219)
    if (native && scheme->value != CQ_VALUE_Q8F && scheme->value != CQ_VALUE_Q8S && scheme->value != CQ_VALUE_E4M3 &&
        scheme->value != CQ_VALUE_E5M2 && scheme->value != CQ_VALUE_E2M1 && scheme->value != CQ_VALUE_E2M1_OCP)
        return CQ_ERR_UNSUPPORTED_SCHEME;
    if (!tensor_ok(values) || !tensor_ok(params) || !tensor_ok(x) || !tensor_ok(y) || !valid_dtype(dtype) ||
        !valid_dtype(y_dtype))
        return CQ_ERR_INVALID_ARGUMENT;
    const int pd = param_to_dtype(scheme->param);
    // x: [cols] or [vectors, cols]; y: [rows] or [vectors, rows]
    if (values->rank != 2 || x->rank < 1 || x->rank > 2 || y->rank != x->rank) return CQ_ERR_SHAPE_MISMATCH;
    const uint32_t last = x->rank - 1;
    const uint64_t vectors = x->rank == 2 ? x->shape[0] : 1;
    if (values->elem_size != (native ? 1u : 4u) || x->elem_size != dtype_size(dtype) || y->elem_size != dtype_size(y_dtype) ||
        params->elem_size != dtype_size(pd))
        return CQ_ERR_SHAPE_MISMATCH;
    const uint32_t bits = value_bits(scheme->value);
    const uint32_t nq = stored_nq(scheme);  // values per stored element
    const uint64_t rows = values->shape[0], cols = values->shape[1] * nq;
    if (rows > 0xffffffffull || cols > 0xffffffffull) return CQ_ERR_TOO_LARGE;
    if (x->shape[last] != cols || y->shape[last] != rows || (x->rank == 2 && y->shape[0] != vectors))
        return CQ_ERR_SHAPE_MISMATCH;
    if (vectors > 0xffffffffull) return CQ_ERR_TOO_LARGE;
    if ((values->shape[1] != 1 && values->strides[1] != 1) || (cols != 1 && x->strides[last] != 1) ||
        (rows != 1 && y->strides[last] != 1))
        return CQ_ERR_NON_CONTIGUOUS;
    cq::GemvArgs a{};
    if (scheme->level == CQ_LEVEL_BLOCK) {
        if (scheme->block_rank > 2 || params->rank != 2) return CQ_ERR_SHAPE_MISMATCH;
        a.block_cols = scheme->block[scheme->block_rank - 1];
        a.block_rows = scheme->block_rank == 2 ? scheme->block[0] : 1;
        if (rows % a.block_rows || cols % a.block_cols || params->shape[0] != rows / a.block_rows ||
            params->shape[1] != cols / a.block_cols)
            return CQ_ERR_SHAPE_MISMATCH;
        a.scale_stride_row = params->strides[0];
        a.scale_stride_col = params->strides[1];
    } else if (numel(params) < 1) {
        return CQ_ERR_SHAPE_MISMATCH;
    }
    if (rows == 0 || vectors == 0) return CQ_OK;
    a.vectors = static_cast<uint32_t>(vectors);
    a.x_stride = x->rank == 2 ? x->strides[0] : 0;
    a.y_stride = y->rank == 2 ? y->strides[0] : 0;
    a.words = values->ptr;
    a.scales = params->ptr;
    a.x = x->ptr;
    a.y = y->ptr;
    a.dtype = dtype;
    a.y_dtype = y_dtype;
    a.param_dtype = pd;
    a.bits = bits;
    a.rows = static_cast<uint32_t>(rows);
    a.cols = static_cast<uint32_t>(cols);
    a.word_pitch = values->strides[0];
    a.x_aligned16 = aligned(x->ptr, 16);
    a.words_aligned16 = aligned(values->ptr, 16);
    if (native) {
        // only the streaming kernel reads the native store: rows of whole 16-byte units on 16-byte boundaries
        a.native = scheme->value == CQ_VALUE_E4M3 ? 1u : scheme->value == CQ_VALUE_E5M2 ? 2u
                   : (scheme->value == CQ_VALUE_E2M1 || scheme->value == CQ_VALUE_E2M1_OCP) ? 3u : 0u;
        if (values->strides[0] % 16 != 0 && rows > 1) return CQ_ERR_UNSUPPORTED_SCHEME;
        a.word_pitch = values->strides[0] / 4;
        if (!cq::gemv_streams(a)) return CQ_ERR_UNSUPPORTED_SCHEME;
    } else if (scheme->value == CQ_VALUE_E2M1_OCP) {
        // e2m1 nibbles in u32 words are the native store's bytes: the same kernel, the pitch already in words
        a.native = 3u;
        if (values->strides[0] % 4 != 0 && rows > 1) return CQ_ERR_UNSUPPORTED_SCHEME;
        if (!cq::gemv_streams(a)) return CQ_ERR_UNSUPPORTED_SCHEME;
    }
    return CQ_RUN(cq::gemv_streams(a) ? CQ_FAMILY_FLAT : CQ_FAMILY_ROWS, cq::launch_gemv_quantized(stream, a));
}

cq_status cq_plan_kind(cq_op op, const cq_tensor* floats, const cq_tensor* values, const cq_tensor* scale,
                       const cq_tensor* out_scale, const cq_scheme* scheme, cq_dtype dtype, uint32_t* family) {
    if (!family) return CQ_ERR_INVALID_ARGUMENT;
    *family = CQ_FAMILY_NONE;
    // a workspace that satisfies every check; with the launches switched off nothing touches it
    alignas(256) static char workspace[CQ_STATIC_SCRATCH_BYTES];
    g_probe = PlanProbe{};
    g_probe.on = true;
    cq_status st = CQ_ERR_INVALID_ARGUMENT;
    switch (op) {
        case CQ_OP_QUANTIZE: st = cq_quantize(nullptr, floats, values, scale, out_scale, scheme, dtype); break;
        case CQ_OP_QUANTIZE_DYNAMIC:
            st = quantize_dynamic(nullptr, floats, values, out_scale, scheme, dtype, workspace, sizeof(workspace));
            break;
        case CQ_OP_DEQUANTIZE: st = cq_dequantize(nullptr, values, floats, scale, scheme, dtype); break;
        case CQ_OP_COMPUTE_SCALES:
            st = cq_compute_scales(nullptr, floats, scale, scheme, dtype, workspace, sizeof(workspace));
            break;
        case CQ_OP_GEMV:
            st = cq_gemv_quantized(nullptr, values, scale, scheme, floats, out_scale, dtype,
                                   out_scale && out_scale->elem_size == 4 ? CQ_F32 : dtype);
            break;
    }
    *family = g_probe.main != CQ_FAMILY_NONE ? g_probe.main : g_probe.aux;
    g_probe = PlanProbe{};
    return st;
}

static bool reduce_view(const cq_tensor* input, uint32_t axis, uint64_t* outer, uint64_t* len, uint64_t* inner) {
    *outer = *inner = 1;
    for (uint32_t d = 0; d < axis; d++) *outer *= input->shape[d];
    for (uint32_t d = axis + 1; d < input->rank; d++) *inner *= input->shape[d];
    *len = input->shape[axis];
    return true;
}

// A reduction does not care about the order of the dimensions.  Where the input's last dimension is not the
// contiguous one (a transposed view), the dimensions are put in the order of the input's strides, slowest
// first, if the output, permuted the same way, is still contiguous (always so for matrices): the kernels
// for contiguous rows then apply.  `out_strides` NULL: the output is taken to be contiguous.  Returns
// the tensors to launch with (the caller's, or the permuted copies in `store`) and the axis among them.
struct PermutedReduce {
    uint64_t shape[CQ_MAX_RANK], in_strides[CQ_MAX_RANK], out_shape[CQ_MAX_RANK], out_strides[CQ_MAX_RANK];
    cq_tensor input, output;
};
static uint32_t canonical_reduce(const cq_tensor* input, const cq_tensor* output, uint32_t axis, PermutedReduce* store,
                                 const cq_tensor** in_used, const cq_tensor** out_used) {
    *in_used = input;
    *out_used = output;
    const uint32_t rank = input->rank;
    if (rank < 2 || input->shape[rank - 1] == 1 || input->strides[rank - 1] == 1) return axis;
    uint32_t order[CQ_MAX_RANK];
    for (uint32_t d = 0; d < rank; d++) order[d] = d;
    for (uint32_t i = 1; i < rank; i++)  // insertion sort, stable: strides descending
        for (uint32_t j = i; j > 0 && input->strides[order[j - 1]] < input->strides[order[j]]; j--) std::swap(order[j - 1], order[j]);
    uint64_t contiguous_out[CQ_MAX_RANK], expect = 1;
    for (int d = static_cast<int>(rank) - 1; d >= 0; d--) {
        contiguous_out[d] = expect;
        expect *= static_cast<uint32_t>(d) == axis ? 1 : input->shape[d];
    }
    uint32_t new_axis = axis;
    for (uint32_t i = 0; i < rank; i++) {
        const uint32_t d = order[i];
        store->shape[i] = input->shape[d];
        store->in_strides[i] = input->strides[d];
        store->out_shape[i] = d == axis ? 1 : input->shape[d];
        store->out_strides[i] = output ? output->strides[d] : contiguous_out[d];
        if (d == axis) new_axis = i;
    }
    store->input = cq_tensor{input->ptr, store->shape, store->in_strides, rank, input->elem_size};
    store->output = cq_tensor{output ? output->ptr : nullptr, store->out_shape, store->out_strides, rank, input->elem_size};
    if (!is_contiguous(&store->output)) return axis;
    *in_used = &store->input;
    *out_used = &store->output;
    return new_axis;
}

size_t cq_reduce_workspace_bytes(const cq_tensor* input, uint32_t axis, cq_dtype dtype) {
    if (!tensor_ok(input) || axis >= input->rank || !valid_dtype(dtype)) return 0;
    PermutedReduce store;
    const cq_tensor* out_unused;
    axis = canonical_reduce(input, nullptr, axis, &store, &input, &out_unused);
    uint64_t outer, len, inner;
    reduce_view(input, axis, &outer, &len, &inner);
    if (outer == 0 || inner == 0) return 0;
    return cq::reduce_workspace_bytes(outer, len, inner, dtype);
}

cq_status cq_reduce_max_abs(cq_stream_t stream, const cq_tensor* input, const cq_tensor* output, uint32_t axis,
                            cq_dtype dtype, void* workspace, size_t workspace_bytes) {
    drop_stale_hip_error();
    if (!tensor_ok(input) || !tensor_ok(output) || !valid_dtype(dtype)) return CQ_ERR_INVALID_ARGUMENT;
    if (axis >= input->rank) return CQ_ERR_INVALID_AXIS;
    if (input->elem_size != dtype_size(dtype) || output->elem_size != dtype_size(dtype)) return CQ_ERR_SHAPE_MISMATCH;
    if (output->rank != input->rank) return CQ_ERR_SHAPE_MISMATCH;
    for (uint32_t d = 0; d < input->rank; d++) {
        if (output->shape[d] != (d == axis ? 1 : input->shape[d])) return CQ_ERR_SHAPE_MISMATCH;
        if (input->shape[d] > 0xffffffffull) return CQ_ERR_TOO_LARGE;
    }
    PermutedReduce store;
    axis = canonical_reduce(input, output, axis, &store, &input, &output);
    cq::ReduceArgs a{};
    for (uint32_t d = 0; d < input->rank; d++) {
        a.shape[d] = input->shape[d];
        a.in_strides[d] = input->strides[d];
        a.out_strides[d] = output->strides[d];
    }
    a.input = input->ptr;
    a.output = output->ptr;
    a.workspace = aligned(workspace, 16) ? workspace : nullptr;
    a.workspace_bytes = a.workspace ? workspace_bytes : 0;
    a.rank = input->rank;
    a.axis = axis;
    a.out_contiguous = is_contiguous(output);
    a.in_contiguous = is_contiguous(input);
    a.contiguous = a.in_contiguous && a.out_contiguous;
    reduce_view(input, axis, &a.outer, &a.len, &a.inner);
    if (a.outer == 0 || a.inner == 0) return CQ_OK;  // no outputs
    return hip_status(cq::launch_reduce_max_abs(stream, dtype, a));
}

}  // extern "C"
