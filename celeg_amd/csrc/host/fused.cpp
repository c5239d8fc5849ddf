// Helpers of the fused path for steps of few rows (decode and small portions) and, with the
// tiled products, of many rows.  See parts.hpp.
#include "parts.hpp"

namespace celeg {
namespace fused {

// Whether products of `rows` rows that read a stream of this width take the fused path through
// the tiled products (otherwise they run the library's products with separate norm and activation
// kernels).  The choice is by the sizes of the products, not by the model: Runtime::tiled_max_width
// holds the widest stream for which the tiled products were measured faster.
bool tiled_step(const Runtime& rt, int rows, long long width) {
    return rows > FUSED_MAX_ROWS && width <= rt.tiled_max_width && rt.dtype == DType::BF16 && rt.use_fused;
}

// Whether this step's rows can take the fused path through products with these inner sizes.
bool fused_rows_ok(const Runtime& rt, const StepBatch& batch, std::initializer_list<long long> inner) {
    const int rows = batch.n_tokens;
    long long widest = 0;
    for (long long k : inner) widest = std::max(widest, k);
    if (rows > FUSED_MAX_ROWS)
        // every inner size is also the width of some product's output
        // (the first inner size is the width of the stream)
        return inner.size() > 0 && tiled_step(rt, rows, *inner.begin()) && rt.ops.tiled_linear_ok(rows, 4, inner) &&
               widest <= 64 * TILED_MAX_STAT_BLOCKS;
    if (!(rt.dtype == DType::BF16 && rt.use_fused && rt.ops.fused_linear_ok(rows, inner))) return false;
    int limit = rt.fused_max_rows;
    if (limit < 0) limit = rt.ops.rows_kernel_ok(rows, inner) ? FUSED_MAX_ROWS : FUSED_MAX_ROWS_OLD_KERNEL;
    return rows <= limit;
}

Tensor stream_stats(Runtime& rt, long long width, int rows) {
    if (rows > STAT_COLUMNS)     // a step of many rows: one partial sum per tile of columns
        return rt.ws.buf("stream_stats_many", DType::F32, {rows, TILED_MAX_STAT_BLOCKS});
    // up to one partial sum per 4 columns (the products for few rows use narrow workgroups)
    return rt.ws.buf("stream_stats", DType::F32, {STAT_COLUMNS, (width + 3) / 4});
}

// Room for a bfloat16 operand of the fused products, [rows, width] (up to 16 rows, or sizes the
// kernel for 9 to 64 rows does not take) or the view [rows, width/8, 8] of [width/8, 64, 8]: the
// rows side by side inside every group of 8 values, the layout that the kernel for 9 to 64 rows
// reads whole runs of memory from, where that kernel both reads it and, if a product writes it
// (inner size producer_inner), writes it.
Tensor operand_rows(Runtime& rt, const std::string& name, int rows, long long width,
                    std::initializer_list<long long> producer_inner) {
    if (rows > STAT_COLUMNS) return rt.ws.buf(name + "_many", DType::BF16, {rows, width});
    bool side_by_side = rt.ops.rows_kernel_ok(rows, {width});
    for (long long k : producer_inner) side_by_side = side_by_side && rt.ops.rows_kernel_ok(rows, {k});
    if (side_by_side) {
        Tensor t = rt.ws.buf(name + "_side_by_side", DType::BF16, {width / 8, STAT_COLUMNS, 8});
        Tensor view;
        view.data = t.data;
        view.dtype = DType::BF16;
        view.ndim = 3;
        view.shape[0] = rows;
        view.shape[1] = width / 8;
        view.shape[2] = 8;
        view.stride[0] = 8;
        view.stride[1] = STAT_COLUMNS * 8;
        view.stride[2] = 1;
        return view;
    }
    return rt.ws.buf(name, DType::BF16, {STAT_COLUMNS, width}).rows(0, rows);
}

// The bfloat16 copy of the residual stream that products behind a norm read.
Tensor stream_bf16(Runtime& rt, int rows, long long width) { return operand_rows(rt, "stream_bf16", rows, width, {}); }

// Whether a product of `rows` bfloat16 rows with this inner size takes the form with the norm
// folded into the weights (the kernels for up to 16 and for 9 to 64 rows).
bool sliced(const Runtime& rt, int rows, long long inner) {
    if (rt.ops.rows_kernel_ok(rows, {inner})) return true;
    return rows <= SLICED_MAX_ROWS && rt.ops.use_sliced;
}

namespace {
// w with the norm's weight multiplied into its columns, (x * nw) w^T = x (w * nw)^T, in the
// layout the products for few rows read best.  Made once per (weight, norm) pair and kept.
std::shared_ptr<DeviceTensor> folded_weight(Runtime& rt, const Tensor& w, const Tensor& norm_weight, bool* packed) {
    *packed = w.shape[1] % 32 == 0;
    const auto key = std::make_pair(static_cast<const void*>(w.data), static_cast<const void*>(norm_weight.data));
    auto it = rt.folded_weights.find(key);
    if (it == rt.folded_weights.end()) it = rt.folded_weights.emplace(key, rt.ops.fold_weight(w, &norm_weight, *packed)).first;
    return it->second;
}
std::shared_ptr<DeviceTensor> folded_plain_weight(Runtime& rt, const Tensor& w, const Tensor& norm_weight) {
    const auto key = std::make_pair(static_cast<const void*>(w.data), static_cast<const void*>(norm_weight.data));
    auto it = rt.folded_plain_weights.find(key);
    if (it == rt.folded_plain_weights.end())
        it = rt.folded_plain_weights.emplace(key, rt.ops.fold_weight(w, &norm_weight, false)).first;
    return it->second;
}
// a copy of w in the layout the products for few rows read best; made once
std::shared_ptr<DeviceTensor> packed_weight(Runtime& rt, const Tensor& w) {
    auto it = rt.packed_weights.find(w.data);
    if (it == rt.packed_weights.end()) it = rt.packed_weights.emplace(w.data, rt.ops.fold_weight(w, nullptr, true)).first;
    return it->second;
}
}  // namespace

bool qkv_tail_ok(const Runtime& rt, int rows, long long width) { return tiled_step(rt, rows, width); }

void norm_linear(Runtime& rt, const Tensor& h, const Norm::Foldable& norm, const Tensor& w, const Tensor& out,
                 Epilogue epilogue, const LinearExtras& extras) {
    int blocks = rt.stream_stat_blocks;
    const int T = static_cast<int>(h.shape[0]);
    const long long width = h.shape[1];
    const int M = extras.n_rows >= 0 ? extras.n_rows : T;
    if (tiled_step(rt, T, width)) {
        if (extras.rows || (epilogue != Epilogue::Store && epilogue != Epilogue::Swiglu) || w.dtype != DType::BF16)
            throw KernelError("norm_linear: not a product of the path for many rows");
        Tensor stats = stream_stats(rt, width, T);
        Tensor xb = stream_bf16(rt, T, width);
        if (!(blocks > 0 && blocks <= TILED_MAX_STAT_BLOCKS && rt.stream_has_bf16)) {
            rt.ops.stream_prepare(h, xb, stats);
            rt.stream_stat_blocks = blocks = 1;
            rt.stream_has_bf16 = true;
        }
        rt.ops.tiled_linear(xb, folded_plain_weight(rt, w, norm.weight)->view, out, epilogue, norm.eps, &stats, blocks,
                            extras.bias.defined() ? &extras.bias : nullptr, nullptr, nullptr, extras.qkv);
        return;
    }
    if (extras.qkv) throw KernelError("norm_linear: the q/k/v tail goes with steps of many rows");
    const int streams = epilogue == Epilogue::Swiglu ? 2 : epilogue == Epilogue::Conv ? 3 : 1;
    const bool streamed = rt.ops.rows_kernel_ok(M, {width});
    FusedArgs args;
    args.epilogue = epilogue;
    args.eps = norm.eps;
    args.rows = extras.rows;
    args.n_rows = extras.n_rows;
    args.bias = extras.bias;
    args.conv = extras.conv;
    args.row_best = extras.row_best;
    args.row_best_ld = extras.row_best_ld;
    args.row_best_rows = extras.row_best_rows;
    rt.ops.last_best_parts = 0;
    if (sliced(rt, M, width) && w.dtype == DType::BF16 && (streamed || w.shape[0] / streams <= SLICED_MAX_COLUMNS)) {
        // the stream's bfloat16 copy times the weight with the norm's weight folded in, scaled
        // by the rows' 1/rms at the end
        Tensor stats = stream_stats(rt, width);
        Tensor xb = stream_bf16(rt, T, width);
        if (xb.ndim == 3 && !streamed) {
            // few wanted rows of a step of many: the kernel for few rows reads rows that lie one
            // after the other, so the stream gets such a copy too
            xb = rt.ws.buf("stream_bf16", DType::BF16, {STAT_COLUMNS, width}).rows(0, T);
            rt.ops.stream_prepare(h, xb, stats);
            rt.stream_stat_blocks = blocks = 1;
        } else if (!(blocks > 0 && blocks <= SLICED_MAX_STAT_BLOCKS && rt.stream_has_bf16)) {
            rt.ops.stream_prepare(h, xb, stats);
            rt.stream_stat_blocks = blocks = 1;
            rt.stream_has_bf16 = true;
        }
        bool packed = false;
        auto folded = folded_weight(rt, w, norm.weight, &packed);
        args.stats = stats;
        args.stat_blocks = blocks;
        args.packed = packed;
        rt.ops.fused_linear(xb, folded->view, out, args);
        return;
    }
    args.norm_weight = norm.weight;
    if (blocks) args.stats = stream_stats(rt, width);
    args.stat_blocks = blocks;
    if (w.dtype == DType::BF16 && w.ndim == 2 && w.shape[1] % 32 == 0 && w.shape[1] >= 2048 &&
        w.shape[0] / streams > SLICED_MAX_COLUMNS) {
        // a product of very many long weight rows (the output head of a wide model): a copy of w in
        // blocks of 32 values of k with the rows side by side, which the kernel reads whole kilobytes
        // of; made once and kept (65,536 rows of 2,048 values at 8 rows: 54.6 against 62.4 us; of 1,024
        // values: 29.3 against 29.5, not worth a second copy of the table)
        args.packed = true;
        rt.ops.fused_linear(h, packed_weight(rt, w)->view, out, args);
        return;
    }
    rt.ops.fused_linear(h, w, out, args);
}

void linear_into_stream(Runtime& rt, const Tensor& a, const Tensor& w, const Tensor& h, const Tensor* bias) {
    const int T = static_cast<int>(h.shape[0]);
    const long long width = h.shape[1];
    if (tiled_step(rt, T, width)) {
        Tensor stats = stream_stats(rt, width, T);
        Tensor xb = stream_bf16(rt, T, width);
        rt.ops.tiled_linear(a, w, h, Epilogue::Residual, 0.f, nullptr, 0, bias, &stats, &xb);
        rt.stream_stat_blocks = rt.ops.last_stat_blocks;
        rt.stream_has_bf16 = true;
        return;
    }
    Tensor stats = stream_stats(rt, width);
    const long long inner = a.ndim == 3 ? a.shape[1] * 8 : a.shape[1];
    const bool is_sliced = sliced(rt, T, inner);
    Tensor xb;
    if (is_sliced) {
        xb = stream_bf16(rt, T, width);
        // this product's kernel writes rows one after the other only: the next norm prepares the copy
        if (xb.ndim == 3 && !rt.ops.rows_kernel_ok(T, {inner})) xb = Tensor();
    }
    FusedArgs args;
    args.epilogue = Epilogue::Residual;
    if (bias) args.bias = *bias;
    args.stats_out = stats;
    args.out_bf16 = xb;
    const bool pack = is_sliced && w.shape[1] % 32 == 0;
    args.packed = pack;
    rt.ops.fused_linear(a, pack ? packed_weight(rt, w)->view : w, h, args);
    rt.stream_stat_blocks = rt.ops.last_stat_blocks;
    rt.stream_has_bf16 = xb.defined();
}

}  // namespace fused
}  // namespace celeg
