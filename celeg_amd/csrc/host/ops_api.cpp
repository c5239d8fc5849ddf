// The kernels' dispatcher alone, by JSON calls: `celeg_ops_call(handle, op, arguments)` calls the
// method of Ops that `op` names, the one the parts call, with its shape checks and its choice of
// kernel.  Tensors travel as {"data": address, "dtype": name, "shape": [...], "stride": [...]}
// (strides in elements), a step's arrays and a cache view as objects of addresses and counts.  It
// is what the tests of single kernels drive, so that no second copy of the checks and choices
// exists outside this library.
#include "../include/celeg_amd.h"

#include <map>
#include <mutex>
#include <vector>

#include "ops.hpp"

using namespace celeg;

extern "C" void celeg_set_last_error_(const char* message);

struct celeg_ops {
    Ops ops{nullptr};
    Workspace ws;
    std::string answer;
    // the frequencies last seen at an address: the dispatcher keeps its tables of cosines and sines
    // by that address, and a caller's tensors are freed and their addresses used again
    std::map<const void*, std::vector<float>> frequencies;
};

namespace {

template <typename T>
T* address(const Json& j) {
    if (j.is_null()) return nullptr;
    return reinterpret_cast<T*>(static_cast<uintptr_t>(j.as_int()));
}
template <typename T>
T* address(const Json& args, const char* key) {
    return args.contains(key) ? address<T>(args[key]) : nullptr;
}

Tensor tensor_of(const Json& j) {
    Tensor t;
    if (j.is_null()) return t;
    t.data = address<void>(j["data"]);
    const std::string dtype = j["dtype"].as_string();
    t.dtype = dtype == "int32" ? DType::I32 : dtype == "uint8" ? DType::U8 : parse_dtype(dtype);
    const auto& shape = j["shape"].items();
    const auto& stride = j["stride"].items();
    if (shape.size() > 4 || stride.size() != shape.size()) throw KernelError("a tensor has up to four dimensions, with a stride each");
    t.ndim = static_cast<int>(shape.size());
    for (int i = 0; i < t.ndim; ++i) {
        t.shape[i] = shape[static_cast<size_t>(i)].as_int();
        t.stride[i] = stride[static_cast<size_t>(i)].as_int();
    }
    return t;
}

struct Maybe {
    Tensor t;
    const Tensor* ptr() const { return t.defined() ? &t : nullptr; }
};
Maybe maybe(const Json& args, const char* key) {
    Maybe m;
    if (args.contains(key)) m.t = tensor_of(args[key]);
    return m;
}
Tensor must(const Json& args, const char* key) {
    if (!args.contains(key) || args[key].is_null()) throw KernelError(std::string(key) + " is missing");
    return tensor_of(args[key]);
}

StepBatch batch_of(const Json& j) {
    StepBatch b;
    b.n_tokens = static_cast<int>(j["n_tokens"].as_int());
    b.n_seqs = static_cast<int>(j["n_seqs"].as_int());
    b.n_logit_rows = static_cast<int>(j.get_int("n_logit_rows", 0));
    b.n_real_seqs = static_cast<int>(j.get_int("n_real_seqs", b.n_seqs));
    b.max_seg_len = static_cast<int>(j.get_int("max_seg_len", 0));
    b.max_context_len = static_cast<int>(j.get_int("max_context_len", 0));
    b.context_bound = static_cast<int>(j.get_int("context_bound", 0));
    b.decode_only = j.get_bool("decode_only", false);
    b.single_rows = static_cast<int>(j.get_int("single_rows", 0));
    b.token_ids = address<int>(j, "token_ids");
    b.positions = address<int>(j, "positions");
    b.token_seq = address<int>(j, "token_seq");
    b.token_slot = address<int>(j, "token_slot");
    b.cu_seqlens = address<int>(j, "cu_seqlens");
    b.seq_slot = address<int>(j, "seq_slot");
    b.seq_start = address<int>(j, "seq_start");
    b.logit_rows = address<int>(j, "logit_rows");
    return b;
}

KVView kv_of(const Json& j) {
    KVView kv;
    kv.k = address<void>(j["k"]);
    kv.v = address<void>(j["v"]);
    kv.dtype = parse_dtype(j["dtype"].as_string());
    kv.layer = static_cast<int>(j["layer"].as_int());
    kv.n_layers = static_cast<int>(j["n_layers"].as_int());
    kv.table = address<int>(j["table"]);
    kv.table_stride = static_cast<int>(j["table_stride"].as_int());
    kv.table_rows = static_cast<int>(j["table_rows"].as_int());
    kv.page_tokens = static_cast<int>(j["page_tokens"].as_int());
    kv.kv_heads = static_cast<int>(j["kv_heads"].as_int());
    kv.head_dim = static_cast<int>(j["head_dim"].as_int());
    kv.v_head_dim = static_cast<int>(j.get_int("v_head_dim", kv.head_dim));
    kv.n_pages = static_cast<int>(j.get_int("n_pages", 0));
    kv.group = static_cast<int>(j.get_int("group", 0));
    return kv;
}

// Before a call that brings rotation frequencies: if the address held other frequencies (or
// another number of them) when a table was last made for it, that table is set aside.
void refresh_frequencies(celeg_ops& h, const Tensor* inv_freq) {
    if (!inv_freq || !inv_freq->defined() || inv_freq->dtype != DType::F32) return;
    hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(h.ops.stream, &capturing) != hipSuccess) (void)hipGetLastError();
    if (capturing != hipStreamCaptureStatusNone) return;      // (a recording runs what was run before it)
    std::vector<float> now(static_cast<size_t>(inv_freq->numel()));
    CELEG_HIP(hipStreamSynchronize(h.ops.stream));
    CELEG_HIP(hipMemcpy(now.data(), inv_freq->data, now.size() * sizeof(float), hipMemcpyDeviceToHost));
    auto it = h.frequencies.find(inv_freq->data);
    if (it != h.frequencies.end() && it->second == now) return;
    h.ops.forget_rope_tables(inv_freq->data);
    h.frequencies[inv_freq->data] = std::move(now);
}

Epilogue epilogue_of(const std::string& name) {
    if (name == "store") return Epilogue::Store;
    if (name == "store_f32") return Epilogue::StoreF32;
    if (name == "residual") return Epilogue::Residual;
    if (name == "swiglu") return Epilogue::Swiglu;
    if (name == "conv") return Epilogue::Conv;
    throw KernelError("unknown epilogue '" + name + "'");
}

std::vector<long long> ints_of(const Json& j) {
    std::vector<long long> out;
    for (const Json& v : j.items()) out.push_back(v.as_int());
    return out;
}
// (the dispatcher's predicates take lists of inner sizes)
bool all_sizes(const std::vector<long long>& inner, const std::function<bool(long long)>& ok) {
    for (long long k : inner)
        if (!ok(k)) return false;
    return true;
}

void set_knobs(Ops& ops, const Json& knobs) {
    for (const auto& m : knobs.members()) {
        const std::string& name = m.first;
        const long long v = m.second.is_bool() ? (m.second.as_bool() ? 1 : 0) : m.second.as_int();
        if (name == "attention_decode_whole") ops.attention_decode_whole = static_cast<int>(v);
        else if (name == "use_blaslt") ops.use_blaslt = v != 0;
        else if (name == "attention_rows_per_tile") ops.attention_rows_per_tile = static_cast<int>(v);
        else if (name == "attention_rows_form") ops.attention_rows_form = static_cast<int>(v);
        else if (name == "decode_parts_few") ops.decode_part_thresholds[0] = static_cast<int>(v);
        else if (name == "decode_parts_some") ops.decode_part_thresholds[1] = static_cast<int>(v);
        else if (name == "attention_general") ops.attention_general = v != 0;
        else if (name == "use_rope_table") ops.use_rope_table = v != 0;
        else if (name == "use_argmax_parts") ops.use_argmax_parts = v != 0;
        else if (name == "use_head_argmax") ops.use_head_argmax = v != 0;
        else if (name == "decode_parts_fill") ops.decode_parts_fill = v != 0;
        else if (name == "use_sliced") ops.use_sliced = v != 0;
        else if (name == "use_rows_kernel") ops.use_rows_kernel = v != 0;
        else if (name == "use_tiles") ops.use_tiles = v != 0;
        else if (name == "use_qkv_tail") ops.use_qkv_tail = v != 0;
        else if (name == "use_fresh_decode") ops.use_fresh_decode = v != 0;
        else if (name == "rows_kernel_min_rows") ops.rows_kernel_min_rows = static_cast<int>(v);
        else if (name == "tiles_min_rows") ops.tiles_min_rows = static_cast<int>(v);
        else if (name == "fused_linear_shape") ops.fused_linear_shape = static_cast<int>(v);
        else throw KernelError("unknown knob '" + name + "'");
    }
}

Json call(celeg_ops& h, const std::string& op, const Json& a) {
    Ops& ops = h.ops;
    Json out = Json::object();
    if (op == "embed") {
        ops.embed(must(a, "table"), address<int>(a, "token_ids"), must(a, "out"));
    } else if (op == "rmsnorm") {
        const Maybe delta = maybe(a, "delta");
        ops.rmsnorm(must(a, "x"), must(a, "weight"), static_cast<float>(a["eps"].as_double()), must(a, "out"), delta.ptr(),
                    address<int>(a, "rows"));
    } else if (op == "swiglu") {
        ops.swiglu(must(a, "gate_up"), must(a, "out"));
    } else if (op == "add_bias") {
        ops.add_bias(must(a, "x"), must(a, "bias"));
    } else if (op == "cast") {
        ops.cast(must(a, "src"), must(a, "dst"));
    } else if (op == "apply_table_updates") {
        const Tensor table = must(a, "table");
        ops.apply_table_updates(table.as<int>(), static_cast<int>(table.shape[1]), static_cast<int>(table.shape[0]),
                                address<int>(a, "updates"), static_cast<int>(a["capacity"].as_int()));
    } else if (op == "step_prologue") {
        const Tensor table = must(a, "table");
        ops.step_prologue(table.as<int>(), static_cast<int>(table.shape[1]), static_cast<int>(table.shape[0]),
                          address<int>(a, "updates"), static_cast<int>(a["capacity"].as_int()), address<int>(a, "token_ids"),
                          address<int>(a, "token_slot"), address<int>(a, "last_tokens"), static_cast<int>(a["n"].as_int()));
    } else if (op == "resolve_tokens") {
        ops.resolve_tokens(address<int>(a, "token_ids"), address<int>(a, "token_slot"), address<int>(a, "last_tokens"),
                           static_cast<int>(a["n"].as_int()));
    } else if (op == "linear") {
        const Maybe bias = maybe(a, "bias");
        ops.linear(must(a, "x"), must(a, "w"), must(a, "out"), bias.ptr(), h.ws);
    } else if (op == "short_conv") {
        const Maybe bias = maybe(a, "bias");
        ops.short_conv(must(a, "bcx"), must(a, "weight"), bias.ptr(), must(a, "state"), must(a, "out"), batch_of(a["batch"]));
    } else if (op == "qk_norm_rope_store") {
        const Maybe k = maybe(a, "k"), v = maybe(a, "v"), qw = maybe(a, "q_weight"), kw = maybe(a, "k_weight"),
                    inv_freq = maybe(a, "inv_freq");
        refresh_frequencies(h, inv_freq.ptr());
        ops.qk_norm_rope_store(must(a, "q"), k.ptr(), v.ptr(), qw.ptr(), kw.ptr(), static_cast<float>(a["eps"].as_double()),
                               inv_freq.ptr(), static_cast<int>(a["rotary_dim"].as_int()), static_cast<int>(a.get_int("pairing", 0)),
                               static_cast<int>(a["heads"].as_int()), static_cast<int>(a["kv_heads"].as_int()),
                               static_cast<int>(a["head_dim"].as_int()), batch_of(a["batch"]), kv_of(a["kv"]));
    } else if (op == "paged_attention" || op == "attention_fresh_ok") {
        const int heads = static_cast<int>(a["heads"].as_int()), head_dim = static_cast<int>(a["head_dim"].as_int());
        const StepBatch batch = batch_of(a["batch"]);
        const KVView kv = kv_of(a["kv"]);
        Maybe fk, fv, fqw, fkw, finv;
        FreshKV fresh;
        const bool has_fresh = a.contains("fresh") && !a["fresh"].is_null();
        if (has_fresh) {
            const Json& f = a["fresh"];
            fk = maybe(f, "k"), fv = maybe(f, "v"), fqw = maybe(f, "q_weight"), fkw = maybe(f, "k_weight"), finv = maybe(f, "inv_freq");
            fresh.k = fk.ptr();
            fresh.v = fv.ptr();
            fresh.q_weight = fqw.ptr();
            fresh.k_weight = fkw.ptr();
            fresh.eps = static_cast<float>(f.get_double("eps", 0.0));
            fresh.inv_freq = finv.ptr();
            refresh_frequencies(h, fresh.inv_freq);
        }
        if (op == "attention_fresh_ok") {
            out.set("ok", ops.attention_fresh_ok(heads, head_dim, fresh.inv_freq, static_cast<int>(a.get_int("rotary_dim", head_dim)),
                                                 static_cast<int>(a.get_int("pairing", 0)), batch, kv,
                                                 parse_dtype(a.get_string("dtype", "bfloat16"))));
        } else {
            ops.paged_attention(must(a, "q"), must(a, "out"), heads, static_cast<int>(a["kv_heads"].as_int()), head_dim,
                                static_cast<float>(a["scale"].as_double()), static_cast<int>(a.get_int("window", 0)), batch, kv,
                                h.ws, has_fresh ? &fresh : nullptr);
        }
    } else if (op == "sample") {
        const Tensor logits = must(a, "logits");
        HeadBest best;
        best.best = address<unsigned long long>(a, "row_best");
        if (best.best) {
            best.logits = logits.data;
            best.ld = static_cast<int>(a.get_int("row_best_ld", 0));
            best.parts = static_cast<int>(a.get_int("row_best_parts", 0));
            best.rows = static_cast<int>(logits.shape[0]);
            best.cols = static_cast<int>(a.get_int("row_best_cols", 0));
        }
        ops.sample(logits, address<float>(a, "fparams"), address<int>(a, "iparams"), address<uint8_t>(a, "seen"),
                   static_cast<size_t>(a.get_int("seen_stride", 0)), address<int>(a, "out_tokens"), address<int>(a, "last_tokens"),
                   a.get_bool("all_greedy", false), h.ws, best.best ? &best : nullptr, a.get_bool("penalised", false));
    } else if (op == "mark_seen") {
        const Tensor seen = must(a, "seen");
        ops.mark_seen(seen.as<uint8_t>(), static_cast<size_t>(seen.stride[0]), static_cast<int>(seen.shape[0]),
                      static_cast<int>(seen.shape[1]), address<int>(a, "token_ids"), address<int>(a, "token_slot"),
                      static_cast<int>(a["n"].as_int()));
    } else if (op == "fused_linear_ok") {
        const int rows = static_cast<int>(a["rows"].as_int());
        out.set("ok", all_sizes(ints_of(a["inner"]), [&](long long k) { return ops.fused_linear_ok(rows, {k}); }));
    } else if (op == "rows_kernel_ok") {
        const int rows = static_cast<int>(a["rows"].as_int());
        out.set("ok", all_sizes(ints_of(a["inner"]), [&](long long k) { return ops.rows_kernel_ok(rows, {k}); }));
    } else if (op == "tiled_linear_ok") {
        const int rows = static_cast<int>(a["rows"].as_int()), n = static_cast<int>(a["n"].as_int());
        out.set("ok", all_sizes(ints_of(a["inner"]), [&](long long k) { return ops.tiled_linear_ok(rows, n, {k}); }));
    } else if (op == "residual_stat_blocks") {
        out.set("blocks", ops.residual_stat_blocks(static_cast<int>(a["rows"].as_int()), static_cast<int>(a["n"].as_int()),
                                                   static_cast<int>(a["k"].as_int())));
    } else if (op == "tiled_stat_blocks") {
        out.set("blocks", ops.tiled_stat_blocks(static_cast<int>(a["rows"].as_int()), static_cast<int>(a["n"].as_int()),
                                                static_cast<int>(a["k"].as_int())));
    } else if (op == "stream_prepare") {
        ops.stream_prepare(must(a, "h"), must(a, "xb"), must(a, "stats"));
    } else if (op == "embed_stream") {
        ops.embed_stream(must(a, "table"), address<int>(a, "token_ids"), must(a, "out"), must(a, "xb"), must(a, "stats"));
    } else if (op == "embed_stats") {
        ops.embed_stats(must(a, "table"), address<int>(a, "token_ids"), must(a, "out"), must(a, "stats"));
    } else if (op == "fused_linear") {
        FusedArgs args;
        args.epilogue = epilogue_of(a.get_string("epilogue", "store"));
        args.norm_weight = maybe(a, "norm_weight").t;
        args.eps = static_cast<float>(a.get_double("eps", 0.0));
        args.stats = maybe(a, "stats").t;
        args.stat_blocks = static_cast<int>(a.get_int("stat_blocks", 0));
        args.rows = address<int>(a, "rows");
        args.n_rows = static_cast<int>(a.get_int("n_rows", -1));
        args.bias = maybe(a, "bias").t;
        args.stats_out = maybe(a, "stats_out").t;
        args.out_bf16 = maybe(a, "out_bf16").t;
        args.packed = a.get_bool("packed", false);
        ConvOperands conv;
        if (a.contains("conv") && !a["conv"].is_null()) {
            const Json& c = a["conv"];
            conv.taps = must(c, "taps");
            conv.bias = maybe(c, "bias").t;
            conv.state = must(c, "state");
            conv.seq_slot = address<int>(c, "seq_slot");
            args.conv = &conv;
        }
        args.row_best = address<unsigned long long>(a, "row_best");
        args.row_best_ld = static_cast<int>(a.get_int("row_best_ld", 0));
        args.row_best_rows = static_cast<int>(a.get_int("row_best_rows", 0));
        ops.fused_linear(must(a, "a"), must(a, "w"), must(a, "out"), args);
    } else if (op == "tiled_linear") {
        const Maybe stats = maybe(a, "stats"), bias = maybe(a, "bias"), stats_out = maybe(a, "stats_out"), out_bf16 = maybe(a, "out_bf16");
        Maybe qw, kw, inv_freq;
        QkvTail tail;
        StepBatch batch;
        KVView kv;
        const bool has_tail = a.contains("qkv") && !a["qkv"].is_null();
        if (has_tail) {
            const Json& q = a["qkv"];
            qw = maybe(q, "q_weight"), kw = maybe(q, "k_weight"), inv_freq = maybe(q, "inv_freq");
            batch = batch_of(q["batch"]);
            kv = kv_of(q["kv"]);
            tail.heads = static_cast<int>(q["heads"].as_int());
            tail.kv_heads = static_cast<int>(q["kv_heads"].as_int());
            tail.head_dim = static_cast<int>(q.get_int("head_dim", 64));
            tail.q_weight = qw.ptr();
            tail.k_weight = kw.ptr();
            tail.eps = static_cast<float>(q.get_double("eps", 0.0));
            tail.inv_freq = inv_freq.ptr();
            refresh_frequencies(h, tail.inv_freq);
            tail.batch = &batch;
            tail.kv = &kv;
        }
        ops.tiled_linear(must(a, "a"), must(a, "w"), must(a, "out"), epilogue_of(a.get_string("epilogue", "store")),
                         static_cast<float>(a.get_double("eps", 0.0)), stats.ptr(), static_cast<int>(a.get_int("stat_blocks", 0)),
                         bias.ptr(), stats_out.ptr(), out_bf16.ptr(), has_tail ? &tail : nullptr);
    } else if (op == "tiled_qkv_ok") {
        const Maybe inv_freq = maybe(a, "inv_freq");
        const int head_dim = static_cast<int>(a["head_dim"].as_int());
        out.set("ok", ops.tiled_qkv_ok(head_dim, inv_freq.ptr(), static_cast<int>(a.get_int("rotary_dim", head_dim)),
                                       static_cast<int>(a.get_int("pairing", 0)), kv_of(a["kv"])));
    } else if (op == "fold_weight") {
        // the re-laid weight goes to `out`, which the caller owns
        const Maybe scale = maybe(a, "scale");
        const Tensor dst = must(a, "out");
        auto made = ops.fold_weight(must(a, "w"), scale.ptr(), a.get_bool("packed", false));
        if (dst.dtype != made->view.dtype || dst.numel() != made->view.numel() || !dst.contiguous())
            throw KernelError("fold_weight: out must be contiguous bfloat16 of the weight's size");
        CELEG_HIP(hipMemcpyAsync(dst.data, made->view.data, made->view.bytes(), hipMemcpyDeviceToDevice, ops.stream));
        CELEG_HIP(hipStreamSynchronize(ops.stream));     // (`made` goes away)
    } else if (op == "state") {
        // nothing to run: the knobs were set, the answer below tells the counters
    } else {
        throw KernelError("unknown operation '" + op + "'");
    }
    out.set("last_stat_blocks", ops.last_stat_blocks);
    out.set("last_best_parts", ops.last_best_parts);
    out.set("last_best_cols", ops.last_best_cols);
    if (op == "state") out.set("paths", ops.paths_json());
    return out;
}

}  // namespace

extern "C" {

celeg_status celeg_ops_create(celeg_ops** out) {
    if (!out) return CELEG_INVALID_ARGUMENT;
    *out = nullptr;
    try {
        int count = 0;
        if (hipGetDeviceCount(&count) != hipSuccess || count <= 0) {
            (void)hipGetLastError();
            throw KernelError("celeg_amd needs a GPU: no HIP device is visible and there is no CPU path");
        }
        *out = new celeg_ops();
        return CELEG_OK;
    } catch (const std::exception& e) {
        celeg_set_last_error_(e.what());
        return CELEG_ERROR;
    }
}

void celeg_ops_destroy(celeg_ops* ops) { delete ops; }

const char* celeg_ops_call(celeg_ops* ops, const char* op, const char* args_json, void* stream) {
    if (!ops || !op || !args_json) {
        celeg_set_last_error_("celeg_ops_call: ops, op and args_json must not be null");
        return nullptr;
    }
    try {
        const Json args = Json::parse(args_json);
        ops->ops.stream = static_cast<hipStream_t>(stream);
        if (args.contains("knobs")) set_knobs(ops->ops, args["knobs"]);
        ops->answer = call(*ops, op, args).dump();
        return ops->answer.c_str();
    } catch (const std::exception& e) {
        celeg_set_last_error_(e.what());
        return nullptr;
    }
}

}  // extern "C"
