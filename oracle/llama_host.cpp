// Test infrastructure only: the reference's own host stack driving a ggml backend.  Built by this directory's Makefile
// (target `host`) against the reference's headers and its libllama / cactus objects compiled where they lie; nothing
// the product ships links or loads it.
//
//   llama_host make-gguf <file>                       a small random-init LLaMA-shaped model written with the reference's
//                                                     gguf writer (cactus/gguf.cpp) and weight quantizers
//                                                     (cactus/ggml-quants.c), types mixed the way a Q4_K_M file mixes them
//   llama_host run <file> <logits.bin> [backend.so] [n_gpu_layers] [mmap]
//                                                     cactus_init_context_c (cactus/cactus_ffi.cpp:43) -> loadModel ->
//                                                     common_init_from_params -> llama_model_load_from_file; then
//                                                     llama_decode on the context for a prompt batch, single tokens and
//                                                     a small batch, logits appended to <logits.bin>; then
//                                                     cactus_bench_c (cactus/cactus_bench.cpp:10) and cactus_completion_c.
//                                                     With backend.so, lm_ggml_backend_load() registers it first, as an
//                                                     application would.
#include "cactus.h"
#include "cactus_ffi.h"
#include "ggml-backend.h"
#include "ggml.h"
#include "gguf.h"
#include "llama-model.h"
#include "llama.h"

#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <random>
#include <string>
#include <vector>

namespace {

constexpr int N_EMBD = 1024, N_HEAD = 8, N_HEAD_KV = 2, N_FF = 2816, N_LAYER = 4, N_VOCAB = 4096, N_CTX_TRAIN = 2048;

std::mt19937 g_rng(20240607);

lm_ggml_tensor *add_weight(lm_ggml_context *ctx, lm_gguf_context *gg, const std::string &name, lm_ggml_type type, int64_t K, int64_t N,
                           float sigma, float mean = 0.0f) {
    lm_ggml_tensor *t = N > 0 ? lm_ggml_new_tensor_2d(ctx, type, K, N) : lm_ggml_new_tensor_1d(ctx, type, K);
    lm_ggml_set_name(t, name.c_str());
    const int64_t rows = N > 0 ? N : 1;
    std::vector<float> w((size_t)K * rows);
    std::normal_distribution<float> dist(mean, sigma);
    for (float &v : w) v = dist(g_rng);
    if (type == LM_GGML_TYPE_F32)
        std::memcpy(t->data, w.data(), w.size() * sizeof(float));
    else
        lm_ggml_quantize_chunk(type, w.data(), t->data, 0, rows, K, nullptr);
    lm_gguf_add_tensor(gg, t);
    return t;
}

int make_gguf(const char *path) {
    lm_ggml_init_params ip = {(size_t)512 << 20, nullptr, false};
    lm_ggml_context *ctx = lm_ggml_init(ip);
    lm_gguf_context *gg = lm_gguf_init_empty();
    lm_gguf_set_val_str(gg, "general.architecture", "llama");
    lm_gguf_set_val_str(gg, "general.name", "random-init llama-shaped test model");
    lm_gguf_set_val_u32(gg, "general.file_type", 15);                        // LLAMA_FTYPE_MOSTLY_Q4_K_M
    lm_gguf_set_val_u32(gg, "llama.context_length", N_CTX_TRAIN);
    lm_gguf_set_val_u32(gg, "llama.embedding_length", N_EMBD);
    lm_gguf_set_val_u32(gg, "llama.block_count", N_LAYER);
    lm_gguf_set_val_u32(gg, "llama.feed_forward_length", N_FF);
    lm_gguf_set_val_u32(gg, "llama.attention.head_count", N_HEAD);
    lm_gguf_set_val_u32(gg, "llama.attention.head_count_kv", N_HEAD_KV);
    lm_gguf_set_val_u32(gg, "llama.rope.dimension_count", N_EMBD / N_HEAD);
    lm_gguf_set_val_f32(gg, "llama.rope.freq_base", 500000.0f);
    lm_gguf_set_val_f32(gg, "llama.attention.layer_norm_rms_epsilon", 1e-5f);
    lm_gguf_set_val_u32(gg, "llama.vocab_size", N_VOCAB);

    // a sentencepiece-style vocabulary: unk / bos / eos, the 256 byte tokens, then made-up pieces
    std::vector<std::string> pieces(N_VOCAB);
    std::vector<float> scores(N_VOCAB);
    std::vector<int32_t> kinds(N_VOCAB);
    for (int i = 0; i < N_VOCAB; ++i) {
        char buf[32];
        if (i == 0) { pieces[i] = "<unk>"; kinds[i] = 2; }
        else if (i == 1) { pieces[i] = "<s>"; kinds[i] = 3; }
        else if (i == 2) { pieces[i] = "</s>"; kinds[i] = 3; }
        else if (i < 259) { std::snprintf(buf, sizeof buf, "<0x%02X>", i - 3); pieces[i] = buf; kinds[i] = 6; }
        else { std::snprintf(buf, sizeof buf, "\xe2\x96\x81w%d", i); pieces[i] = buf; kinds[i] = 1; }
        scores[i] = -(float)i;
    }
    std::vector<const char *> piece_ptrs(N_VOCAB);
    for (int i = 0; i < N_VOCAB; ++i) piece_ptrs[i] = pieces[i].c_str();
    lm_gguf_set_val_str(gg, "tokenizer.ggml.model", "llama");
    lm_gguf_set_arr_str(gg, "tokenizer.ggml.tokens", piece_ptrs.data(), N_VOCAB);
    lm_gguf_set_arr_data(gg, "tokenizer.ggml.scores", LM_GGUF_TYPE_FLOAT32, scores.data(), N_VOCAB);
    lm_gguf_set_arr_data(gg, "tokenizer.ggml.token_type", LM_GGUF_TYPE_INT32, kinds.data(), N_VOCAB);
    lm_gguf_set_val_u32(gg, "tokenizer.ggml.unknown_token_id", 0);
    lm_gguf_set_val_u32(gg, "tokenizer.ggml.bos_token_id", 1);
    lm_gguf_set_val_u32(gg, "tokenizer.ggml.eos_token_id", 2);

    const int kv = N_EMBD / N_HEAD * N_HEAD_KV;
    const float s_embd = 1.0f / std::sqrt((float)N_EMBD), s_ff = 1.0f / std::sqrt((float)N_FF);
    add_weight(ctx, gg, "token_embd.weight", LM_GGML_TYPE_Q4_K, N_EMBD, N_VOCAB, 1.0f);
    for (int l = 0; l < N_LAYER; ++l) {
        const std::string p = "blk." + std::to_string(l) + ".";
        // a Q4_K_M file keeps attn_v and ffn_down of some layers in Q6_K (llama-quant's use_more_bits), the rest in Q4_K
        const lm_ggml_type more = (l % 2 == 0) ? LM_GGML_TYPE_Q6_K : LM_GGML_TYPE_Q4_K;
        add_weight(ctx, gg, p + "attn_norm.weight", LM_GGML_TYPE_F32, N_EMBD, 0, 0.1f, 1.0f);
        add_weight(ctx, gg, p + "attn_q.weight", LM_GGML_TYPE_Q4_K, N_EMBD, N_EMBD, s_embd);
        add_weight(ctx, gg, p + "attn_k.weight", LM_GGML_TYPE_Q4_K, N_EMBD, kv, s_embd);
        add_weight(ctx, gg, p + "attn_v.weight", more, N_EMBD, kv, s_embd);
        add_weight(ctx, gg, p + "attn_output.weight", LM_GGML_TYPE_Q4_K, N_EMBD, N_EMBD, s_embd);
        add_weight(ctx, gg, p + "ffn_norm.weight", LM_GGML_TYPE_F32, N_EMBD, 0, 0.1f, 1.0f);
        add_weight(ctx, gg, p + "ffn_gate.weight", LM_GGML_TYPE_Q4_K, N_EMBD, N_FF, s_embd);
        add_weight(ctx, gg, p + "ffn_up.weight", LM_GGML_TYPE_Q4_K, N_EMBD, N_FF, s_embd);
        add_weight(ctx, gg, p + "ffn_down.weight", more, N_FF, N_EMBD, s_ff);
    }
    add_weight(ctx, gg, "output_norm.weight", LM_GGML_TYPE_F32, N_EMBD, 0, 0.1f, 1.0f);
    add_weight(ctx, gg, "output.weight", LM_GGML_TYPE_Q6_K, N_EMBD, N_VOCAB, s_embd);
    const bool ok = lm_gguf_write_to_file(gg, path, false);
    lm_gguf_free(gg);
    lm_ggml_free(ctx);
    std::printf("make-gguf %s %s\n", path, ok ? "ok" : "FAILED");
    return ok ? 0 : 1;
}

void quiet_log(lm_ggml_log_level level, const char *text, void *) {
    if (level >= LM_GGML_LOG_LEVEL_WARN || std::getenv("LLAMA_HOST_VERBOSE")) std::fputs(text, stderr);
}

bool decode_and_dump(llama_context *lctx, const std::vector<llama_token> &tokens, int pos0, std::FILE *out) {
    const int n = (int)tokens.size();
    llama_batch batch = llama_batch_init(n, 0, 1);
    for (int i = 0; i < n; ++i) {
        batch.token[i] = tokens[i];
        batch.pos[i] = pos0 + i;
        batch.n_seq_id[i] = 1;
        batch.seq_id[i][0] = 0;
        batch.logits[i] = 1;
    }
    batch.n_tokens = n;
    const int rc = llama_decode(lctx, batch);
    if (rc != 0) {
        std::printf("llama_decode failed: %d\n", rc);
        llama_batch_free(batch);
        return false;
    }
    const int n_vocab = llama_vocab_n_tokens(llama_model_get_vocab(llama_get_model(lctx)));
    for (int i = 0; i < n; ++i) std::fwrite(llama_get_logits_ith(lctx, i), sizeof(float), n_vocab, out);
    llama_batch_free(batch);
    return true;
}

int run(int argc, char **argv) {
    const char *model_path = argv[2], *out_path = argv[3];
    const char *backend_path = argc > 4 && argv[4][0] ? argv[4] : nullptr;
    const int n_gpu_layers = argc > 5 ? std::atoi(argv[5]) : 0;
    const bool use_mmap = argc > 6 && std::atoi(argv[6]) != 0;

    llama_log_set(quiet_log, nullptr);
    lm_ggml_backend_reg_t reg = nullptr;
    if (backend_path) {
        reg = lm_ggml_backend_load(backend_path);
        if (!reg) { std::printf("lm_ggml_backend_load(%s) failed\n", backend_path); return 2; }
        std::printf("stat backend_devices %zu\n", lm_ggml_backend_reg_dev_count(reg));
    }
    for (size_t i = 0; i < lm_ggml_backend_dev_count(); ++i) {
        lm_ggml_backend_dev_t dev = lm_ggml_backend_dev_get(i);
        std::printf("device %zu %s type %d\n", i, lm_ggml_backend_dev_name(dev), (int)lm_ggml_backend_dev_type(dev));
    }

    cactus_init_params_c_t ip = {};
    ip.model_path = model_path;
    ip.n_ctx = 512;
    ip.n_batch = 256;
    ip.n_ubatch = 256;
    ip.n_gpu_layers = n_gpu_layers;
    ip.n_threads = 8;
    ip.use_mmap = use_mmap;
    ip.pooling_type = -1;                                 // LLAMA_POOLING_TYPE_UNSPECIFIED
    ip.embd_normalize = 2;
    cactus_context_handle_t handle = cactus_init_context_c(&ip);
    if (!handle) { std::printf("cactus_init_context_c failed\n"); return 3; }
    cactus::cactus_context *cc = reinterpret_cast<cactus::cactus_context *>(handle);

    // where the loader put the weights
    size_t on_device = 0, elsewhere = 0;
    for (const auto &it : cc->model->tensors_by_name) {
        const char *bname = it.second->buffer ? lm_ggml_backend_buffer_name(it.second->buffer) : "(none)";
        if (std::strcmp(bname, "HIP") == 0) ++on_device; else ++elsewhere;
        if (std::getenv("LLAMA_HOST_VERBOSE")) std::printf("tensor %s buffer %s\n", it.first.c_str(), bname);
    }
    std::printf("stat tensors_in_hip_buffers %zu\nstat tensors_elsewhere %zu\n", on_device, elsewhere);

    std::FILE *out = std::fopen(out_path, "wb");
    if (!out) return 4;
    llama_kv_self_clear(cc->ctx);
    std::mt19937 rng(7);
    auto toks = [&](int n) {
        std::vector<llama_token> t(n);
        for (auto &v : t) v = 259 + (llama_token)(rng() % (N_VOCAB - 259));
        return t;
    };
    int pos = 0;
    bool ok = decode_and_dump(cc->ctx, toks(40), pos, out);       // a prompt batch: the GEMM kernels
    pos += 40;
    for (int i = 0; ok && i < 3; ++i, ++pos) ok = decode_and_dump(cc->ctx, toks(1), pos, out);      // decode steps: GEMV
    if (ok) { ok = decode_and_dump(cc->ctx, toks(7), pos, out); pos += 7; }                           // a small batch
    if (ok) { ok = decode_and_dump(cc->ctx, toks(3), pos, out); pos += 3; }
    std::fclose(out);
    if (!ok) return 5;
    std::printf("stat logits_rows %d\n", 40 + 3 + 7 + 3);

    cactus_bench_result_c_t br = cactus_bench_c(handle, 64, 16, 1, 2);
    std::printf("bench model \"%s\" size %lld params %lld pp_avg %.2f tg_avg %.2f\n", br.model_name ? br.model_name : "",
                (long long)br.model_size, (long long)br.model_params, br.pp_avg, br.tg_avg);
    const bool bench_ok = br.pp_avg > 0 && br.tg_avg > 0;
    cactus_free_bench_result_members_c(&br);

    cactus_completion_params_c_t cp = {};
    cp.prompt = "w300 w301 w302";
    cp.n_predict = 8;
    cp.n_threads = 8;
    cp.seed = 1;
    cp.temperature = 0.0;
    cp.top_k = 40;
    cp.top_p = 0.95;
    cp.penalty_last_n = 0;
    cp.penalty_repeat = 1.0;
    cp.ignore_eos = true;
    cactus_completion_result_c_t cr = {};
    const int crc = cactus_completion_c(handle, &cp, &cr);
    std::printf("completion rc %d predicted %d text \"%s\"\n", crc, cr.tokens_predicted, cr.text ? cr.text : "");
    const bool completion_ok = crc == 0 && cr.tokens_predicted >= 1 && cr.text && cr.text[0];
    cactus_free_completion_result_members_c(&cr);

    if (reg) {
        typedef void (*stats_fn)(unsigned long long *, unsigned long long *);
        typedef unsigned long long (*count_fn)(void);
        stats_fn stats = (stats_fn)lm_ggml_backend_reg_get_proc_address(reg, "lm_ggml_backend_hip_get_stats");
        count_fn async_up = (count_fn)lm_ggml_backend_reg_get_proc_address(reg, "lm_ggml_backend_hip_get_async_uploaded");
        count_fn grouped = (count_fn)lm_ggml_backend_reg_get_proc_address(reg, "lm_ggml_backend_hip_get_grouped_matmuls");
        unsigned long long nodes = 0, uploaded = 0;
        if (stats) stats(&nodes, &uploaded);
        std::printf("stat mul_mat_nodes %llu\nstat uploaded_bytes %llu\nstat async_uploaded_bytes %llu\nstat grouped_matmuls %llu\n", nodes,
                    uploaded, async_up ? async_up() : 0ull, grouped ? grouped() : 0ull);
    }
    cactus_free_context_c(handle);
    std::printf("stat bench_ok %d\nstat completion_ok %d\n", (int)bench_ok, (int)completion_ok);
    return bench_ok && completion_ok ? 0 : 6;
}

}  // namespace

int main(int argc, char **argv) {
    if (argc >= 3 && std::strcmp(argv[1], "make-gguf") == 0) return make_gguf(argv[2]);
    if (argc >= 4 && std::strcmp(argv[1], "run") == 0) return run(argc, argv);
    std::fprintf(stderr, "usage: %s make-gguf <file> | run <file> <logits.bin> [backend.so] [n_gpu_layers] [mmap]\n", argv[0]);
    return 64;
}
