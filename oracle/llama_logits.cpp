// Test infrastructure (not shipped): drives the reference's own model runtime (libllama, built from the reference
// sources by this directory's Makefile) through its public API and dumps logits, so that a test can compare the
// reference CPU backend with the plug-in, and the plug-in's fused graph execution with its node-by-node execution,
// on the same synthetic model and token ids.
//
//   llama_logits <model.gguf> <n_gpu_layers> <n_prompt> <n_decode> <out.bin> [<type_k> <type_v>]
//
// type_k / type_v: f16 (default), q8_0 or q4_0 - the KV cache types of llama.cpp's -ctk / -ctv.
// LLAMA_LOGITS_NO_MMAP=1 in the environment loads the file with read() instead of mmap (llama.cpp's --no-mmap), which is the
// path that uploads through pinned buffers, set_tensor_async and events when the device offers them.
//
// LLAMA_LOGITS_SHIFT=<n> drops the first n cells of the sequence after the prompt and moves the rest down by n (what llama-cli's
// context shift does: llama_kv_cache_seq_rm + llama_kv_cache_seq_add + llama_kv_cache_update, which runs the K-shift graph -
// ROPE in place on an f16 cache, cast to f32 / ROPE / copy back on a quantized one) before the decoded tokens.
// LLAMA_LOGITS_DEFRAG=<n> instead removes n cells from the middle of the sequence after the prompt and asks for a defragmentation
// (llama_kv_cache_defrag + llama_kv_cache_update: build_defrag's row copies inside the K and V caches).
//
// LLAMA_LOGITS_CTX=<n> sets the context size (default 1024); a prompt longer than the batch size of 512 is fed 512 tokens at a time.
//
// Tokens are (7 i + 3) mod n_vocab.  Output: float32 rows of n_vocab logits, one for the last prompt token and one per
// decoded token (the token ids are fixed, the logits are not fed back).
#include "ggml-backend.h"
#include "llama.h"

#include <cstdio>
#include <cstdlib>
#include <string>
#include <vector>

int main(int argc, char ** argv) {
    if (argc != 6 && argc != 8) {
        fprintf(stderr, "usage: %s model.gguf n_gpu_layers n_prompt n_decode out.bin [type_k type_v]\n", argv[0]);
        return 2;
    }
    auto cache_type = [](const char * name) {
        const std::string s = name;
        return s == "q8_0" ? GGML_TYPE_Q8_0 : s == "q4_0" ? GGML_TYPE_Q4_0 : GGML_TYPE_F16;
    };
    const int ngl = atoi(argv[2]), n_prompt = atoi(argv[3]), n_decode = atoi(argv[4]);
    ggml_backend_load_all();   // honours GGML_BACKEND_PATH, like the reference's example programs
    llama_backend_init();
    llama_model_params mp = llama_model_default_params();
    mp.n_gpu_layers = ngl;
    if (getenv("LLAMA_LOGITS_NO_MMAP")) mp.use_mmap = false;
    llama_model * model = llama_model_load_from_file(argv[1], mp);
    if (!model) return 1;
    llama_context_params cp = llama_context_default_params();
    cp.n_ctx = getenv("LLAMA_LOGITS_CTX") ? atoi(getenv("LLAMA_LOGITS_CTX")) : 1024;
    cp.n_batch = 512;
    cp.n_ubatch = 512;
    cp.flash_attn = true;
    if (argc == 8) {
        cp.type_k = cache_type(argv[6]);
        cp.type_v = cache_type(argv[7]);
    }
    cp.n_threads = 8;
    cp.n_threads_batch = 8;
    llama_context * ctx = llama_init_from_model(model, cp);
    if (!ctx) return 1;
    const int n_vocab = llama_vocab_n_tokens(llama_model_get_vocab(model));
    FILE * f = fopen(argv[5], "wb");
    if (!f) return 1;
    std::vector<llama_token> toks(n_prompt);
    for (int i = 0; i < n_prompt; i++) toks[i] = (7 * i + 3) % n_vocab;
    for (int i0 = 0; i0 < n_prompt; i0 += 512) {
        const int n = n_prompt - i0 < 512 ? n_prompt - i0 : 512;
        if (llama_decode(ctx, llama_batch_get_one(toks.data() + i0, n)) != 0) return 1;
    }
    fwrite(llama_get_logits_ith(ctx, -1), sizeof(float), n_vocab, f);
    if (const char * sh = getenv("LLAMA_LOGITS_SHIFT")) {
        const int n_discard = atoi(sh);
        if (n_discard <= 0 || n_discard >= n_prompt) return 2;
        llama_kv_cache_seq_rm(ctx, 0, 0, n_discard);
        llama_kv_cache_seq_add(ctx, 0, n_discard, n_prompt, -n_discard);
        llama_kv_cache_update(ctx);
    }
    if (const char * df = getenv("LLAMA_LOGITS_DEFRAG")) {
        const int n_hole = atoi(df);
        if (n_hole <= 0 || 2 * n_hole >= n_prompt) return 2;
        llama_kv_cache_seq_rm(ctx, 0, n_hole, 2 * n_hole);
        llama_kv_cache_defrag(ctx);
        llama_kv_cache_update(ctx);
    }
    for (int i = 0; i < n_decode; i++) {
        llama_token t = (7 * (n_prompt + i) + 3) % n_vocab;
        if (llama_decode(ctx, llama_batch_get_one(&t, 1)) != 0) return 1;
        fwrite(llama_get_logits_ith(ctx, -1), sizeof(float), n_vocab, f);
    }
    fclose(f);
    llama_free(ctx);
    llama_model_free(model);
    return 0;
}
