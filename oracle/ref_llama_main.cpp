// TEST INFRASTRUCTURE ONLY.  A minimal driver around the reference's own llama.cpp: loads a PowerInfer GGUF, feeds
// the given tokens one llama_decode at a time, then continues greedily, and dumps for every step the token
// consumed, the greedy choice and the full logits.  Built by oracle/Makefile from the reference sources where they
// lie, twice: oracle/_ref/ref_llama is the CPU-only build (used by tests/golden/make_llama_fixture.py), and
// oracle/_ref/ref_llama_gpu is the build with the accelerator hooks enabled (-DGGML_USE_CUBLAS) linked against
// this repository's libpowerinfer_hip.so in place of ggml-cuda.cu -- the reference's own loader, graph builder
// and executor driving the ggml_cuda_* boundary.
//
//   ref_llama <model.gguf> <n_ctx> <n_threads> <n_generate> <out.bin> tok0 tok1 ...
//
// REF_VRAM_GB=<GiB> sets llama_model_params.vram_budget_gb (the accelerator build offloads by budget; the neuron split is
// read from <model.gguf>.generated.gpuidx).  The time of the greedy steps is printed as "decode_ms_per_token <ms>".
//
// With REF_SHIFT_AT=s REF_N_KEEP=k REF_N_DISCARD=d in the environment the driver does, before step s, what the reference's
// examples do when the context is full (examples/main/main.cpp): llama_kv_cache_seq_rm(ctx, 0, k, k + d), then
// llama_kv_cache_seq_shift(ctx, 0, k + d, n_past, -d), and continues at position n_past - d.
#include "llama.h"

#include <chrono>
#include <csignal>
#include <cstdio>
#include <cstdlib>
#include <vector>

#include <execinfo.h>
#include <unistd.h>

// a crash of the host side names its call chain on stderr (the binary is linked with -rdynamic)
static void on_fatal_signal(int sig, siginfo_t * info, void *) {
    void * frames[48];
    const int n = backtrace(frames, 48);
    char msg[96];
    const int len = snprintf(msg, sizeof msg, "ref_llama: fatal signal %d at address %p, call chain:\n", sig, info ? info->si_addr : (void *)0);
    if (write(2, msg, len) < 0) {}
    backtrace_symbols_fd(frames, n, 2);
    signal(sig, SIG_DFL);
    raise(sig);
}

int main(int argc, char ** argv) {
    if (argc < 7) { fprintf(stderr, "usage: %s model n_ctx n_threads n_generate out.bin tok...\n", argv[0]); return 2; }
    const char * path = argv[1];
    const int n_ctx = atoi(argv[2]), n_threads = atoi(argv[3]), n_gen = atoi(argv[4]);
    const char * out_path = argv[5];
    std::vector<llama_token> prompt;
    for (int i = 6; i < argc; ++i) prompt.push_back(atoi(argv[i]));

    struct sigaction sa;
    sa.sa_sigaction = on_fatal_signal;
    sigemptyset(&sa.sa_mask);
    sa.sa_flags = SA_SIGINFO;
    sigaction(SIGSEGV, &sa, NULL);
    sigaction(SIGABRT, &sa, NULL);
    llama_backend_init(false);
    llama_model_params mp = llama_model_default_params();
    mp.n_gpu_layers = 0;                                      // sparse models offload by VRAM budget, not by layer count
    if (getenv("REF_VRAM_GB")) mp.vram_budget_gb = (float)atof(getenv("REF_VRAM_GB"));
    llama_context_params cp = llama_context_default_params();
    cp.seed = 1; cp.n_ctx = n_ctx; cp.n_batch = 512; cp.n_threads = n_threads; cp.n_threads_batch = n_threads;
    // as the reference's examples load (common/common.cpp:966): with the context parameters, so that an accelerator build can
    // reserve the KV cache inside the VRAM budget
    llama_model * model = llama_load_model_from_file_with_context(path, mp, &cp);
    if (!model) { fprintf(stderr, "failed to load %s\n", path); return 1; }
    llama_context * ctx = llama_new_context_with_model(model, cp);
    if (!ctx) { fprintf(stderr, "failed to create context\n"); return 1; }
    const int n_vocab = llama_n_vocab(model);

    FILE * f = fopen(out_path, "wb");
    if (!f) return 1;
    const int n_steps = (int)prompt.size() + n_gen;
    int32_t hdr[2] = { n_steps, n_vocab };
    fwrite(hdr, 4, 2, f);
    const char * e_at = getenv("REF_SHIFT_AT");
    const int shift_at = e_at ? atoi(e_at) : -1;
    const int n_keep = getenv("REF_N_KEEP") ? atoi(getenv("REF_N_KEEP")) : 0, n_discard = getenv("REF_N_DISCARD") ? atoi(getenv("REF_N_DISCARD")) : 0;
    llama_token tok = prompt[0];
    int n_past = 0;
    double gen_ms = 0.0;
    for (int s = 0; s < n_steps; ++s, ++n_past) {
        if (s < (int)prompt.size()) tok = prompt[s];
        const std::chrono::steady_clock::time_point t0 = std::chrono::steady_clock::now();
        if (s == shift_at) {
            llama_kv_cache_seq_rm(ctx, 0, n_keep, n_keep + n_discard);
            llama_kv_cache_seq_shift(ctx, 0, n_keep + n_discard, n_past, -n_discard);
            n_past -= n_discard;
        }
        if (llama_decode(ctx, llama_batch_get_one(&tok, 1, n_past, 0)) != 0) { fprintf(stderr, "llama_decode failed at step %d\n", s); return 1; }
        const float * lg = llama_get_logits(ctx);
        if (s >= (int)prompt.size()) gen_ms += std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - t0).count();
        int best = 0;
        for (int i = 1; i < n_vocab; ++i) if (lg[i] > lg[best]) best = i;
        int32_t rec[2] = { tok, best };
        fwrite(rec, 4, 2, f);
        fwrite(lg, 4, n_vocab, f);
        tok = best;
    }
    fclose(f);
    if (n_gen > 0) printf("decode_ms_per_token %.4f\n", gen_ms / n_gen);
    llama_free(ctx);
    llama_free_model(model);
    llama_backend_free();
    return 0;
}
