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
// With REF_SCRIPT=<file> the tokens on the command line are ignored and the file is executed line by line instead:
//     decode n  tok pos seq  tok pos seq ...   one llama_decode of n entries (token, position, sequence id); the logits of every entry
//                                              are appended to <out.bin> in entry order
//     rm seq p0 p1 | shift seq p0 p1 delta | cp src dst p0 p1      llama_kv_cache_seq_rm / _seq_shift / _seq_cp
// <out.bin> then starts with {number of logits rows, n_vocab}.
//
// REF_VRAM_GB=<GiB> sets llama_model_params.vram_budget_gb (the accelerator build offloads by budget; the neuron split is
// read from <model.gguf>.generated.gpuidx).  The time of the greedy steps is printed as "decode_ms_per_token <ms>".
//
// REF_ONE_CORE=1 binds the process, and with it every thread it starts, to the core it is on.  The reference's CPU share of the
// down projection lets each worker add its partial sum into the result without a lock (ggml.c:14436-14452); with its workers
// on one core they run one at a time and change over where they yield between graph nodes (ggml.c:16946), so two of them are
// never inside that addition together and a multi-threaded run repeats the single-threaded numbers.
//
// With REF_SHIFT_AT=s REF_N_KEEP=k REF_N_DISCARD=d in the environment the driver does, before step s, what the reference's
// examples do when the context is full (examples/main/main.cpp): llama_kv_cache_seq_rm(ctx, 0, k, k + d), then
// llama_kv_cache_seq_shift(ctx, 0, k + d, n_past, -d), and continues at position n_past - d.
#include "llama.h"

#include <chrono>
#include <csignal>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>

#include <execinfo.h>
#include <sched.h>
#include <unistd.h>
#ifdef GGML_USE_CUBLAS
extern "C" void pi_ggml_backend_get_stats(int64_t * out);      // libpowerinfer_hip.so: four counters
#endif

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
    if (getenv("REF_ONE_CORE") && atoi(getenv("REF_ONE_CORE"))) {
        cpu_set_t one;
        CPU_ZERO(&one);
        CPU_SET(sched_getcpu(), &one);
        if (sched_setaffinity(0, sizeof one, &one) != 0) { perror("sched_setaffinity"); return 2; }
    }
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
    if (const char * script = getenv("REF_SCRIPT")) {
        FILE * sf = fopen(script, "r");
        if (!sf) { fprintf(stderr, "cannot open %s\n", script); return 1; }
        int32_t hdr2[2] = { 0, n_vocab };
        fwrite(hdr2, 4, 2, f);
        char op[16];
        int n_rows = 0;
        while (fscanf(sf, "%15s", op) == 1) {
            if (!strcmp(op, "decode")) {
                int n = 0;
                if (fscanf(sf, "%d", &n) != 1 || n <= 0) return 1;
                llama_batch b = llama_batch_init(n, 0, 1);
                b.n_tokens = n;
                for (int i = 0; i < n; ++i) {
                    int tok_i, pos_i, seq_i;
                    if (fscanf(sf, "%d %d %d", &tok_i, &pos_i, &seq_i) != 3) return 1;
                    b.token[i] = tok_i; b.pos[i] = pos_i; b.n_seq_id[i] = 1; b.seq_id[i][0] = seq_i; b.logits[i] = 1;
                }
                if (llama_decode(ctx, b) != 0) { fprintf(stderr, "llama_decode failed\n"); return 1; }
                for (int i = 0; i < n; ++i) { fwrite(llama_get_logits_ith(ctx, i), 4, n_vocab, f); ++n_rows; }
                llama_batch_free(b);
            } else if (!strcmp(op, "rm")) {
                int q, p0, p1; if (fscanf(sf, "%d %d %d", &q, &p0, &p1) != 3) return 1;
                llama_kv_cache_seq_rm(ctx, q, p0, p1);
            } else if (!strcmp(op, "shift")) {
                int q, p0, p1, dl; if (fscanf(sf, "%d %d %d %d", &q, &p0, &p1, &dl) != 4) return 1;
                llama_kv_cache_seq_shift(ctx, q, p0, p1, dl);
            } else if (!strcmp(op, "cp")) {
                int a, b2, p0, p1; if (fscanf(sf, "%d %d %d %d", &a, &b2, &p0, &p1) != 4) return 1;
                llama_kv_cache_seq_cp(ctx, a, b2, p0, p1);
            } else { fprintf(stderr, "unknown script line %s\n", op); return 1; }
        }
        fclose(sf);
        hdr2[0] = n_rows;
        fseek(f, 0, SEEK_SET);
        fwrite(hdr2, 4, 2, f);
        fclose(f);
        llama_free(ctx);
        llama_free_model(model);
        llama_backend_free();
        return 0;
    }
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
#ifdef GGML_USE_CUBLAS
    {   // what the backend library's window of deferred nodes did over the run (its own counters, not part of the reference's interface)
        int64_t st[4] = {0, 0, 0, 0};
        pi_ggml_backend_get_stats(st);
        printf("backend_stats deferred %lld flushed %lld ffn_fused %lld attn_fused %lld\n", (long long)st[0], (long long)st[1], (long long)st[2], (long long)st[3]);
    }
#endif
    llama_free(ctx);
    llama_free_model(model);
    llama_backend_free();
    return 0;
}
