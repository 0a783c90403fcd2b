// run_sft — the reference's `--mode sft` driver (main.c:204-278 options, :286-324 model-type detection, :366-524 loop)
// over the HIP library: load a checkpoint (safetensors file / shard directory or GGUF), build the SFT state (LoRA or
// full-parameter), feed batches from a pre-tokenized int32 file (or the reference's synthetic fallback), print
// `step | loss | lr | tok/s`, save the adapters or the full checkpoint.
#include "../../include/data_hip.h"
#include "../../include/loader_hip.h"

#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <string>
#include <sys/stat.h>
#include <time.h>
#include <vector>

namespace {

struct Options {
    std::string model, train_data, lora_adapter, checkpoint_dir = "checkpoints";
    int lora_rank = 16, seq_len = 512, batch = 1, max_steps = 10000, log_interval = 1, full_param = 0, use_q8 = 0;
    float lora_alpha = 32.0f, lr = 0.0f;
};

void usage(const char *prog)
{
    printf("Usage: %s --model <path> [options]\n"
           "  --model <path>        model file or directory (.safetensors, shard directory, .gguf); --gguf is an alias\n"
           "  --train <path>        pre-tokenized training data (int32 token ids); without it: synthetic tokens\n"
           "  --seq <n>             sequence length (default 512)\n"
           "  --batch <n>           sequences per step (default 1)\n"
           "  --steps <n>           training steps (default 10000)\n"
           "  --lr <f>              learning rate (default 1e-5)\n"
           "  --lora-rank <n>       LoRA rank (default 16)\n"
           "  --lora-alpha <f>      LoRA alpha (default 32)\n"
           "  --lora-adapter <p>    adapter file: loaded if present, written at the end\n"
           "  --full-param          full-parameter SGD inside the backward (no LoRA)\n"
           "  --q8                  keep the frozen weights as Q8_0 in HBM (LoRA only)\n"
           "  --checkpoint <dir>    where lora_adapter.bin / full_checkpoint.bin go (default checkpoints)\n"
           "  --log-interval <n>    print every n steps (default 1)\n", prog);
}

// main.c:286-324: "gemma3" / "gemma2" in the config.json next to (or inside) the model path, else Qwen3
ModelType detect_model_type(const std::string &path)
{
    struct stat st;
    std::string cfg;
    if (stat(path.c_str(), &st) == 0 && S_ISDIR(st.st_mode)) cfg = path + "/config.json";
    else { const size_t sl = path.rfind('/'); cfg = sl == std::string::npos ? "config.json" : path.substr(0, sl) + "/config.json"; }
    FILE *fp = fopen(cfg.c_str(), "r");
    if (!fp) return MODEL_QWEN3;
    char buf[4096];
    const size_t n = fread(buf, 1, sizeof buf - 1, fp);
    buf[n] = 0;
    fclose(fp);
    if (strstr(buf, "\"gemma3") || strstr(buf, "\"gemma2")) { printf("[Model] Detected model_type: gemma3 (from config.json)\n"); return MODEL_GEMMA3; }
    if (strstr(buf, "\"qwen3") || strstr(buf, "\"qwen2")) printf("[Model] Detected model_type: qwen3 (from config.json)\n");
    return MODEL_QWEN3;
}

double seconds_since(const timespec &t0)
{
    timespec t;
    clock_gettime(CLOCK_MONOTONIC, &t);
    return (double)(t.tv_sec - t0.tv_sec) + (double)(t.tv_nsec - t0.tv_nsec) / 1e9;
}

}  // namespace

int main(int argc, char **argv)
{
    Options o;
    for (int i = 1; i < argc; i++) {
        const std::string a = argv[i];
        const bool has = i + 1 < argc;
        if (a == "--help") { usage(argv[0]); return 0; }
        else if ((a == "--model" || a == "--gguf") && has) o.model = argv[++i];
        else if (a == "--train" && has) o.train_data = argv[++i];
        else if (a == "--seq" && has) o.seq_len = atoi(argv[++i]);
        else if (a == "--batch" && has) o.batch = atoi(argv[++i]);
        else if (a == "--steps" && has) o.max_steps = atoi(argv[++i]);
        else if (a == "--lr" && has) o.lr = (float)atof(argv[++i]);
        else if (a == "--lora-rank" && has) o.lora_rank = atoi(argv[++i]);
        else if (a == "--lora-alpha" && has) o.lora_alpha = (float)atof(argv[++i]);
        else if (a == "--lora-adapter" && has) o.lora_adapter = argv[++i];
        else if (a == "--checkpoint" && has) o.checkpoint_dir = argv[++i];
        else if (a == "--log-interval" && has) o.log_interval = atoi(argv[++i]);
        else if (a == "--full-param" || a == "--accurate") o.full_param = 1;
        else if (a == "--q8") o.use_q8 = 1;
        else if (a == "--mode" && has) { if (strcmp(argv[++i], "sft") != 0) { fprintf(stderr, "[SFT] this driver only has --mode sft\n"); return 2; } }
        else { fprintf(stderr, "[SFT] unknown option %s\n", a.c_str()); usage(argv[0]); return 2; }
    }
    if (o.model.empty()) { fprintf(stderr, "[SFT] Error: --model is required for SFT mode\n"); return 2; }
    if (o.seq_len <= 0 || o.batch <= 0 || o.max_steps < 0 || o.log_interval <= 0) { fprintf(stderr, "[SFT] Error: --seq, --batch, --log-interval must be positive\n"); return 2; }
    const float lr = o.lr > 0 ? o.lr : 1e-5f;
    const ModelType mtype = detect_model_type(o.model);
    printf("=== %s Fast %s SFT ===\n", mtype == MODEL_GEMMA3 ? "Gemma3" : "Qwen3", o.full_param ? "Full-param SGD" : "LoRA");
    printf("  Model: %s\n", o.model.c_str());
    if (!o.full_param) printf("  LoRA rank: %d, alpha: %.1f\n", o.lora_rank, o.lora_alpha);
    printf("  Seq: %d, Steps: %d\n  LR: %.2e\n\n", o.seq_len, o.max_steps, lr);

    SFTModelRef *ref = model_ref_load(o.model.c_str(), mtype);
    if (!ref) { fprintf(stderr, "[SFT] Failed to load model\n"); return 1; }
    size_t params = (size_t)ref->vocab_size * ref->d_model * (ref->lm_head == ref->token_emb ? 1 : 2);
    for (int L = 0; L < ref->n_layers; L++) {
        const LayerWeightRef &r = ref->layers[L];
        for (const WeightRef *w : {&r.q_proj, &r.k_proj, &r.v_proj, &r.o_proj, &r.gate_proj, &r.up_proj, &r.down_proj}) params += (size_t)w->rows * w->cols;
    }
    printf("[SFT] Total model params: %zu (%.2f B)\n", params, (float)params / 1e9f);
    SFTState *sft = sft_state_create_from_ref(ref, o.batch, o.seq_len, o.full_param ? 0 : o.lora_rank, o.lora_alpha, o.use_q8 ? 0 : 1);
    const int vocab = ref->vocab_size;
    model_ref_free(ref);                                       // the state holds its own copies (the embedding table excepted)
    if (!sft) { fprintf(stderr, "[SFT] Failed to create SFT state\n"); return 1; }
    struct stat st;
    if (!o.full_param && !o.lora_adapter.empty() && stat(o.lora_adapter.c_str(), &st) == 0 && sft_load_lora(sft, o.lora_adapter.c_str()) == 0)
        printf("[SFT] LoRA adapters loaded from %s\n", o.lora_adapter.c_str());

    TokenLoader *loader = nullptr;
    if (!o.train_data.empty()) {
        loader = token_loader_open(o.train_data.c_str(), o.batch, o.seq_len);
        if (!loader) fprintf(stderr, "[SFT] Warning: could not load train data: %s\n", o.train_data.c_str());
    }
    const int BN = o.batch * o.seq_len;
    std::vector<uint32_t> input(BN), target(BN);
    timespec start;
    clock_gettime(CLOCK_MONOTONIC, &start);
    printf("\n=== Fast SFT Training Start ===\n");
    for (int step = 0; step < o.max_steps; step++) {
        if (loader) {
            if (token_loader_next(loader, input.data(), target.data()) < 0) {
                token_loader_reset(loader);
                token_loader_shuffle(loader);
                if (token_loader_next(loader, input.data(), target.data()) < 0) { fprintf(stderr, "[SFT] train data shorter than one batch\n"); break; }
            }
            for (int i = 0; i < BN; i++) { input[i] %= (uint32_t)vocab; target[i] %= (uint32_t)vocab; }   // ids beyond the table would read outside it
        } else {
            srand(42);                                         // main.c:471-477
            for (int i = 0; i < BN; i++) input[i] = (uint32_t)(rand() % 1000) % (uint32_t)vocab;
            for (int i = 0; i < BN; i++) target[i] = (i + 1) % o.seq_len ? input[i + 1] : input[i + 1 - o.seq_len];
        }
        const float loss = sft_train_step(sft, input.data(), target.data(), lr);
        if (step % o.log_interval == 0)
            printf("step %5d | loss %.4f | lr %.2e | %.1f tok/s\n", step, loss, lr, (double)(step + 1) * BN / seconds_since(start));
    }

    std::string save_path;
    if (o.full_param) {
        save_path = o.checkpoint_dir + "/full_checkpoint.bin";
        mkdir(o.checkpoint_dir.c_str(), 0755);
        sft_save_full_checkpoint(sft, save_path.c_str());
    } else {
        if (!o.lora_adapter.empty()) save_path = o.lora_adapter;
        else { save_path = o.checkpoint_dir + "/lora_adapter.bin"; mkdir(o.checkpoint_dir.c_str(), 0755); }
        sft_save_lora(sft, save_path.c_str());
    }
    printf("\n=== Fast SFT Complete ===\nTotal time: %.1f seconds\nCheckpoint saved: %s\n", seconds_since(start), save_path.c_str());
    sft_state_free(sft);
    if (loader) token_loader_free(loader);
    return 0;
}
