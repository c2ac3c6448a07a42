// Drives the UNMODIFIED reference CPU backend (llm::Model, built from
// /root/reference/src/{gguf,model_common,model_cpu}.cpp by oracle/Makefile) over a
// synthetic one-layer GGUF and dumps the logits of every step.  Test infrastructure
// only: used in the build container to produce tests/golden/cfg1_*.npz.
//
//   ref_driver MODEL.gguf N_TOKENS N_CTX N_LOGITS OUT.bin [POS0]
//
// Step t feeds token id t at position POS0 + t (POS0 = 0 unless given; cache rows below POS0 stay
// as the backend's zero-initialised vectors leave them) (Model::forward, reference src/model.h:75),
// i.e. the token-at-a-time causal prefill of src/model_cpu.cpp:314-319 followed by
// decode, which are the same call on the CPU backend.  OUT.bin receives
// N_TOKENS x N_LOGITS little-endian fp32 values.
#include <cstdio>
#include <cstdlib>
#include <string>
#include <vector>

#include "gguf.h"
#include "model.h"

int main(int argc, char** argv) {
    if (argc != 6 && argc != 7) {
        fprintf(stderr, "usage: %s MODEL.gguf N_TOKENS N_CTX N_LOGITS OUT.bin [POS0]\n", argv[0]);
        return 2;
    }
    const std::string path = argv[1];
    const int n_tokens = atoi(argv[2]);
    const int n_ctx = atoi(argv[3]);
    const int n_logits = atoi(argv[4]);
    const int pos0 = argc == 7 ? atoi(argv[6]) : 0;
    if (pos0 < 0 || pos0 + n_tokens > n_ctx) {
        fprintf(stderr, "positions [%d, %d) do not fit n_ctx %d\n", pos0, pos0 + n_tokens, n_ctx);
        return 2;
    }

    llm::GGUF gguf;
    gguf.load(path);
    llm::Model model;
    model.load(gguf);
    model.init_buffers(n_ctx, 1);
    if (n_logits > model.hparams.n_vocab) {
        fprintf(stderr, "n_logits %d exceeds n_vocab %d\n", n_logits, model.hparams.n_vocab);
        return 2;
    }

    FILE* f = fopen(argv[5], "wb");
    if (!f) {
        perror("fopen");
        return 1;
    }
    for (int t = 0; t < n_tokens; ++t) {
        const float* logits = model.forward(t, pos0 + t);
        if (fwrite(logits, sizeof(float), (size_t)n_logits, f) != (size_t)n_logits) {
            perror("fwrite");
            return 1;
        }
    }
    fclose(f);
    fprintf(stderr, "ref_driver: %d steps, head_dim %d, n_head %d, n_head_kv %d, n_ctx %d\n", n_tokens,
            model.hparams.head_dim, model.hparams.n_head, model.hparams.n_head_kv, model.hparams.n_ctx);
    return 0;
}
