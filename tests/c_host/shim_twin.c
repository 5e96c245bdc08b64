/* The call sequence of the Rust shim (bindings/rust/model-transformer-mi355x/src/lib.rs) in plain
 * C, compiled against include/coeus.h and linked to libcoeus_mi355x.so: a host that is neither
 * Python nor ctypes drives the boundary the way the crate's build() / forward() / load() do.
 *
 *   shim_twin host                 config default / validate / counts / init loop / .rustllm write+read (no GPU)
 *   shim_twin forward OUT IDS...   build(config) with the reference's init, forward(ids), logits -> OUT (f32)
 *   shim_twin errors               the error mapping of forward(): statuses and messages
 */
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "coeus.h"

static void small_config(coeus_config *c) {
    coeus_config_default(c);
    c->hidden_dim = 64; c->num_layers = 2; c->num_heads = 4; c->intermediate_dim = 128;
    c->vocab_size = 300; c->max_seq_len = 32;
}

#define REQUIRE(cond) do { if (!(cond)) { fprintf(stderr, "FAILED %s:%d: %s (last error: %s)\n", __FILE__, __LINE__, #cond, coeus_last_error()); return 1; } } while (0)

static int host_only(const char *tmp_path) {
    coeus_config c;
    coeus_config_default(&c);
    REQUIRE(c.hidden_dim == 768 && c.num_layers == 12 && c.num_heads == 12 && c.intermediate_dim == 3072);
    REQUIRE(c.vocab_size == 50257 && c.max_seq_len == 1024 && c.use_bias == 1);
    REQUIRE(coeus_config_validate(&c) == COEUS_OK);
    REQUIRE(coeus_config_num_parameters(&c) == 163087441ull);   /* lib.rs:541-580 */
    c.hidden_dim = 767;
    REQUIRE(coeus_config_validate(&c) == COEUS_INVALID_CONFIG);
    REQUIRE(strstr(coeus_last_error(), "divisible by number of heads") != NULL);
    small_config(&c);
    REQUIRE(coeus_config_validate(&c) == COEUS_OK);
    const uint64_t n = coeus_config_num_parameters(&c);
    float *p = (float *)malloc(n * sizeof(float));
    REQUIRE(p && coeus_init_default_parameters(p, n, c.hidden_dim) == COEUS_OK);
    REQUIRE(p[0] == 0.0f);                                      /* sin(0) */
    REQUIRE(coeus_rustllm_write(tmp_path, &c, p, n) == COEUS_OK);
    coeus_config back;
    uint64_t n_back = 0;
    REQUIRE(coeus_rustllm_read_header(tmp_path, &back, &n_back) == COEUS_OK);
    REQUIRE(n_back == n && back.hidden_dim == 64 && back.intermediate_dim == 128 && back.vocab_size == 300);
    float *q = (float *)malloc(n * sizeof(float));
    REQUIRE(q && coeus_rustllm_read_parameters(tmp_path, q, n) == COEUS_OK);
    REQUIRE(memcmp(p, q, n * sizeof(float)) == 0);
    free(p); free(q);
    printf("host ok: %llu parameters\n", (unsigned long long)n);
    return 0;
}

static int build_default(coeus_model **m, coeus_config *c) {   /* ModelBuilder::build, lib.rs:587-638 */
    small_config(c);
    REQUIRE(coeus_config_validate(c) == COEUS_OK);
    const uint64_t n = coeus_config_num_parameters(c);
    float *p = (float *)malloc(n * sizeof(float));
    REQUIRE(p && coeus_init_default_parameters(p, n, c->hidden_dim) == COEUS_OK);
    const int rc = coeus_model_create(c, p, n, m);
    free(p);                                                     /* the weights live in HBM now */
    REQUIRE(rc == COEUS_OK);
    REQUIRE(coeus_model_num_parameters(*m) == n && strcmp(coeus_model_name(*m), "TransformerModel") == 0);
    return 0;
}

static int forward(const char *out_path, int n_ids, char **ids_txt) {
    coeus_config c;
    coeus_model *m = NULL;
    if (build_default(&m, &c)) return 1;
    uint64_t ids[64];
    REQUIRE(n_ids >= 1 && n_ids <= 32);
    for (int i = 0; i < n_ids; i++) ids[i] = strtoull(ids_txt[i], NULL, 10);
    float *logits = (float *)malloc(c.vocab_size * sizeof(float));
    REQUIRE(logits && coeus_model_forward(m, ids, (uint64_t)n_ids, logits) == COEUS_OK);
    FILE *f = fopen(out_path, "wb");
    REQUIRE(f && fwrite(logits, sizeof(float), c.vocab_size, f) == c.vocab_size);
    fclose(f);
    free(logits);
    coeus_model_destroy(m);
    printf("forward ok: %d ids -> %llu logits\n", n_ids, (unsigned long long)c.vocab_size);
    return 0;
}

static int errors(void) {
    coeus_config c;
    coeus_model *m = NULL;
    if (build_default(&m, &c)) return 1;
    float logits[300];
    uint64_t ids[40] = {1, 300};
    REQUIRE(coeus_model_forward(m, ids, 2, logits) == COEUS_INVALID_INPUT);              /* lib.rs:816-822 */
    REQUIRE(strcmp(coeus_last_error(), "Token ID 300 out of range [0, 299]") == 0);
    memset(ids, 0, sizeof ids);
    REQUIRE(coeus_model_forward(m, ids, 33, logits) == COEUS_INVALID_INPUT);             /* lib.rs:797-802 */
    REQUIRE(strcmp(coeus_last_error(), "Sequence length 33 out of range [1, 32]") == 0);
    REQUIRE(coeus_model_forward(m, ids, 0, logits) == COEUS_INVALID_INPUT);              /* a panic in the reference */
    REQUIRE(coeus_model_forward(NULL, ids, 1, logits) == COEUS_INVALID_INPUT);
    coeus_model_destroy(m);
    printf("errors ok\n");
    return 0;
}

int main(int argc, char **argv) {
    if (argc >= 3 && strcmp(argv[1], "host") == 0) return host_only(argv[2]);
    if (argc >= 4 && strcmp(argv[1], "forward") == 0) return forward(argv[2], argc - 3, argv + 3);
    if (argc >= 2 && strcmp(argv[1], "errors") == 0) return errors();
    fprintf(stderr, "usage: shim_twin host TMPFILE | forward OUT IDS... | errors\n");
    return 2;
}
