// Greedy generation through the engine's C interface, in the manner of the reference's own example
// (example/load_model/load_model.cu:8-25: load a model, set the runtime up, encode, infer).
//
//   engine_demo MODEL_DIR|--random CONFIG.json:SEED  N_PREDICT  IDS [IDS ...]     (IDS: 3,14,15)
//
// Prints one line per request: its id, then the tokens it was given.
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "tffinfer_engine.h"

static int parse_ids(const char* s, int32_t* out, int cap) {
    int n = 0;
    while (*s && n < cap) {
        char* end;
        out[n++] = (int32_t)strtol(s, &end, 10);
        if (end == s) return -1;
        s = *end == ',' ? end + 1 : end;
    }
    return n;
}

int main(int argc, char** argv) {
    if (argc < 4) {
        fprintf(stderr, "usage: %s MODEL_DIR|--random CONFIG.json:SEED N_PREDICT IDS [IDS ...]\n", argv[0]);
        return 2;
    }
    int a = 1;
    tff_engine* e;
    const char* options = getenv("TFF_ENGINE_OPTIONS");      // a JSON object, e.g. {"dtype": "float32"}
    if (strcmp(argv[a], "--random") == 0) {
        char file[1024];
        snprintf(file, sizeof file, "%s", argv[a + 1]);
        char* colon = strrchr(file, ':');
        unsigned long long seed = 0;
        if (colon) {
            *colon = 0;
            seed = strtoull(colon + 1, NULL, 10);
        }
        e = engine_create_random(file, seed, options);
        a += 2;
    } else {
        e = engine_create(argv[a], options);
        a += 1;
    }
    if (!e) {
        fprintf(stderr, "engine: %s\n", engine_last_error());
        return 1;
    }
    const int n_predict = atoi(argv[a++]);
    char params[128];
    snprintf(params, sizeof params, "{\"max_new_tokens\": %d, \"ignore_eos\": true}", n_predict);
    enum { MAX_REQ = 64, MAX_OUT = 4096 };
    static int32_t out[MAX_REQ][MAX_OUT];
    int n_out[MAX_REQ] = {0};
    int n_req = 0;
    for (; a < argc && n_req < MAX_REQ; ++a, ++n_req) {
        int32_t ids[4096];
        const int n = parse_ids(argv[a], ids, 4096);
        if (n <= 0 || engine_add_request(e, ids, n, params) != n_req) {
            fprintf(stderr, "request %d: %s\n", n_req, n <= 0 ? "bad list of ids" : engine_last_error());
            engine_destroy(e);
            return 1;
        }
    }
    while (engine_has_work(e) == 1) {
        tff_step_event ev[MAX_REQ];
        const int n = engine_step(e, ev, MAX_REQ);
        if (n < 0) {
            fprintf(stderr, "step: %s\n", engine_last_error());
            engine_destroy(e);
            return 1;
        }
        for (int i = 0; i < n; ++i)
            if (ev[i].token >= 0 && ev[i].request_id < MAX_REQ && n_out[ev[i].request_id] < MAX_OUT)
                out[ev[i].request_id][n_out[ev[i].request_id]++] = ev[i].token;
    }
    for (int r = 0; r < n_req; ++r) {
        printf("%d:", r);
        for (int i = 0; i < n_out[r]; ++i) printf(" %d", out[r][i]);
        printf("\n");
    }
    engine_destroy(e);
    return 0;
}
