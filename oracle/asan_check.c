/*
 * TEST INFRASTRUCTURE ONLY — driver of the sanitizer build of the oracle (make -C oracle asan): reads one batch and the
 * weights of a network from a file, runs the CSR builders and the whole forward of s2v_oracle.c under
 * AddressSanitizer / UndefinedBehaviorSanitizer, and writes the results for comparison with the regular build.
 *
 *   asan_check <in.bin> <out.bin>
 *   in.bin : int32 N, E, B, K, C, H, Q, L; int32 edge_x[E], edge_y[E], subg_id[N], node_idx[N]; float X[N,K],
 *            W_n2l[K,C], W_conv[C,C], W_h1[C,H], W_h2[H,Q]; int32 label row_ptr[B+1], col[B]; float val[B]
 *   out.bin: int32 a_row_ptr[N+1], a_col[E]; float a_val[E]; int32 s_row_ptr[B+1], s_col[N]; float s_val[N];
 *            float msg[N,C], h[(L+1),N,C], pool[B,C], hidden[B,H], logits[B,Q], probs[B,Q], loss_rows[B];
 *            int32 pred[B], truth[B], hit[B]; float scalars[2]; float jagged[N] (softmax of column 0 of h_L per graph)
 */
#include <stdio.h>
#include <stdlib.h>
#include "s2v_oracle.h"

static void* rd(FILE* f, size_t count, size_t size)
{
    void* p = malloc(count * size > 0 ? count * size : 1);
    if (!p || fread(p, size, count, f) != count) { fprintf(stderr, "short read\n"); exit(2); }
    return p;
}

int main(int argc, char** argv)
{
    if (argc != 3) { fprintf(stderr, "usage: asan_check in.bin out.bin\n"); return 2; }
    FILE* f = fopen(argv[1], "rb");
    if (!f) { fprintf(stderr, "cannot open %s\n", argv[1]); return 2; }
    int* hdr = rd(f, 8, sizeof(int));
    const int N = hdr[0], E = hdr[1], B = hdr[2], K = hdr[3], C = hdr[4], H = hdr[5], Q = hdr[6], L = hdr[7];
    int* ex = rd(f, E, sizeof(int)); int* ey = rd(f, E, sizeof(int));
    int* sid = rd(f, N, sizeof(int)); int* nid = rd(f, N, sizeof(int));
    float* X = rd(f, (size_t)N * K, sizeof(float));
    float* Wn = rd(f, (size_t)K * C, sizeof(float)); float* Wc = rd(f, (size_t)C * C, sizeof(float));
    float* W1 = rd(f, (size_t)C * H, sizeof(float)); float* W2 = rd(f, (size_t)H * Q, sizeof(float));
    int* lrp = rd(f, B + 1, sizeof(int)); int* lci = rd(f, B, sizeof(int)); float* lv = rd(f, B, sizeof(float));
    fclose(f);

    /* exact sizes everywhere: an access one element past any of these is caught */
    int* arp = malloc(sizeof(int) * (N + 1)); int* aci = malloc(sizeof(int) * (E ? E : 1)); float* av = malloc(sizeof(float) * (E ? E : 1));
    int* srp = malloc(sizeof(int) * (B + 1)); int* sci = malloc(sizeof(int) * (N ? N : 1)); float* sv = malloc(sizeof(float) * (N ? N : 1));
    orc_csr_node2node(N, E, ex, ey, 0, arp, aci, av);
    orc_csr_subgraph(B, N, sid, nid, 0, srp, sci, sv);
    const size_t NC = (size_t)N * C;
    float* msg = malloc(sizeof(float) * NC); float* h = malloc(sizeof(float) * NC * (L + 1));
    float* pool = malloc(sizeof(float) * B * C); float* hidden = malloc(sizeof(float) * B * H);
    float* logits = malloc(sizeof(float) * B * Q); float* probs = malloc(sizeof(float) * B * Q);
    float* loss = malloc(sizeof(float) * B); int* pred = malloc(sizeof(int) * B); int* truth = malloc(sizeof(int) * B);
    int* hit = malloc(sizeof(int) * B); float scalars[2];
    orc_s2v_forward(N, B, K, C, H, Q, L, arp, aci, av, srp, sci, sv, X, Wn, Wc, W1, W2, lrp, lci, lv, msg, h, pool, hidden, logits,
                    probs, loss, pred, truth, hit, scalars);
    float* jag = malloc(sizeof(float) * (N ? N : 1));
    int* lens = malloc(sizeof(int) * B);
    for (int g = 0; g < B; ++g) lens[g] = srp[g + 1] - srp[g];
    for (int i = 0; i < N; ++i) jag[i] = h[(size_t)L * NC + (size_t)i * C];
    orc_jagged_softmax(jag, lens, B);

    f = fopen(argv[2], "wb");
    if (!f) { fprintf(stderr, "cannot write %s\n", argv[2]); return 2; }
    fwrite(arp, sizeof(int), N + 1, f); fwrite(aci, sizeof(int), E, f); fwrite(av, sizeof(float), E, f);
    fwrite(srp, sizeof(int), B + 1, f); fwrite(sci, sizeof(int), N, f); fwrite(sv, sizeof(float), N, f);
    fwrite(msg, sizeof(float), NC, f); fwrite(h, sizeof(float), NC * (L + 1), f); fwrite(pool, sizeof(float), (size_t)B * C, f);
    fwrite(hidden, sizeof(float), (size_t)B * H, f); fwrite(logits, sizeof(float), (size_t)B * Q, f);
    fwrite(probs, sizeof(float), (size_t)B * Q, f); fwrite(loss, sizeof(float), B, f);
    fwrite(pred, sizeof(int), B, f); fwrite(truth, sizeof(int), B, f); fwrite(hit, sizeof(int), B, f);
    fwrite(scalars, sizeof(float), 2, f); fwrite(jag, sizeof(float), N, f);
    fclose(f);
    free(hdr); free(ex); free(ey); free(sid); free(nid); free(X); free(Wn); free(Wc); free(W1); free(W2); free(lrp); free(lci); free(lv);
    free(arp); free(aci); free(av); free(srp); free(sci); free(sv); free(msg); free(h); free(pool); free(hidden); free(logits);
    free(probs); free(loss); free(pred); free(truth); free(hit); free(jag); free(lens);
    printf("asan_check ok: N=%d E=%d B=%d\n", N, E, B);
    return 0;
}
