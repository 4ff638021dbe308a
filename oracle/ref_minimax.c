/*
 * TEST INFRASTRUCTURE ONLY.  Runs the reference's OWN in-test models of the MiniMax-M3 operators on given inputs:
 * ref_topk (tests/test_minimax_m3_sparse_attention.c:145-213), ref_sparse_fwd (:231-288) and ref_sparse_fwd_gqa
 * (:423-483) are file-static functions of the reference's test program, reached by compiling that file where it
 * lies (the #include below, its main renamed).  Pure host code; the output is the golden data of the tests of
 * gd_minimax_m3_index_topk / gd_minimax_m3_sparse_attention.
 *
 * Input file:  int32 B, Hq, Hkv, Dh, block, topk, init_blocks, local_blocks, topk_given; float scale;
 *              int32 cu[B+1]; uint16 q[N*Hq*Dh], k[N*Hkv*Dh], v[N*Hkv*Dh]; if topk_given: int32 topk[Hkv*N*topk]
 * Output file: int32 topk[Hkv*N*topk] (ref_topk on q and k, which needs Hq == Hkv and topk <= 4, or the given
 *              one), float out[N*Hq*Dh]
 */
#define main gd_reference_test_program_main
#include "tests/test_minimax_m3_sparse_attention.c"
#undef main

static void die(const char *what)
{
    fprintf(stderr, "ref_minimax: %s\n", what);
    exit(2);
}

int main(int argc, char **argv)
{
    int32_t head[9], *cu, *topk;
    float scale, *out;
    uint16_t *q, *k, *v;
    uint32_t B, Hq, Hkv, Dh, block, tk, N;
    FILE *f;
    if (argc != 3) die("usage: ref_minimax <in> <out>");
    f = fopen(argv[1], "rb");
    if (f == NULL || fread(head, sizeof(int32_t), 9, f) != 9 || fread(&scale, sizeof(scale), 1, f) != 1) die("short header");
    B = (uint32_t)head[0]; Hq = (uint32_t)head[1]; Hkv = (uint32_t)head[2]; Dh = (uint32_t)head[3];
    block = (uint32_t)head[4]; tk = (uint32_t)head[5];
    cu = (int32_t *)calloc(B + 1U, sizeof(int32_t));
    if (fread(cu, sizeof(int32_t), B + 1U, f) != B + 1U) die("short cu");
    N = (uint32_t)cu[B];
    q = (uint16_t *)calloc((size_t)N * Hq * Dh, 2U);
    k = (uint16_t *)calloc((size_t)N * Hkv * Dh, 2U);
    v = (uint16_t *)calloc((size_t)N * Hkv * Dh, 2U);
    topk = (int32_t *)calloc((size_t)Hkv * N * tk, sizeof(int32_t));
    out = (float *)calloc((size_t)N * Hq * Dh, sizeof(float));
    if (fread(q, 2U, (size_t)N * Hq * Dh, f) != (size_t)N * Hq * Dh || fread(k, 2U, (size_t)N * Hkv * Dh, f) != (size_t)N * Hkv * Dh ||
        fread(v, 2U, (size_t)N * Hkv * Dh, f) != (size_t)N * Hkv * Dh)
        die("short tensors");
    if (head[8]) {
        if (fread(topk, sizeof(int32_t), (size_t)Hkv * N * tk, f) != (size_t)Hkv * N * tk) die("short topk");
    } else {
        if (Hq != Hkv || tk > 4U) die("ref_topk needs Hq == Hkv and topk <= 4");
        ref_topk(q, k, cu, B, Hq, Dh, block, tk, (uint32_t)head[6], (uint32_t)head[7], topk);
    }
    fclose(f);
    if (Hq == Hkv) ref_sparse_fwd(q, k, v, cu, topk, B, Hq, Dh, block, tk, scale, out);
    else ref_sparse_fwd_gqa(q, k, v, cu, topk, B, Hq, Hkv, Dh, block, tk, scale, out);
    f = fopen(argv[2], "wb");
    if (f == NULL) die("cannot open the output");
    fwrite(topk, sizeof(int32_t), (size_t)Hkv * N * tk, f);
    fwrite(out, sizeof(float), (size_t)N * Hq * Dh, f);
    fclose(f);
    printf("ref_minimax: ok N=%u Hq=%u Hkv=%u Dh=%u\n", N, Hq, Hkv, Dh);
    return 0;
}
