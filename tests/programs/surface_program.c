/* The less-used entry points of the program-facing runtime, each checked on the GPU against the entry points
 * the committed programs use (bit for bit) or against the message it must decrypt to.
 *
 * usage: surface_program <poly degree> <mul depth> <q0 bits> <scale bits> <seed> [bootstrap]
 * prints one "ok <what>" line per check and "surface ok"; exit status 1 at the first failure.
 * With "bootstrap" the three staged bootstrap operators are run too (needs depth >= 13).
 */
#include <math.h>
#include <unistd.h>

#include "rt_ant/rt_ant.h"

static CKKS_PARAMS* Params;
CKKS_PARAMS*        Get_context_params(void) { return Params; }
static RT_DATA_INFO Data_info = {"", "surface", DE_PLAINTEXT};
static int          Has_file;
RT_DATA_INFO*       Get_rt_data_info(void) { return Has_file ? &Data_info : NULL; }
static MAP_DESC     Whole = {NORMAL, 0, 0, 0, 1};
static DATA_SCHEME  In_scheme = {"image", {0, 0, 0, 0}, 1, &Whole};
int                 Get_input_count(void) { return 1; }
DATA_SCHEME*        Get_encode_scheme(int i) { return i == 0 ? &In_scheme : NULL; }

static uint64_t State;
static double   Unit(void) { /* in [-1, 1) */
  State = State * 6364136223846793005ull + 1442695040888963407ull;
  return (double)(int64_t)(State >> 11) / (double)(1ull << 52) - 1.0;
}
#define CHECK(cond, ...)                 \
  do {                                   \
    if (!(cond)) {                       \
      fprintf(stderr, "FAILED: " __VA_ARGS__); \
      fprintf(stderr, "\n");             \
      exit(1);                           \
    }                                    \
  } while (0)

static int64_t* Words(POLY p) {
  int64_t* h = (int64_t*)malloc(Get_poly_len(p) * sizeof(int64_t));
  Rt_download_poly(h, p);
  return h;
}
static int Same(POLY a, POLY b) {
  if (Get_poly_len(a) != Get_poly_len(b)) return 0;
  int64_t *x = Words(a), *y = Words(b);
  int      r = memcmp(x, y, Get_poly_len(a) * sizeof(int64_t)) == 0;
  free(x);
  free(y);
  return r;
}
static void Random_poly(POLY p, int ntt) { /* uniform residues */
  size_t   n = p->_ring_degree, T = Get_num_pq(p);
  int64_t* h = (int64_t*)malloc(T * n * sizeof(int64_t));
  for (size_t t = 0; t < T; ++t) {
    uint64_t q = (uint64_t)(t < Poly_level(p) ? Q_modulus()[t]._val : P_modulus()[t - Poly_level(p)]._val);
    for (size_t i = 0; i < n; ++i) {
      State = State * 6364136223846793005ull + 1442695040888963407ull;
      h[t * n + i] = (int64_t)((State >> 3) % q);
    }
  }
  Rt_upload_poly(p, h);
  Set_is_ntt(p, ntt);
  free(h);
}
static double Max_err(CIPHER c, const double* want, uint32_t len) {
  double* m = Get_msg(c);
  double  e = 0;
  for (uint32_t i = 0; i < len; ++i)
    if (fabs(m[i] - want[i]) > e) e = fabs(m[i] - want[i]);
  free(m);
  return e;
}

int main(int argc, char** argv) {
  if (argc < 6) {
    fprintf(stderr, "usage: %s <degree> <depth> <q0 bits> <scale bits> <seed> [bootstrap]\n", argv[0]);
    return 2;
  }
  int32_t rots[] = {1, -1, 3};
  Params         = (CKKS_PARAMS*)calloc(1, sizeof(CKKS_PARAMS) + sizeof(rots));
  Params->_provider         = LIB_ANT;
  Params->_poly_degree      = (uint32_t)strtoul(argv[1], NULL, 0);
  Params->_mul_depth        = strtoul(argv[2], NULL, 0);
  Params->_first_mod_size   = strtoul(argv[3], NULL, 0);
  Params->_scaling_mod_size = strtoul(argv[4], NULL, 0);
  Params->_hamming_weight   = 192 < Params->_poly_degree / 2 ? 192 : 0;
  Params->_num_rot_idx      = 3;
  memcpy(Params->_rot_idxs, rots, sizeof(rots));
  State         = strtoull(argv[5], NULL, 0) * 2654435761u + 1;
  int bootstrap = argc > 6 && strcmp(argv[6], "bootstrap") == 0;

  Prepare_context();
  Rt_generate_keys(strtoull(argv[5], NULL, 0));
  uint32_t N = Degree(), slots = N / 2;
  size_t   L = Get_q_cnt(), K = Get_p_cnt();

  /* ---- one-limb views and arithmetic against the Hw_* calls ------------------------------------------ */
  POLY a = Alloc_poly(N, L, 1), b = Alloc_poly(N, L, 1), r1 = Alloc_poly(N, L, 1), r2 = Alloc_poly(N, L, 1);
  Random_poly(a, 1);
  Random_poly(b, 1);
  for (size_t t = 0; t < L + K; ++t) {
    MODULUS* m  = t < L ? Q_modulus() + t : P_modulus() + (t - L);
    L_POLY   la = Lpoly_from_poly(a, t), lb = Lpoly_from_poly(b, t), lr = Lpoly_from_poly(r1, t);
    Mul_lpoly(&lr, la, lb, m);
    Mac_lpoly(&lr, la, lb, m);
    Add_lpoly(&lr, lr, la, m);
    Sub_lpoly(&lr, lr, lb, m);
    Mul_scalar(&lr, lr, 12345, m);
    Add_scalar(&lr, lr, 7, m);
    Sub_scalar(&lr, lr, 9, m);
    Mac_scalar(&lr, la, 3, m);
    int64_t* x = Coeffs(r2, t, N);
    Hw_modmul(x, Coeffs(a, t, N), Coeffs(b, t, N), m, N);
    Hw_modmuladd(x, Coeffs(a, t, N), Coeffs(b, t, N), m, N);
    Hw_modadd(x, x, Coeffs(a, t, N), m, N);
    Hw_modsub(x, x, Coeffs(b, t, N), m, N);
    Hw_modmul_scalar(x, x, 12345, m, N);
    Hw_modadd_scalar(x, x, 7, m, N);
    Hw_modsub_scalar(x, x, 9, m, N);
    Hw_modmuladd_scalar(x, Coeffs(a, t, N), 3, m, N);
  }
  CHECK(Same(r1, r2), "one-limb arithmetic differs from the Hw_* calls");
  {
    LPOLY  tmp = Alloc_lpoly(N);
    L_POLY la  = Lpoly_from_poly(a, 1);
    Intt(tmp, la, 1);
    CHECK(!Is_lpoly_ntt(tmp), "Intt must clear the flag");
    L_POLY back = Lpoly_from_poly(r1, 1);
    Ntt(&back, *tmp, 1);
    Set_poly_data(r2, la, 0); /* limb 0 of r2 := limb 1 of a */
    int64_t *x = (int64_t*)malloc(N * 8), *y = (int64_t*)malloc(N * 8);
    POLYNOMIAL v1 = *r1, v2 = *a;
    v1._data = Coeffs(r1, 1, N), v1._num_primes = 1, v1._num_primes_p = 0, v1._num_alloc_primes = 1;
    v2._data = Coeffs(a, 1, N), v2._num_primes = 1, v2._num_primes_p = 0, v2._num_alloc_primes = 1;
    Rt_download_poly(x, &v1);
    Rt_download_poly(y, &v2);
    CHECK(memcmp(x, y, N * 8) == 0, "Intt then Ntt of a limb is not the identity");
    v1._data = Coeffs(r2, 0, N);
    Rt_download_poly(x, &v1);
    CHECK(memcmp(x, y, N * 8) == 0, "Set_poly_data");
    free(x), free(y);
    Free_lpoly(tmp);
  }
  printf("ok lpoly\n");

  /* ---- per-limb scalars ------------------------------------------------------------------------------- */
  {
    VALUE_LIST* sc = Alloc_value_list(I64_TYPE, L + K);
    for (size_t t = 0; t < L + K; ++t) Set_i64_value(sc, t, (int64_t)(1000003 * (t + 1)));
    Scalars_integer_multiply_poly(r1, a, sc);
    Scalars_integer_add_poly(r1, r1, sc);
    for (size_t t = 0; t < L + K; ++t) {
      MODULUS* m = t < L ? Q_modulus() + t : P_modulus() + (t - L);
      Hw_modmul_scalar(Coeffs(r2, t, N), Coeffs(a, t, N), Get_i64_value_at(sc, t), m, N);
      Hw_modadd_scalar(Coeffs(r2, t, N), Coeffs(r2, t, N), Get_i64_value_at(sc, t), m, N);
    }
    CHECK(Same(r1, r2), "Scalars_integer_* differ from per-limb Hw_* calls");
    /* one negative integer for every limb, checked on the host */
    Scalar_integer_multiply_poly(r1, a, -5);
    int64_t *x = Words(a), *y = Words(r1);
    for (size_t t = 0; t < L + K; ++t) {
      int64_t q = t < L ? Q_modulus()[t]._val : P_modulus()[t - L]._val;
      for (uint32_t i = 0; i < N; i += 97) {
        __int128 w = ((__int128)x[t * N + i] * -5) % q;
        if (w < 0) w += q;
        CHECK((int64_t)w == y[t * N + i], "Scalar_integer_multiply_poly limb %zu coefficient %u", t, i);
      }
    }
    free(x), free(y);
    /* one digit only: the other limbs keep what they held */
    POLY v = Alloc_poly(N, L, 0), w = Alloc_poly(N, L, 0);
    Random_poly(v, 1);
    Copy_poly(w, v);
    size_t part = Get_q_parts() > 1 ? 1 : 0, ps = (L + Get_q_parts() - 1) / Get_q_parts();
    Scalars_integer_multiply_poly_qpart(w, v, sc, part);
    int64_t *hv = Words(v), *hw = Words(w);
    for (size_t t = 0; t < L; ++t) {
      int      in = t >= ps * part && t < ps * (part + 1);
      int64_t  q  = Q_modulus()[t]._val;
      __int128 e  = in ? ((__int128)hv[t * N + 5] * Get_i64_value_at(sc, t)) % q : hv[t * N + 5];
      CHECK((int64_t)e == hw[t * N + 5], "Scalars_integer_multiply_poly_qpart limb %zu", t);
    }
    free(hv), free(hw);
    Free_poly(v), Free_poly(w);
    Free_value_list(sc);
  }
  printf("ok scalars\n");

  /* ---- Alloc_precomp's box, Conv_poly2ntt, Automorphism_transform, Mul_poly_fast ------------------------- */
  {
    POLY c = Alloc_poly(N, L, 0);
    Random_poly(c, 1);
    VALUE_LIST* box = Alloc_precomp(c);
    CHECK(LIST_TYPE(box) == PTR_TYPE && LIST_LEN(box) == Num_decomp(c), "Alloc_precomp list shape");
    POLY_ARR arr = Alloc_polys((uint32_t)Num_decomp(c), N, L, 1);
    Precomp(arr, Num_decomp(c), c);
    for (size_t d = 0; d < Num_decomp(c); ++d)
      CHECK(Same((POLY)Get_ptr_value_at(box, d), &arr[d]), "Alloc_precomp digit %zu differs from Precomp", d);
    Free_precomp(box);
    Free_polys(arr);

    POLY co = Alloc_poly(N, L, 0), n1 = Alloc_poly(N, L, 0);
    Random_poly(co, 0);
    Conv_poly2ntt(n1, co);
    CHECK(!Is_ntt(co) && Is_ntt(n1), "Conv_poly2ntt flags");
    Conv_poly2ntt_inplace(co);
    CHECK(Same(n1, co), "Conv_poly2ntt differs from the in-place transform");

    POLYNOMIAL tab = {N, 1, 1, 0, false, Auto_order(3)};
    VALUE_LIST* order = Alloc_value_list(I64_TYPE, N);
    Rt_download_poly(Get_i64_values(order), &tab);
    POLY rot = Alloc_poly(N, L, 0), want = Alloc_poly(N, L, 0);
    Automorphism_transform(rot, c, order);
    for (size_t t = 0; t < L; ++t) Hw_rotate(Coeffs(want, t, N), Coeffs(c, t, N), Auto_order(3), Q_modulus() + t, N);
    CHECK(Same(rot, want), "Automorphism_transform differs from Hw_rotate with the same table");
    Free_value_list(order);

    Mul_poly(want, c, co);
    Mul_poly_fast(rot, c, co, co);
    CHECK(Same(rot, want), "Mul_poly_fast differs from Mul_poly");
    Chk_level(rot, c, co);
    POLY by = Alloc_poly(N, 1, 0);
    Init_poly_by_opnd(by, c, NULL, false);
    CHECK(Poly_level(by) == L && Num_p(by) == 0, "Init_poly_by_opnd");
    Free_poly(by), Free_poly(rot), Free_poly(want), Free_poly(co), Free_poly(n1), Free_poly(c);
  }
  printf("ok poly\n");

  /* ---- ciphertext-level: scales, views, inputs ---------------------------------------------------------- */
  double* x = (double*)malloc(slots * sizeof(double));
  for (uint32_t i = 0; i < slots; ++i) x[i] = 0.5 * Unit();
  PLAINTEXT  pt, pt2;
  CIPHERTEXT ct, up, down, raised;
  memset(&pt, 0, sizeof(pt)), memset(&pt2, 0, sizeof(pt2)), memset(&ct, 0, sizeof(ct)), memset(&up, 0, sizeof(up));
  memset(&down, 0, sizeof(down)), memset(&raised, 0, sizeof(raised));
  Encode_double(&pt, x, slots, 1, (uint32_t)L);
  Encrypt(&ct, &pt);
  CHECK(Max_err(&ct, x, slots) < 1e-5, "fresh ciphertext");
  CHECK(Within_value_range(&ct, x, slots), "Within_value_range on a message in range");
  {
    /* one slot spreads over the coefficients divided by the slot count (at most 2^15 here) */
    double big = ldexp(1.0, (int)(Params->_first_mod_size + (L - 1) * Params->_scaling_mod_size - Params->_scaling_mod_size) + 20);
    if (isfinite(big * Get_default_sc())) /* deep chains hold more bits than a double's exponent */
      CHECK(!Within_value_range(&ct, &big, 1), "Within_value_range on a message out of range");
  }
  Copy_plain(&pt2, &pt);
  CHECK(Same(&pt._poly, &pt2._poly) && pt2._sf_degree == pt._sf_degree && pt2._slots == pt._slots, "Copy_plain");

  /* Upscale by 2^10 then Downscale brings the scale back to one degree at the next level */
  uint32_t sf_bits = (uint32_t)Params->_scaling_mod_size;
  Upscale_ciph(&up, &ct, 10);
  CHECK(up._sf_degree == 2 && fabs(up._scaling_factor / ct._scaling_factor - 1024.0) < 1e-9, "Upscale_ciph scale");
  CHECK(Max_err(&up, x, slots) < 1e-5, "Upscale_ciph message");
  Downscale_ciph(&down, &up, sf_bits);
  /* the degree bookkeeping is the reference's: each scalar multiplication adds one, Downscale one more, the rescale takes one */
  CHECK(Level(&down) == L - 1 && down._sf_degree == 3 && fabs(down._scaling_factor / Get_default_sc() - 1.0) < 1e-9,
        "Downscale_ciph shape (level %zu degree %u)", Level(&down), down._sf_degree);
  CHECK(Max_err(&down, x, slots) < 1e-4, "Downscale_ciph message: %g", Max_err(&down, x, slots));

  /* Reset_ciph: limbs written back to back at a lower level are regrouped */
  {
    CIPHERTEXT low, work;
    memset(&low, 0, sizeof(low)), memset(&work, 0, sizeof(work));
    Copy_ciph(&low, &ct);
    for (size_t l = L; l > 2; --l) Modswitch_ciph(&low);
    CHECK(Level(&low) == 2, "Modswitch_ciph level");
    Copy_ciph(&work, &ct); /* allocated at L limbs */
    size_t lvl = 2;
    for (size_t i = 0; i < 2 * lvl; ++i) { /* what the per-limb generator does: limb i of the 2*lvl-limb result */
      L_POLY src = Lpoly_from_ciph(&low, i);
      L_POLY dst;
      Init_lpoly_data(&dst, N, work._c0_poly._data + i * (size_t)N);
      Copy_lpoly(&dst, src);
    }
    Reset_ciph(&work, lvl);
    CHECK(Level(&work) == lvl && Same(&work._c0_poly, &low._c0_poly) && Same(&work._c1_poly, &low._c1_poly), "Reset_ciph");
    L_POLY l0 = Lpoly_from_ciph(&low, 1);
    Set_ciph_data(&work, l0, 2); /* c1's limb 0 := c0's limb 1 */
    POLYNOMIAL v1 = work._c1_poly, v2 = low._c0_poly;
    v1._num_primes = 1, v1._num_alloc_primes = 1;
    v2._data += N, v2._num_primes = 1, v2._num_alloc_primes = 1;
    CHECK(Same(&v1, &v2), "Set_ciph_data");
    Free_ciph_poly(&low, 1), Free_ciph_poly(&work, 1);
  }
  /* rotations and the conjugation written over their operand (Fast_rotate builds its result in a temporary and
   * assigns it last, evaluator.c:503-522, so Rotate_ciph(&x, &x, k) is valid there): the words of the out-of-place
   * call */
  {
    CIPHERTEXT apart, inplace, many[3];
    memset(&apart, 0, sizeof(apart)), memset(&inplace, 0, sizeof(inplace)), memset(many, 0, sizeof(many));
    Rotate_ciph(&apart, &ct, 3);
    Copy_ciph(&inplace, &ct);
    Rotate_ciph(&inplace, &inplace, 3);
    CHECK(Same(&apart._c0_poly, &inplace._c0_poly) && Same(&apart._c1_poly, &inplace._c1_poly), "Rotate_ciph in place");
    double* want = (double*)malloc(slots * sizeof(double));
    for (uint32_t i = 0; i < slots; ++i) want[i] = x[(i + 3) % slots];
    CHECK(Max_err(&inplace, want, slots) < 1e-4, "Rotate_ciph in place, message: %g", Max_err(&inplace, want, slots));
    extern void* Rt_find_rot(int32_t rot_idx); /* the runtime's key registry; a deep chain has the key already */
    if (!Rt_find_rot((int32_t)(2 * N - 1))) Rt_generate_rotation_key((int32_t)(2 * N - 1));
    Conjugate_ciph(&apart, &ct);
    Copy_ciph(&inplace, &ct);
    Conjugate_ciph(&inplace, &inplace);
    CHECK(Same(&apart._c0_poly, &inplace._c0_poly) && Same(&apart._c1_poly, &inplace._c1_poly), "Conjugate_ciph in place");
    CHECK(Max_err(&inplace, x, slots) < 1e-4, "conjugate of a real message");
    /* a batch whose first result is the operand itself */
    int32_t idx[3] = {1, -1, 3};
    Copy_ciph(&many[0], &ct);
    Rotate_batch_ciph(many, &many[0], idx, 3);
    for (int k = 0; k < 3; ++k) {
      Rotate_ciph(&apart, &ct, idx[k]);
      CHECK(Same(&apart._c0_poly, &many[k]._c0_poly) && Same(&apart._c1_poly, &many[k]._c1_poly),
            "Rotate_batch_ciph over its operand, rotation %d", idx[k]);
    }
    free(want);
    Free_ciph_poly(&apart, 1), Free_ciph_poly(&inplace, 1);
    for (int k = 0; k < 3; ++k) Free_ciph_poly(&many[k], 1);
  }
  printf("ok ciph\n");

  /* Raise_mod from level 1: the message survives modulo q0 (values are small against q0 / scale) */
  {
    CIPHERTEXT low;
    memset(&low, 0, sizeof(low));
    PLAINTEXT p1;
    memset(&p1, 0, sizeof(p1));
    Encode_double(&p1, x, slots, 1, 1);
    Encrypt(&low, &p1);
    Raise_mod(&raised, &low, 3);
    CHECK(Level(&raised) == 3 && raised._sf_degree == 1, "Raise_mod shape");
    /* decrypting at 3 primes gives m + q0 * I; only its residue modulo q0 is the message: drop back to one prime */
    CIPHERTEXT back;
    memset(&back, 0, sizeof(back));
    Copy_ciph(&back, &raised);
    Set_poly_level(&back._c0_poly, 1), Set_poly_level(&back._c1_poly, 1);
    CHECK(Max_err(&back, x, slots) < 1e-4, "Raise_mod keeps the residues of q0: %g", Max_err(&back, x, slots));
    Free_ciph_poly(&low, 1), Free_ciph_poly(&back, 1), Free_plain_poly(&p1);
  }
  printf("ok raise\n");

  /* Encode_float_with_scale at 1.5 * the scaling factor */
  {
    float*    f = (float*)malloc(slots * sizeof(float));
    for (uint32_t i = 0; i < slots; ++i) f[i] = (float)x[i];
    PLAINTEXT ps;
    memset(&ps, 0, sizeof(ps));
    double scale = 1.5 * Get_default_sc();
    Encode_float_with_scale(&ps, f, slots, scale, (uint32_t)L);
    CHECK(ps._sf_degree == 2 && ps._scaling_factor == scale, "Encode_float_with_scale metadata");
    double* m = Get_msg_from_plain(&ps);
    double  e = 0;
    for (uint32_t i = 0; i < slots; ++i) e = fmax(e, fabs(m[i] - (double)f[i]));
    CHECK(e < 1e-6, "Encode_float_with_scale message: %g", e);
    free(m), free(f);
    Free_plain_poly(&ps);
  }
  /* Prepare_input_dup: 12 values repeated with period 16 over every slot */
  {
    double  img[12];
    for (int i = 0; i < 12; ++i) img[i] = 0.01 * (i + 1);
    TENSOR* t = Alloc_tensor(1, 3, 2, 2, img);
    Prepare_input_dup(t, "image");
    CIPHERTEXT in = Get_input_data("image", 0);
    double*    m  = Get_msg(&in);
    for (uint32_t i = 0; i < slots; ++i) {
      double want = (i % 16) < 12 ? img[i % 16] : 0.0;
      CHECK(fabs(m[i] - want) < 1e-5, "Prepare_input_dup slot %u: %g != %g", i, m[i], want);
    }
    free(m);
    TENSOR* s = Add_tensor(t, t);
    CHECK(Is_tensor_match(s, t) && s->_vals[11] == 2 * img[11], "Add_tensor");
    Free_tensor(s), Free_tensor(t);
    Free_ciph_poly(&in, 1);
  }
  /* Real_relu */
  {
    CIPHER   r = Real_relu(&ct);
    double*  want = (double*)malloc(slots * sizeof(double));
    for (uint32_t i = 0; i < slots; ++i) want[i] = x[i] > 0 ? x[i] : 0;
    CHECK(Level(r) == L && Max_err(r, want, slots) < 1e-5, "Real_relu");
    free(want);
    Free_cipher(r);
  }
  printf("ok encode\n");

  /* ---- a file of pre-encoded plaintexts, written with Encode_dcmplx_ext_buffer and read back by Pt_get ----- */
  {
    char path[64] = "/tmp/surface_pt_XXXXXX";
    int  fd = mkstemp(path);
    CHECK(fd >= 0, "mkstemp");
    FILE*   f = fdopen(fd, "wb");
    DCMPLX* z = (DCMPLX*)calloc(slots, sizeof(DCMPLX));
    struct PLAINTEXT_BUFFER* ent[2];
    for (int e = 0; e < 2; ++e) {
      for (uint32_t i = 0; i < slots; ++i) z[i] = x[i] * (e + 1);
      ent[e] = Encode_dcmplx_ext_buffer(z, slots, (uint32_t)(L - e), e ? (uint32_t)K : 0);
    }
    /* header (136 bytes), first page padded, the entries 4 KiB-aligned, then 32-byte lookup records */
    unsigned char hdr[136] = {0};
    memcpy(hdr, "!ANTFHE\0", 8);
    uint32_t ver = 1;
    memcpy(hdr + 8, &ver, 4);
    hdr[14] = DE_PLAINTEXT, hdr[15] = 12;
    uint64_t cnt = 2, ofs[2], sz[2], pos = 4096;
    for (int e = 0; e < 2; ++e) {
      ofs[e] = pos, sz[e] = 16 + (uint64_t)ent[e]->_size;
      pos += (sz[e] + 4095) & ~4095ull;
    }
    memcpy(hdr + 16, &cnt, 8);
    memcpy(hdr + 24, &pos, 8);
    fwrite(hdr, 1, sizeof(hdr), f);
    for (int e = 0; e < 2; ++e) {
      fseek(f, (long)ofs[e], SEEK_SET);
      fwrite(ent[e], 1, sz[e], f);
    }
    fseek(f, (long)pos, SEEK_SET);
    for (uint32_t e = 0; e < 2; ++e) {
      unsigned char rec[32] = {0};
      snprintf((char*)rec, 16, "pt%u", e);
      uint32_t size32 = (uint32_t)sz[e];
      memcpy(rec + 16, &e, 4);
      memcpy(rec + 20, &size32, 4);
      uint64_t packed = 1ull | ((uint64_t)(L - e) << 8) | (ofs[e] << 16);
      memcpy(rec + 24, &packed, 8);
      fwrite(rec, 1, 32, f);
    }
    fclose(f);
    CHECK(Pt_mgr_init(path), "Pt_mgr_init on a plaintext file");
    Has_file = 1;
    Pt_prefetch(1);
    PLAIN p0 = (PLAIN)Pt_get(0, slots, 1, (uint32_t)L);
    CHECK(Same(&p0->_poly, &pt._poly) && p0->_sf_degree == 1 && p0->_poly._is_ntt, "Pt_get entry 0 differs from Encode_double");
    CIPHERTEXT m1, m2;
    memset(&m1, 0, sizeof(m1)), memset(&m2, 0, sizeof(m2));
    Mul_plain(&m1, &ct, p0);
    Mul_plain(&m2, &ct, &pt);
    CHECK(Same(&m1._c0_poly, &m2._c0_poly) && Same(&m1._c1_poly, &m2._c1_poly), "Mul_plain with a plaintext of Pt_get");
    PLAIN     p1 = (PLAIN)Pt_get(1, slots, 1, (uint32_t)(L - 1));
    PLAINTEXT direct;
    memset(&direct, 0, sizeof(direct));
    for (uint32_t i = 0; i < slots; ++i) z[i] = x[i] * 2;
    Encode_dcmplx_ext(&direct, z, slots, (uint32_t)(L - 1), (uint32_t)K);
    CHECK(Num_p(&p1->_poly) == K && Same(&p1->_poly, &direct._poly), "Pt_get entry 1 (extended) differs from Encode_dcmplx_ext");
    Free_data(&p1->_poly); /* must leave the manager's plaintext alone */
    CHECK(p1->_poly._data != NULL, "Free_data freed a plaintext of Pt_get");
    Pt_free(0), Pt_free(1);
    Pt_mgr_fini();
    Has_file = 0;
    unlink(path);
    free(ent[0]), free(ent[1]), free(z);
    Free_ciph_poly(&m1, 1), Free_ciph_poly(&m2, 1), Free_plain_poly(&direct);
  }
  printf("ok plaintext file\n");

  /* ---- the staged bootstrap operators give what the whole operator gives ---------------------------------- */
  if (bootstrap) {
    CIPHERTEXT low, whole, staged;
    PLAINTEXT  p1;
    memset(&low, 0, sizeof(low)), memset(&whole, 0, sizeof(whole)), memset(&staged, 0, sizeof(staged)), memset(&p1, 0, sizeof(p1));
    Encode_double(&p1, x, slots, 1, 1);
    Encrypt(&low, &p1);
    Eval_bootstrap_ciph(&whole, &low, 0, slots);
    Eval_bootstrap_coeffs_to_slots_ciph(&staged, &low, slots);
    Eval_bootstrap_eval_mod_ciph(&staged, &staged, slots);
    Eval_bootstrap_slots_to_coeffs_ciph(&staged, &staged, slots);
    CHECK(Level(&staged) == Level(&whole), "staged bootstrap level %zu, whole %zu", Level(&staged), Level(&whole));
    /* raised to all primes in both cases here (level_after_bts = 0), so the two are the same computation */
    CHECK(Same(&staged._c0_poly, &whole._c0_poly) && Same(&staged._c1_poly, &whole._c1_poly),
          "staged bootstrap differs from Eval_bootstrap_ciph");
    CHECK(Max_err(&staged, x, slots) < 1e-3, "staged bootstrap message: %g", Max_err(&staged, x, slots));
    printf("ok staged bootstrap (max_err %.3g, level %zu)\n", Max_err(&staged, x, slots), Level(&staged));
  }

  Finalize_context();
  printf("surface ok\n");
  return 0;
}
