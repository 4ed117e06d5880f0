/* A program in the shape the FHE compiler emits for the ANT runtime, run against
 * the HIP-backed runtime.  Key switching is open-coded at polynomial / limb
 * granularity exactly as generated code does it (Decomp_modup per digit, one
 * Hw_modmul + Hw_modadd pair per limb and key half, Mod_down, Hw_rotate),
 * cf. the Rotate and Relinearize bodies of the reference's fixtures
 * (rtlib/ant/dataset/resnet20_cifar10_pre.onnx.inc:6974-7148,
 *  rtlib/ant/example/eg_fhertlib_relin.inc:36-150).
 *
 * Main_graph:
 *   prod   = input * input                    (tensor product, 3 polynomials)
 *   lin    = Relinearize(prod)                (open-coded key switch of c2; digits by Decomp + Mod_up)
 *   res    = rescale(lin)                     -> output 0
 *   rot[i] = Rotate(res, rot_idx[i])          (open-coded; digits by Decomp_modup) -> outputs 1..n
 *   lib    = Rescale_ciph(Mul_ciph(in, in))   (library form)                        -> output n+1
 *   Rotate_batch_ciph(lib, all rot_idx)       (library form, hoisted)               -> outputs n+2..2n+1
 *
 * usage: keyswitch_program <input file> <output file>
 * input file (little-endian int64 words):
 *   N, mul_depth, q0_bits, sf_bits, parts, n_rot, rot_idx[n_rot],
 *   relin key [parts][2][(L+k)][N], n_rot rotation keys of the same shape,
 *   input c0 [L][N], input c1 [L][N]
 * output file: for each output: level, c0 [level][N], c1 [level][N]
 */
#include "rt_ant/rt_ant.h"

static CKKS_PARAMS* Params;
static int32_t*     Rot;
static uint32_t     N_rot;

CKKS_PARAMS* Get_context_params(void) { return Params; }
int          Get_input_count(void) { return 1; }
int          Get_output_count(void) { return (int)(2 * N_rot + 2); }

/* acc_c0/acc_c1 (level + p limbs, zero on entry) += ext * key halves of one digit */
static void Accumulate_digit(POLY acc_c0, POLY acc_c1, POLY ext, POLY key0, POLY key1, POLY tmp, uint32_t degree) {
  MODULUS* modulus = Q_modulus();
  uint32_t num_q   = Poly_level(ext);
  for (uint32_t i = 0; i < num_q; i++) {
    Hw_modmul(Coeffs(tmp, 0, degree), Coeffs(key0, i, degree), Coeffs(ext, i, degree), modulus, degree);
    Hw_modadd(Coeffs(acc_c0, i, degree), Coeffs(acc_c0, i, degree), Coeffs(tmp, 0, degree), modulus, degree);
    Hw_modmul(Coeffs(tmp, 0, degree), Coeffs(key1, i, degree), Coeffs(ext, i, degree), modulus, degree);
    Hw_modadd(Coeffs(acc_c1, i, degree), Coeffs(acc_c1, i, degree), Coeffs(tmp, 0, degree), modulus, degree);
    modulus = modulus + 1;
  }
  modulus             = P_modulus();
  uint32_t num_p      = Num_p(ext);
  uint32_t p_ofst     = Num_alloc(ext) - num_p;
  uint32_t key_p_ofst = Poly_level(key0);
  for (uint32_t j = 0; j < num_p; j++) {
    uint32_t p_idx = j + p_ofst, key_p_idx = j + key_p_ofst;
    Hw_modmul(Coeffs(tmp, 0, degree), Coeffs(key0, key_p_idx, degree), Coeffs(ext, p_idx, degree), modulus, degree);
    Hw_modadd(Coeffs(acc_c0, p_idx, degree), Coeffs(acc_c0, p_idx, degree), Coeffs(tmp, 0, degree), modulus, degree);
    Hw_modmul(Coeffs(tmp, 0, degree), Coeffs(key1, key_p_idx, degree), Coeffs(ext, p_idx, degree), modulus, degree);
    Hw_modadd(Coeffs(acc_c1, p_idx, degree), Coeffs(acc_c1, p_idx, degree), Coeffs(tmp, 0, degree), modulus, degree);
    modulus = modulus + 1;
  }
}

static CIPHERTEXT Relinearize(CIPHERTEXT3 ciph3) {
  CIPHERTEXT res;
  uint32_t   degree = Degree();
  memset(&res, 0, sizeof(res));
  Init_ciph_same_scale_ciph3(&res, &ciph3);
  size_t level  = Poly_level(&ciph3._c2_poly);
  POLY   swk_c0 = Alloc_poly(degree, level, Get_p_cnt());
  POLY   swk_c1 = Alloc_poly(degree, level, Get_p_cnt());
  POLY   ext    = Alloc_poly(degree, level, Get_p_cnt());
  POLY   tmp    = Alloc_poly(degree, 1, 0);
  POLY   md_c0  = Alloc_poly(degree, level, 0);
  POLY   md_c1  = Alloc_poly(degree, level, 0);
  POLY   decomp = Alloc_poly(degree, level, 0);
  SWITCH_KEY* swk = Swk(0, 0);
  for (uint32_t part = 0; part < Num_decomp(&ciph3._c2_poly); part++) {
    Decomp(decomp, &ciph3._c2_poly, part);
    Mod_up(ext, decomp, part);
    Accumulate_digit(swk_c0, swk_c1, ext, Pk0_at(swk, part), Pk1_at(swk, part), tmp, degree);
  }
  Mod_down(md_c0, swk_c0);
  Mod_down(md_c1, swk_c1);
  MODULUS* modulus = Q_modulus();
  for (uint32_t i = 0; i < level; i++) {
    Hw_modadd(Coeffs(&res._c0_poly, i, degree), Coeffs(md_c0, i, degree), Coeffs(&ciph3._c0_poly, i, degree), modulus,
              degree);
    Hw_modadd(Coeffs(&res._c1_poly, i, degree), Coeffs(md_c1, i, degree), Coeffs(&ciph3._c1_poly, i, degree), modulus,
              degree);
    modulus = modulus + 1;
  }
  Free_poly(swk_c0);
  Free_poly(swk_c1);
  Free_poly(ext);
  Free_poly(tmp);
  Free_poly(md_c0);
  Free_poly(md_c1);
  Free_poly(decomp);
  return res;
}

static CIPHERTEXT Rotate(CIPHERTEXT ciph, int32_t rot_idx) {
  CIPHERTEXT res;
  uint32_t   degree = Degree();
  memset(&res, 0, sizeof(res));
  Init_ciph_same_scale(&res, &ciph, 0);
  size_t level  = Poly_level(&ciph._c1_poly);
  POLY   swk_c0 = Alloc_poly(degree, level, Get_p_cnt());
  POLY   swk_c1 = Alloc_poly(degree, level, Get_p_cnt());
  POLY   ext    = Alloc_poly(degree, level, Get_p_cnt());
  POLY   tmp    = Alloc_poly(degree, 1, 0);
  POLY   md_c0  = Alloc_poly(degree, level, 0);
  POLY   md_c1  = Alloc_poly(degree, level, 0);
  SWITCH_KEY* swk = Swk(1, rot_idx);
  for (uint32_t part = 0; part < Num_decomp(&ciph._c1_poly); part++) {
    Decomp_modup(ext, &ciph._c1_poly, part);
    Accumulate_digit(swk_c0, swk_c1, ext, Pk0_at(swk, part), Pk1_at(swk, part), tmp, degree);
  }
  Mod_down(md_c0, swk_c0);
  Mod_down(md_c1, swk_c1);
  MODULUS* modulus = Q_modulus();
  for (uint32_t i = 0; i < level; i++) {
    Hw_modadd(Coeffs(md_c0, i, degree), Coeffs(md_c0, i, degree), Coeffs(&ciph._c0_poly, i, degree), modulus, degree);
    modulus = modulus + 1;
  }
  int64_t* order = Auto_order(rot_idx);
  modulus        = Q_modulus();
  for (uint32_t i = 0; i < level; i++) {
    Hw_rotate(Coeffs(&res._c0_poly, i, degree), Coeffs(md_c0, i, degree), order, modulus, degree);
    Hw_rotate(Coeffs(&res._c1_poly, i, degree), Coeffs(md_c1, i, degree), order, modulus, degree);
    modulus = modulus + 1;
  }
  Free_poly(swk_c0);
  Free_poly(swk_c1);
  Free_poly(ext);
  Free_poly(tmp);
  Free_poly(md_c0);
  Free_poly(md_c1);
  return res;
}

bool Main_graph(void) {
  CIPHERTEXT  input, scaled, lib_prod, lib_scaled;
  CIPHERTEXT3 prod;
  uint32_t    degree = Degree();
  input              = Get_input_data("input", 0);
  memset(&scaled, 0, sizeof(scaled));
  memset(&prod, 0, sizeof(prod));
  memset(&lib_prod, 0, sizeof(lib_prod));
  memset(&lib_scaled, 0, sizeof(lib_scaled));

  /* tensor product, limb by limb */
  Init_ciph3_up_scale(&prod, &input, &input);
  {
    MODULUS* modulus = Q_modulus();
    uint32_t num_q   = Poly_level(&prod._c0_poly);
    POLY     t1 = Alloc_poly(degree, 1, 0), t2 = Alloc_poly(degree, 1, 0);
    for (uint32_t i = 0; i < num_q; i++) {
      Hw_modmul(Coeffs(t1, 0, degree), Coeffs(&input._c0_poly, i, degree), Coeffs(&input._c1_poly, i, degree), modulus,
                degree);
      Hw_modmul(Coeffs(t2, 0, degree), Coeffs(&input._c1_poly, i, degree), Coeffs(&input._c0_poly, i, degree), modulus,
                degree);
      Hw_modmul(Coeffs(&prod._c0_poly, i, degree), Coeffs(&input._c0_poly, i, degree),
                Coeffs(&input._c0_poly, i, degree), modulus, degree);
      Hw_modadd(Coeffs(&prod._c1_poly, i, degree), Coeffs(t1, 0, degree), Coeffs(t2, 0, degree), modulus, degree);
      Hw_modmul(Coeffs(&prod._c2_poly, i, degree), Coeffs(&input._c1_poly, i, degree),
                Coeffs(&input._c1_poly, i, degree), modulus, degree);
      modulus = modulus + 1;
    }
    Free_poly(t1);
    Free_poly(t2);
  }
  CIPHERTEXT lin = Relinearize(prod);
  Init_ciph_down_scale(&scaled, &lin);
  Rescale(&scaled._c0_poly, &lin._c0_poly);
  Rescale(&scaled._c1_poly, &lin._c1_poly);

  for (uint32_t r = 0; r < N_rot; r++) {
    CIPHERTEXT rot = Rotate(scaled, Rot[r]);
    Set_output_data("output", 1 + r, &rot);
  }

  /* the same through the library-level entry points */
  Mul_ciph(&lib_prod, &input, &input);
  Rescale_ciph(&lib_scaled, &lib_prod);
  CIPHERTEXT* batch = (CIPHERTEXT*)calloc(N_rot ? N_rot : 1, sizeof(CIPHERTEXT));
  Rotate_batch_ciph(batch, &lib_scaled, Rot, N_rot);
  for (uint32_t r = 0; r < N_rot; r++) Set_output_data("output", N_rot + 2 + r, &batch[r]);
  free(batch);

  Set_output_data("output", 0, &scaled);
  Set_output_data("output", N_rot + 1, &lib_scaled);
  Free_ciph_poly(&input, 1);
  Free_ciph_poly(&lin, 1);
  Free_ciph_poly(&lib_prod, 1);
  Free_poly_data(&prod._c0_poly);
  Free_poly_data(&prod._c1_poly);
  Free_poly_data(&prod._c2_poly);
  return true;
}

static int64_t* Read_words(FILE* f, size_t n) {
  int64_t* p = (int64_t*)malloc(n * sizeof(int64_t));
  if (!p || fread(p, sizeof(int64_t), n, f) != n) {
    fprintf(stderr, "keyswitch_program: short read (%zu words)\n", n);
    exit(2);
  }
  return p;
}

int main(int argc, char** argv) {
  if (argc != 3) {
    fprintf(stderr, "usage: %s <input file> <output file>\n", argv[0]);
    return 2;
  }
  FILE* in = fopen(argv[1], "rb");
  if (!in) {
    perror(argv[1]);
    return 2;
  }
  int64_t* head = Read_words(in, 6);
  N_rot         = (uint32_t)head[5];
  Params        = (CKKS_PARAMS*)calloc(1, sizeof(CKKS_PARAMS) + N_rot * sizeof(int32_t));
  Params->_provider         = LIB_ANT;
  Params->_poly_degree      = (uint32_t)head[0];
  Params->_mul_depth        = (size_t)head[1];
  Params->_first_mod_size   = (size_t)head[2];
  Params->_scaling_mod_size = (size_t)head[3];
  Params->_num_q_parts      = (size_t)head[4];
  Params->_num_rot_idx      = N_rot;
  int64_t* rots             = N_rot ? Read_words(in, N_rot) : NULL;
  Rot                       = Params->_rot_idxs;
  for (uint32_t r = 0; r < N_rot; r++) Rot[r] = (int32_t)rots[r];

  Prepare_context();
  size_t n = Degree(), L = Get_q_cnt(), key_words = 2 * Get_q_parts() * (L + Get_p_cnt()) * n;
  int64_t* key = Read_words(in, key_words);
  Rt_load_switch_key(false, 0, key);
  for (uint32_t r = 0; r < N_rot; r++) {
    if (fread(key, sizeof(int64_t), key_words, in) != key_words) return 2;
    Rt_load_switch_key(true, Rot[r], key);
  }
  int64_t *c0 = Read_words(in, L * n), *c1 = Read_words(in, L * n);
  fclose(in);
  double sc = Get_default_sc();
  Rt_set_input("input", 0, c0, c1, L, sc, 1, (uint32_t)(n / 2));

  Tm_start("Main_graph");
  Run_main_graph();
  Tm_taken("Main_graph");

  FILE* out = fopen(argv[2], "wb");
  if (!out) {
    perror(argv[2]);
    return 2;
  }
  int n_out = Get_output_count();
  for (int i = 0; i < n_out; i++) {
    int64_t level = (int64_t)Rt_get_output("output", (size_t)i, c0, c1, NULL);
    if (level == 0) {
      fprintf(stderr, "keyswitch_program: output %d missing\n", i);
      return 3;
    }
    fwrite(&level, sizeof(level), 1, out);
    fwrite(c0, sizeof(int64_t), (size_t)level * n, out);
    fwrite(c1, sizeof(int64_t), (size_t)level * n, out);
  }
  fclose(out);
  Finalize_context();
  free(key);
  free(c0);
  free(c1);
  free(head);
  free(rots);
  printf("keyswitch_program: %d outputs written\n", n_out);
  return 0;
}
