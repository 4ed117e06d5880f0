/* Writes the key material that Rt_generate_keys builds on the device, for a check of every key against the
 * equation that defines it (Generate_switching_key, rtlib/ant/ckks/src/key_gen.c:127-262).
 *
 * usage: keygen_program <out file> <poly degree> <mul depth> <q0 bits> <scale bits> <hamming weight> <seed> <rot idx>...
 * out file, int64 words: the secret (N signed coefficients), pk0, pk1 (L limbs each), the relinearisation key,
 * then one key per rotation index in the order given (2N-1 = conjugation); a key is
 * [digit][b | a][(L+k) limbs][N], NTT form.
 */
#include "rt_ant/rt_ant.h"

static CKKS_PARAMS* Params;
CKKS_PARAMS*        Get_context_params(void) { return Params; }

static void Write_key(FILE* f, SW_KEY key, int64_t* buf, size_t words) {
  for (size_t d = 0; d < Get_swk_size(key); ++d) {
    Rt_download_poly(buf, Pk0_at(key, (uint32_t)d));
    fwrite(buf, sizeof(int64_t), words, f);
    Rt_download_poly(buf, Pk1_at(key, (uint32_t)d));
    fwrite(buf, sizeof(int64_t), words, f);
  }
}

int main(int argc, char** argv) {
  if (argc < 8) {
    fprintf(stderr, "usage: %s <out> <degree> <depth> <q0 bits> <scale bits> <hamming weight> <seed> <rot idx>...\n", argv[0]);
    return 2;
  }
  size_t n_rot = (size_t)argc - 8;
  Params = (CKKS_PARAMS*)calloc(1, sizeof(CKKS_PARAMS) + n_rot * sizeof(int32_t));
  Params->_provider         = LIB_ANT;
  Params->_poly_degree      = (uint32_t)strtoul(argv[2], NULL, 0);
  Params->_mul_depth        = strtoul(argv[3], NULL, 0);
  Params->_first_mod_size   = strtoul(argv[4], NULL, 0);
  Params->_scaling_mod_size = strtoul(argv[5], NULL, 0);
  Params->_hamming_weight   = strtoul(argv[6], NULL, 0);
  Prepare_context();
  Rt_generate_keys(strtoull(argv[7], NULL, 0));
  uint32_t N = Degree();
  size_t   L = Get_q_cnt(), T = L + Get_p_cnt();
  FILE*    f = fopen(argv[1], "wb");
  if (!f) return 3;
  int64_t* buf = (int64_t*)malloc(T * N * sizeof(int64_t));
  int64_t* pk1 = (int64_t*)malloc(L * N * sizeof(int64_t));
  Rt_get_secret(buf);
  fwrite(buf, sizeof(int64_t), N, f);
  Rt_get_public_key(buf, pk1);
  fwrite(buf, sizeof(int64_t), L * N, f);
  fwrite(pk1, sizeof(int64_t), L * N, f);
  Write_key(f, Swk(false, 0), buf, T * N);
  for (size_t i = 0; i < n_rot; ++i) {
    int32_t rot = (int32_t)strtol(argv[8 + i], NULL, 0);
    Rt_generate_rotation_key(rot);
    Write_key(f, Swk(true, rot), buf, T * N);
  }
  fclose(f);
  free(buf), free(pk1);
  Finalize_context();
  printf("keygen ok\n");
  return 0;
}
