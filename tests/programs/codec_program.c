/* Plaintext encoding and decoding through the program-facing runtime, for parity checks of
 * Encode_dcmplx / Encode_double (one value) / Get_dcmplx_msg_from_plain against the oracle
 * (reference: rtlib/ant/ckks/src/plain.c:21-73,149-165, encoder.c:234-326,473-575,657-704).
 *
 * usage: codec_program <input file> <output file>
 * input  (int64 words): N, mul_depth, q0_bits, sf_bits, parts, level, sf_degree, n_values,
 *                       then 2*n_values doubles (re, im)
 * output: level*N words of Encode_dcmplx, N/2 (re, im) doubles of its decoding,
 *         level*N words of Encode_double of the first value's real part
 */
#include "rt_ant/rt_ant.h"

static CKKS_PARAMS Params = {._provider = LIB_ANT};
CKKS_PARAMS*       Get_context_params(void) { return &Params; }

int main(int argc, char** argv) {
  if (argc != 3) return 2;
  FILE*   in = fopen(argv[1], "rb");
  int64_t h[8];
  if (!in || fread(h, sizeof(int64_t), 8, in) != 8) return 2;
  size_t  n_values = (size_t)h[7];
  DCMPLX* values   = (DCMPLX*)malloc(n_values * sizeof(DCMPLX));
  if (fread(values, sizeof(DCMPLX), n_values, in) != n_values) return 2;
  fclose(in);
  Params._poly_degree      = (uint32_t)h[0];
  Params._mul_depth        = (size_t)h[1];
  Params._first_mod_size   = (size_t)h[2];
  Params._scaling_mod_size = (size_t)h[3];
  Params._num_q_parts      = (size_t)h[4];
  uint32_t level = (uint32_t)h[5], sf_degree = (uint32_t)h[6];

  Prepare_context();
  size_t    words = (size_t)level * Degree();
  int64_t*  host  = (int64_t*)malloc(words * sizeof(int64_t));
  FILE*     out   = fopen(argv[2], "wb");
  PLAINTEXT pt;
  memset(&pt, 0, sizeof(pt));
  Encode_dcmplx(&pt, values, n_values, sf_degree, level);
  Rt_download_poly(host, &pt._poly);
  fwrite(host, sizeof(int64_t), words, out);
  DCMPLX* msg = Get_dcmplx_msg_from_plain(&pt);
  fwrite(msg, sizeof(DCMPLX), Degree() / 2, out);
  free(msg);
  double first = __real__ values[0];
  Encode_double(&pt, &first, 1, sf_degree, level);
  Rt_download_poly(host, &pt._poly);
  fwrite(host, sizeof(int64_t), words, out);
  fclose(out);
  Free_plain_poly(&pt);
  free(host);
  free(values);
  Finalize_context();
  return 0;
}
