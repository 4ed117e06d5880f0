/* Plaintexts from a weight side-file through the program-facing runtime: Pt_from_msg, Pt_from_msg_ofst and
 * the validating forms (reference: rtlib/ant/porting/pt_mgr.c:188-243).
 *
 * usage: msg_program <side-file> <N> <mul_depth> <q0_bits> <sf_bits> <parts> <level> <output file> {<index> <ofst> <len>}...
 * output: for each triple, level*N words of the plaintext polynomial
 */
#include "rt_ant/rt_ant.h"

static CKKS_PARAMS  Params = {._provider = LIB_ANT};
static RT_DATA_INFO Info   = {NULL, "XXXXXXXX-XXXX-XXXX-XXXX-XXXXXXXXXXXX", DE_MSG_F32};
CKKS_PARAMS*        Get_context_params(void) { return &Params; }
RT_DATA_INFO*       Get_rt_data_info(void) { return &Info; }

int main(int argc, char** argv) {
  if (argc < 9 || (argc - 9) % 3) return 2;
  Info._file_name          = argv[1];
  Params._poly_degree      = (uint32_t)strtoul(argv[2], NULL, 0);
  Params._mul_depth        = strtoul(argv[3], NULL, 0);
  Params._first_mod_size   = strtoul(argv[4], NULL, 0);
  Params._scaling_mod_size = strtoul(argv[5], NULL, 0);
  Params._num_q_parts      = strtoul(argv[6], NULL, 0);
  uint32_t level           = (uint32_t)strtoul(argv[7], NULL, 0);
  Prepare_context();
  FILE*    out   = fopen(argv[8], "wb");
  size_t   words = (size_t)level * Degree();
  int64_t* host  = (int64_t*)malloc(words * sizeof(int64_t));
  for (int a = 9; a < argc; a += 3) {
    uint32_t  index = (uint32_t)strtoul(argv[a], NULL, 0);
    size_t    ofst = strtoul(argv[a + 1], NULL, 0), len = strtoul(argv[a + 2], NULL, 0);
    PLAINTEXT pt;
    memset(&pt, 0, sizeof(pt));
    if (ofst)
      Pt_from_msg_ofst(&pt, index, ofst, len, 1, level);
    else
      Pt_from_msg(&pt, index, len, 1, level);
    Rt_download_poly(host, &pt._poly);
    fwrite(host, sizeof(int64_t), words, out);
    Free_data(&pt._poly);
  }
  fclose(out);
  free(host);
  Finalize_context();
  return 0;
}
