/* CPU oracle -- TEST INFRASTRUCTURE. Weight descriptors shared by the oracle's files. */
#ifndef ORC_TYPES_H
#define ORC_TYPES_H
#include "orc_common.h"

typedef struct orc_kmat {
  int kind, E, O, K;
  const uint8_t* qs;
  const uint8_t* scales;
  const f16_t* dm;
} orc_kmat;

typedef struct orc_linear {
  int mode; /* 0 = k-quant (km), 1 = 8-bit affine g64, 2 = dense bf16; km.O / km.K hold the dims */
  orc_kmat km;
  const uint8_t* aw; /* affine: u8[O,K]; dense: bf16[O,K] */
  const bf16_t* as;
  const bf16_t* ab;
} orc_linear;

typedef struct orc_moe_weights {
  orc_linear router;         /* [E, H] */
  orc_kmat ex_gate, ex_up;   /* [E, I, H] */
  orc_kmat ex_down;          /* [E, H, I] */
  orc_linear sh_gate, sh_up; /* [I, H] */
  orc_linear sh_down;        /* [H, I] */
  orc_linear sh_egate;       /* [1, H] */
  int top_k, normalize;
} orc_moe_weights;
#endif
