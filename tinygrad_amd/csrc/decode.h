// Device-resident decode bookkeeping shared by the decode-step kernels.
#pragma once
#include <stdint.h>

struct DecodeState {   // 16 int32
  int pos;             // position of the token being processed
  int token;           // current input token id
  int step;            // tokens generated so far
  int n_prompt;        // prompt length: while pos + 1 < n_prompt the next input token comes from the prompt, not from argmax
  int error;           // set by kernels that refuse their input instead of reading out of bounds: bit 0 token id outside the table, bit 1 position >= max_ctx
  int vocab;           // rows of the embedding table (0: unknown, token ids are then not checked)
  int pad[10];
};
