/* Decoder / GPT half of the CPU oracle -- TEST INFRASTRUCTURE ONLY (see ls_oracle.h). */
#include "ls_oracle.h"
