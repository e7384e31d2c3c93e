// MIOpen FP32 forward convolution as a comparator library (the `-s miopen` rows of the benchmark scripts).
// Role in the reference: src_template/Ampere_FP32/cudnn_fp32.cu.  The implementation is shared with the FP16
// comparator: common/helix_miopen.h.
#define MIOPEN_ELEM_TYPE miopenFloat
#define MIOPEN_ELEM_BYTES 4
#include "helix_miopen.h"
