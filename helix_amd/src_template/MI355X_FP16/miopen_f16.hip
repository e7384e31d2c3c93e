// MIOpen FP16 forward convolution as a comparator library (the `-s miopen` rows of the benchmark scripts).
// Role in the reference: src_template/Ampere_FP16/cudnn_fp16.cu.  The implementation is shared with the FP32
// comparator: common/helix_miopen.h.
#define MIOPEN_ELEM_TYPE miopenHalf
#define MIOPEN_ELEM_BYTES 2
#include "helix_miopen.h"
