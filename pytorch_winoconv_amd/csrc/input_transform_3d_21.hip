#define WC_K0 KIND_21
#define WC_PICK_NAME pick_in_3d_21
#include "input_transform_3d.inc"
