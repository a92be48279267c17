#define WC_K0 KIND_23
#define WC_PICK_NAME pick_in_3d_23
#include "input_transform_3d.inc"
