#define WC_K0 KIND_22
#define WC_PICK_NAME pick_in_3d_22
#include "input_transform_3d.inc"
