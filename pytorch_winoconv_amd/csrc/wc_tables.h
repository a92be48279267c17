// Winograd transform matrices as compile-time tables.
//
// Kinds (one per axis of a piece):
//   KIND_11  F(1,1)  alpha 1   size-1 axis (the depth of a 2-D problem)
//   KIND_21  F(2,1)  alpha 2   (reference literal: matrix_conv.py:15-20)
//   KIND_22  F(2,2)  alpha 3   (reference literal: matrix_convnd.py:20-27)
//   KIND_23  F(2,3)  alpha 4   (reference literal: matrix_conv.py:21-30)
//   KIND_43  F(4,3)  alpha 6   Cook-Toom over the points 0, 1, -1, 2, -2 - the point set the
//                              reference uses for F(2,5) (matrix_conv.py:33); BT equals the
//                              reference's commented B25 (transform.py:35-40).
//   KIND_41  F(4,1)  alpha 4   identity, like the reference's F(2,1) literal (matrix_conv.py:15-20)
//   KIND_42  F(4,2)  alpha 5   Cook-Toom over the points 0, 1, -1, 2 (the reference's point set
//                              for F(2,4), matrix_conv.py:32), same construction as wincnn.py:49-70
//   KIND_24..KIND_27  F(2,4)..F(2,7)  alpha 5..8   whole-kernel tiles of the reference's PyTorch
//                              path: Cook-Toom (wincnn.py:49-70) over the points 0, 1, -1, 2 for
//                              r = 4, 0, 1, -1, 2, -2 for r = 5 and 0, 1, -1, 1/2, -1/2, 1/3, -1/3
//                              for r = 6, 7 (matrix_conv.py:31-35)
//   KIND_33  F(3,3)  alpha 5   Cook-Toom over the points 0, 1, -1, 2 (wincnn.py:49-70): the tile of the
//                              DWM plans whose three-tap pieces share one transformed input
// KIND_41 / KIND_42 serve the pieces of a decomposed (DWM) kernel when the output tile is 4.
// AT is m x alpha, G is alpha x r, BT is alpha x alpha.
#pragma once
#include "wc_common.h"

namespace wc {

enum Kind { KIND_11 = 0, KIND_21 = 1, KIND_22 = 2, KIND_23 = 3, KIND_43 = 4, KIND_41 = 5, KIND_42 = 6,
            KIND_24 = 7, KIND_25 = 8, KIND_26 = 9, KIND_27 = 10, KIND_33 = 11, KIND_COUNT = 12 };

__host__ __device__ constexpr int kind_m(int k) {
  return k == KIND_11 ? 1 : k == KIND_33 ? 3 : (k == KIND_43 || k == KIND_41 || k == KIND_42) ? 4 : 2;
}
__host__ __device__ constexpr int kind_r(int k) {
  return k == KIND_33 ? 3 : k >= KIND_24 ? 4 + (k - KIND_24)
       : (k == KIND_11 || k == KIND_21 || k == KIND_41) ? 1 : (k == KIND_22 || k == KIND_42) ? 2 : 3;
}
__host__ __device__ constexpr int kind_alpha(int k) { return kind_m(k) + kind_r(k) - 1; }

// kind for (m, r); -1 if the pair is not supported
inline int kind_of(int m, int r) {
  if (m == 1 && r == 1) return KIND_11;
  if (m == 2 && r >= 1 && r <= 3) return KIND_21 + (r - 1);
  if (m == 2 && r >= 4 && r <= 7) return KIND_24 + (r - 4);
  if (m == 4 && r == 3) return KIND_43;
  if (m == 4 && r == 1) return KIND_41;
  if (m == 4 && r == 2) return KIND_42;
  if (m == 3 && r == 3) return KIND_33;
  return -1;
}

template <int KIND> struct Mats;

template <> struct Mats<KIND_11> {
  static constexpr int m = 1, r = 1, alpha = 1;
  __host__ __device__ static constexpr float at(int i, int j) { return 1.f; }
  __host__ __device__ static constexpr float g(int i, int j) { return 1.f; }
  __host__ __device__ static constexpr float bt(int i, int j) { return 1.f; }
};
template <> struct Mats<KIND_21> {
  static constexpr int m = 2, r = 1, alpha = 2;
  __host__ __device__ static constexpr float at(int i, int j) { return i == j ? 1.f : 0.f; }
  __host__ __device__ static constexpr float g(int i, int j) { return 1.f; }
  __host__ __device__ static constexpr float bt(int i, int j) { return i == j ? 1.f : 0.f; }
};
template <> struct Mats<KIND_22> {
  static constexpr int m = 2, r = 2, alpha = 3;
  __host__ __device__ static constexpr float at(int i, int j) {
    constexpr float t[2][3] = {{1, 1, 0}, {0, 1, 1}};
    return t[i][j];
  }
  __host__ __device__ static constexpr float g(int i, int j) {
    constexpr float t[3][2] = {{1, 0}, {1, 1}, {0, 1}};
    return t[i][j];
  }
  __host__ __device__ static constexpr float bt(int i, int j) {
    constexpr float t[3][3] = {{1, -1, 0}, {0, 1, 0}, {0, -1, 1}};
    return t[i][j];
  }
};
template <> struct Mats<KIND_23> {
  static constexpr int m = 2, r = 3, alpha = 4;
  __host__ __device__ static constexpr float at(int i, int j) {
    constexpr float t[2][4] = {{1, 1, 1, 0}, {0, 1, -1, -1}};
    return t[i][j];
  }
  __host__ __device__ static constexpr float g(int i, int j) {
    constexpr float t[4][3] = {{1, 0, 0}, {.5f, .5f, .5f}, {.5f, -.5f, .5f}, {0, 0, 1}};
    return t[i][j];
  }
  __host__ __device__ static constexpr float bt(int i, int j) {
    constexpr float t[4][4] = {{1, 0, -1, 0}, {0, 1, 1, 0}, {0, -1, 1, 0}, {0, 1, 0, -1}};
    return t[i][j];
  }
};
template <> struct Mats<KIND_33> {
  static constexpr int m = 3, r = 3, alpha = 5;
  __host__ __device__ static constexpr float at(int i, int j) {
    constexpr float t[3][5] = {{1, 1, 1, 1, 0}, {0, 1, -1, 2, 0}, {0, 1, 1, 4, 1}};
    return t[i][j];
  }
  __host__ __device__ static constexpr float g(int i, int j) {
    constexpr float t[5][3] = {{1.f / 2, 0, 0},
                               {-1.f / 2, -1.f / 2, -1.f / 2},
                               {-1.f / 6, 1.f / 6, -1.f / 6},
                               {1.f / 6, 1.f / 3, 2.f / 3},
                               {0, 0, 1}};
    return t[i][j];
  }
  __host__ __device__ static constexpr float bt(int i, int j) {
    constexpr float t[5][5] = {{2, -1, -2, 1, 0}, {0, -2, -1, 1, 0}, {0, 2, -3, 1, 0}, {0, -1, 0, 1, 0}, {0, 2, -1, -2, 1}};
    return t[i][j];
  }
};
template <> struct Mats<KIND_43> {
  static constexpr int m = 4, r = 3, alpha = 6;
  __host__ __device__ static constexpr float at(int i, int j) {
    constexpr float t[4][6] = {{1, 1, 1, 1, 1, 0}, {0, 1, -1, 2, -2, 0},
                               {0, 1, 1, 4, 4, 0}, {0, 1, -1, 8, -8, 1}};
    return t[i][j];
  }
  __host__ __device__ static constexpr float g(int i, int j) {
    constexpr float t[6][3] = {{1.f / 4, 0, 0},
                               {-1.f / 6, -1.f / 6, -1.f / 6},
                               {-1.f / 6, 1.f / 6, -1.f / 6},
                               {1.f / 24, 1.f / 12, 1.f / 6},
                               {1.f / 24, -1.f / 12, 1.f / 6},
                               {0, 0, 1}};
    return t[i][j];
  }
  __host__ __device__ static constexpr float bt(int i, int j) {
    constexpr float t[6][6] = {{4, 0, -5, 0, 1, 0},  {0, -4, -4, 1, 1, 0}, {0, 4, -4, -1, 1, 0},
                               {0, -2, -1, 2, 1, 0}, {0, 2, -1, -2, 1, 0}, {0, 4, 0, -5, 0, 1}};
    return t[i][j];
  }
};

template <> struct Mats<KIND_41> {
  static constexpr int m = 4, r = 1, alpha = 4;
  __host__ __device__ static constexpr float at(int i, int j) { return i == j ? 1.f : 0.f; }
  __host__ __device__ static constexpr float g(int i, int j) { return 1.f; }
  __host__ __device__ static constexpr float bt(int i, int j) { return i == j ? 1.f : 0.f; }
};
template <> struct Mats<KIND_42> {
  static constexpr int m = 4, r = 2, alpha = 5;
  __host__ __device__ static constexpr float at(int i, int j) {
    constexpr float t[4][5] = {{1, 1, 1, 1, 0}, {0, 1, -1, 2, 0}, {0, 1, 1, 4, 0}, {0, 1, -1, 8, 1}};
    return t[i][j];
  }
  __host__ __device__ static constexpr float g(int i, int j) {
    constexpr float t[5][2] = {{1.f / 2, 0}, {-1.f / 2, -1.f / 2}, {-1.f / 6, 1.f / 6}, {1.f / 6, 1.f / 3}, {0, 1}};
    return t[i][j];
  }
  __host__ __device__ static constexpr float bt(int i, int j) {
    constexpr float t[5][5] = {{2, -1, -2, 1, 0}, {0, -2, -1, 1, 0}, {0, 2, -3, 1, 0}, {0, -1, 0, 1, 0}, {0, 2, -1, -2, 1}};
    return t[i][j];
  }
};

template <> struct Mats<KIND_24> {
  static constexpr int m = 2, r = 4, alpha = 5;
  __host__ __device__ static constexpr float at(int i, int j) {
    constexpr float t[2][5] = {{1, 1, 1, 1, 0},
                               {0, 1, -1, 2, 1}};
    return t[i][j];
  }
  __host__ __device__ static constexpr float g(int i, int j) {
    constexpr float t[5][4] = {{1.f / 2, 0, 0, 0},
                               {-1.f / 2, -1.f / 2, -1.f / 2, -1.f / 2},
                               {-1.f / 6, 1.f / 6, -1.f / 6, 1.f / 6},
                               {1.f / 6, 1.f / 3, 2.f / 3, 4.f / 3},
                               {0, 0, 0, 1}};
    return t[i][j];
  }
  __host__ __device__ static constexpr float bt(int i, int j) {
    constexpr float t[5][5] = {{2, -1, -2, 1, 0},
                               {0, -2, -1, 1, 0},
                               {0, 2, -3, 1, 0},
                               {0, -1, 0, 1, 0},
                               {0, 2, -1, -2, 1}};
    return t[i][j];
  }
};
template <> struct Mats<KIND_25> {
  static constexpr int m = 2, r = 5, alpha = 6;
  __host__ __device__ static constexpr float at(int i, int j) {
    constexpr float t[2][6] = {{1, 1, 1, 1, 1, 0},
                               {0, 1, -1, 2, -2, 1}};
    return t[i][j];
  }
  __host__ __device__ static constexpr float g(int i, int j) {
    constexpr float t[6][5] = {{1.f / 4, 0, 0, 0, 0},
                               {-1.f / 6, -1.f / 6, -1.f / 6, -1.f / 6, -1.f / 6},
                               {-1.f / 6, 1.f / 6, -1.f / 6, 1.f / 6, -1.f / 6},
                               {1.f / 24, 1.f / 12, 1.f / 6, 1.f / 3, 2.f / 3},
                               {1.f / 24, -1.f / 12, 1.f / 6, -1.f / 3, 2.f / 3},
                               {0, 0, 0, 0, 1}};
    return t[i][j];
  }
  __host__ __device__ static constexpr float bt(int i, int j) {
    constexpr float t[6][6] = {{4, 0, -5, 0, 1, 0},
                               {0, -4, -4, 1, 1, 0},
                               {0, 4, -4, -1, 1, 0},
                               {0, -2, -1, 2, 1, 0},
                               {0, 2, -1, -2, 1, 0},
                               {0, 4, 0, -5, 0, 1}};
    return t[i][j];
  }
};
template <> struct Mats<KIND_26> {
  static constexpr int m = 2, r = 6, alpha = 7;
  __host__ __device__ static constexpr float at(int i, int j) {
    constexpr float t[2][7] = {{1, 1, 1, 1, 1, 1, 0},
                               {0, 1, -1, 1.f / 2, -1.f / 2, 1.f / 3, 1}};
    return t[i][j];
  }
  __host__ __device__ static constexpr float g(int i, int j) {
    constexpr float t[7][6] = {{12, 0, 0, 0, 0, 0},
                               {1, 1, 1, 1, 1, 1},
                               {-1.f / 2, 1.f / 2, -1.f / 2, 1.f / 2, -1.f / 2, 1.f / 2},
                               {-16, -8, -4, -2, -1, -1.f / 2},
                               {16.f / 5, -8.f / 5, 4.f / 5, -2.f / 5, 1.f / 5, -1.f / 10},
                               {243.f / 10, 81.f / 10, 27.f / 10, 9.f / 10, 3.f / 10, 1.f / 10},
                               {0, 0, 0, 0, 0, 1}};
    return t[i][j];
  }
  __host__ __device__ static constexpr float bt(int i, int j) {
    constexpr float t[7][7] = {{1.f / 12, -1.f / 4, -5.f / 12, 5.f / 4, 1.f / 3, -1, 0},
                               {0, 1.f / 12, -1.f / 6, -7.f / 12, 2.f / 3, 1, 0},
                               {0, -1.f / 12, 1.f / 3, 1.f / 12, -4.f / 3, 1, 0},
                               {0, 1.f / 6, -1.f / 6, -7.f / 6, 1.f / 6, 1, 0},
                               {0, -1.f / 6, 5.f / 6, -5.f / 6, -5.f / 6, 1, 0},
                               {0, 1.f / 4, 0, -5.f / 4, 0, 1, 0},
                               {0, -1.f / 12, 1.f / 4, 5.f / 12, -5.f / 4, -1.f / 3, 1}};
    return t[i][j];
  }
};
template <> struct Mats<KIND_27> {
  static constexpr int m = 2, r = 7, alpha = 8;
  __host__ __device__ static constexpr float at(int i, int j) {
    constexpr float t[2][8] = {{1, 1, 1, 1, 1, 1, 1, 0},
                               {0, 1, -1, 1.f / 2, -1.f / 2, 1.f / 3, -1.f / 3, 1}};
    return t[i][j];
  }
  __host__ __device__ static constexpr float g(int i, int j) {
    constexpr float t[8][7] = {{36, 0, 0, 0, 0, 0, 0},
                               {3.f / 4, 3.f / 4, 3.f / 4, 3.f / 4, 3.f / 4, 3.f / 4, 3.f / 4},
                               {3.f / 4, -3.f / 4, 3.f / 4, -3.f / 4, 3.f / 4, -3.f / 4, 3.f / 4},
                               {-96.f / 5, -48.f / 5, -24.f / 5, -12.f / 5, -6.f / 5, -3.f / 5, -3.f / 10},
                               {-96.f / 5, 48.f / 5, -24.f / 5, 12.f / 5, -6.f / 5, 3.f / 5, -3.f / 10},
                               {729.f / 20, 243.f / 20, 81.f / 20, 27.f / 20, 9.f / 20, 3.f / 20, 1.f / 20},
                               {729.f / 20, -243.f / 20, 81.f / 20, -27.f / 20, 9.f / 20, -3.f / 20, 1.f / 20},
                               {0, 0, 0, 0, 0, 0, 1}};
    return t[i][j];
  }
  __host__ __device__ static constexpr float bt(int i, int j) {
    constexpr float t[8][8] = {{1.f / 36, 0, -7.f / 18, 0, 49.f / 36, 0, -1, 0},
                               {0, 1.f / 36, 1.f / 36, -13.f / 36, -13.f / 36, 1, 1, 0},
                               {0, -1.f / 36, 1.f / 36, 13.f / 36, -13.f / 36, -1, 1, 0},
                               {0, 1.f / 18, 1.f / 9, -5.f / 9, -10.f / 9, 1.f / 2, 1, 0},
                               {0, -1.f / 18, 1.f / 9, 5.f / 9, -10.f / 9, -1.f / 2, 1, 0},
                               {0, 1.f / 12, 1.f / 4, -5.f / 12, -5.f / 4, 1.f / 3, 1, 0},
                               {0, -1.f / 12, 1.f / 4, 5.f / 12, -5.f / 4, -1.f / 3, 1, 0},
                               {0, -1.f / 36, 0, 7.f / 18, 0, -49.f / 36, 0, 1}};
    return t[i][j];
  }
};

// Run-time views of the same tables (host planning, the generic filter / multi-piece kernels).
__host__ __device__ inline float table_g(int kind, int i, int j) {
  switch (kind) {
    case KIND_11: return Mats<KIND_11>::g(i, j);
    case KIND_21: return Mats<KIND_21>::g(i, j);
    case KIND_22: return Mats<KIND_22>::g(i, j);
    case KIND_23: return Mats<KIND_23>::g(i, j);
    case KIND_41: return Mats<KIND_41>::g(i, j);
    case KIND_42: return Mats<KIND_42>::g(i, j);
    case KIND_24: return Mats<KIND_24>::g(i, j);
    case KIND_25: return Mats<KIND_25>::g(i, j);
    case KIND_26: return Mats<KIND_26>::g(i, j);
    case KIND_27: return Mats<KIND_27>::g(i, j);
    case KIND_33: return Mats<KIND_33>::g(i, j);
    default: return Mats<KIND_43>::g(i, j);
  }
}
__host__ __device__ inline float table_at(int kind, int i, int j) {
  switch (kind) {
    case KIND_11: return Mats<KIND_11>::at(i, j);
    case KIND_21: return Mats<KIND_21>::at(i, j);
    case KIND_22: return Mats<KIND_22>::at(i, j);
    case KIND_23: return Mats<KIND_23>::at(i, j);
    case KIND_41: return Mats<KIND_41>::at(i, j);
    case KIND_42: return Mats<KIND_42>::at(i, j);
    case KIND_24: return Mats<KIND_24>::at(i, j);
    case KIND_25: return Mats<KIND_25>::at(i, j);
    case KIND_26: return Mats<KIND_26>::at(i, j);
    case KIND_27: return Mats<KIND_27>::at(i, j);
    case KIND_33: return Mats<KIND_33>::at(i, j);
    default: return Mats<KIND_43>::at(i, j);
  }
}

}  // namespace wc
