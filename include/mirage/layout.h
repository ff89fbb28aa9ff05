// Declared layouts of device tensors and of thread-block tiles (values as in the
// reference's include/mirage/layout.h:22-45).  Fingerprints ignore them; this
// backend's fp16 kernels also index device tensors row-major and choose the LDS
// placement of each tile themselves, so the enums are carried as plan metadata.
#pragma once

namespace mirage {
namespace layout {

enum DmemLayout {
  DmemRowMajor = 100,
  DmemColumnMajor = 101,
  DmemUnknownLayout = 199,
};

enum SmemLayout {
  SmemRowMajor = 200,
  SmemColumnMajor = 201,
  SmemRowMajorTensorOpMultiplicand_Crosswise16 = 202,
  SmemRowMajorTensorOpMultiplicand_Crosswise32 = 203,
  SmemRowMajorTensorOpMultiplicand_Crosswise64 = 204,
  SmemColumnMajorTensorOpMultiplicand_Crosswise16 = 205,
  SmemColumnMajorTensorOpMultiplicand_Crosswise32 = 206,
  SmemColumnMajorTensorOpMultiplicand_Crosswise64 = 207,
  SmemUnknownLayout = 299,
};

char const *to_string(DmemLayout l);
char const *to_string(SmemLayout l);

}  // namespace layout
}  // namespace mirage
