// Kernel-level operators.  Each owns its output DTensors (allocated from the
// device arena in the constructor, released in reverse order by the destructor)
// and knows how to fingerprint itself over Z_25651 and how to run / time itself
// in fp16.  Interface of the reference's include/mirage/kernel/{operator,matmul,
// element_unary,element_binary,reduction}.h; the device work goes through the C
// ABI in mi355_abi.h.
#pragma once

#include "mirage/kernel/device_tensor.h"
#include "mirage/profile_result.h"
#include "mirage/utils/json_value.h"
#include <vector>

namespace mirage {
namespace kernel {

class KNOperator {
public:
  KNOperator(mirage::type::KNOperatorType _type);
  KNOperator(mirage::type::KNOperatorType _type, DTensor const &input1);
  KNOperator(mirage::type::KNOperatorType _type, DTensor const &input1, DTensor const &input2);
  KNOperator(mirage::type::KNOperatorType _type, std::vector<DTensor> const &inputs);
  virtual ~KNOperator();
  // fp16: run the operator and report its mean time per launch
  virtual bool profile(ProfileResult &result) = 0;
  // uint16: evaluate the operator over the fingerprint ring into fp_ptr
  virtual bool fingerprint(void) = 0;
  // the operator's entry in the JSON form of its graph (reference operator.h:41,
  // src/kernel/graph.cc:35 `json(*op)`)
  virtual operator json() const = 0;

  mirage::type::KNOperatorType op_type;
  std::vector<DTensor> input_tensors;
  std::vector<DTensor> output_tensors;

protected:
  void release_outputs();
};

class KNInputOp : public KNOperator {
public:
  KNInputOp(std::vector<int> const &dims, mirage::type::DataType data_type,
            mirage::layout::DmemLayout layout);
  ~KNInputOp();
  bool profile(ProfileResult &profile) override;
  bool fingerprint(void) override;
  operator json() const override;
};

class KNMatmulOp : public KNOperator {
public:
  KNMatmulOp(DTensor const &A, DTensor const &B);
  ~KNMatmulOp();
  bool profile(ProfileResult &profile) override;
  bool fingerprint(void) override;
  operator json() const override;
};

class KNElementUnaryOp : public KNOperator {
public:
  KNElementUnaryOp(DTensor const &input, mirage::type::KNOperatorType type);
  ~KNElementUnaryOp();
  bool profile(ProfileResult &profile) override;
  bool fingerprint(void) override;
  operator json() const override;
};

class KNElementBinaryOp : public KNOperator {
public:
  KNElementBinaryOp(DTensor const &input1, DTensor const &input2,
                    mirage::type::KNOperatorType type);
  ~KNElementBinaryOp();
  bool profile(ProfileResult &profile) override;
  bool fingerprint(void) override;
  operator json() const override;
};

class KNReductionOp : public KNOperator {
public:
  KNReductionOp(DTensor const &input, int dim, int size);
  ~KNReductionOp();
  bool profile(ProfileResult &profile) override;
  bool fingerprint(void) override;
  operator json() const override;

  int reduction_dim_idx, reduction_dim_size;
};

}  // namespace kernel
}  // namespace mirage
