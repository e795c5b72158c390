// Pulls in the reference's own test helpers (QuantizationParams, Quantize,
// Dequantize) from where they lie, and replaces only ArraysMatch by a
// recorder of the expected vector and its tolerance.
#pragma once
#define ArraysMatch ArraysMatch_reference_unused
#include TVX_REF_TEST_UTILS
#undef ArraysMatch

template <typename T>
::testing::AssertionResult ArraysMatch(const std::vector<T>& expected,
                                       const std::vector<T>&, T abs_error) {
  ::tvxcap::RecordGolden(::tvxcap::ToDouble(expected),
                         static_cast<double>(static_cast<float>(abs_error)), "near");
  return ::testing::AssertionSuccess();
}
