// The compile-time contract between the model driver and a backend, restated from the reference
// (models/common/ops/concept.hh:16-40 and models/llama2/ops/concept.hh:15-42) so that the hip
// classes can be checked against it without the reference's headers.
#pragma once

#include <concepts>
#include <cstdint>
#include <string>
#include <vector>

#include "glint/types.hh"

namespace glint {

namespace detail {
constexpr uint64_t ONE = 1;
}

template<typename T, typename DType>
concept OperationsConcept = requires( const T t,
                                      DType* ptr1,
                                      const DType* ptr2,
                                      float32_t* ptr_f32,
                                      uint32_t* ptr_uint32,
                                      const uint64_t size,
                                      const float32_t val_f32,
                                      const bool flag,
                                      const std::vector<float>& vec_f,
                                      const CopyType cpt,
                                      const std::string base ) {
  typename T::DeviceUniquePtr;
  { t.template accum<detail::ONE>( ptr1, ptr2, size ) } -> std::same_as<void>;
  { t.template rmsnorm<detail::ONE>( ptr1, ptr2, ptr_f32, ptr2, size ) } -> std::same_as<void>;
  { t.template argmax<detail::ONE>( ptr_uint32, ptr2, ptr1, size ) } -> std::same_as<void>;
  { t.template silu<detail::ONE>( ptr1, ptr1, size ) } -> std::same_as<void>;
  { t.template matmul<detail::ONE, detail::ONE>( ptr1, ptr2, ptr2, size ) } -> std::same_as<void>;
  { t.untemplated_matmul( ptr1, ptr2, ptr2, size, size, size ) } -> std::same_as<void>;
  { t.soft_sample( ptr1, vec_f, size ) } -> std::same_as<void>;
  { t.copy( ptr1, ptr2, size, cpt, flag ) } -> std::same_as<void>;
  { t.print( ptr2, size, base ) } -> std::same_as<void>;
  { t.device_allocate( size ) } -> std::same_as<typename T::DeviceUniquePtr>;
  { t.randomize_device_buffer( ptr1, size, val_f32, val_f32 ) } -> std::same_as<void>;
};

template<typename T, typename DType, typename Settings>
concept AdditionalLlamaOperationsConcept = requires( const T t,
                                                     void* ptr_void,
                                                     DType* ptr,
                                                     const DType* cptr,
                                                     const uint64_t size,
                                                     const uint32_t* int_arr,
                                                     const CopyType cpt,
                                                     const Settings& s,
                                                     typename T::ContextType::LayerContextType lc[],
                                                     typename T::ContextType::TokenContextType tc[] ) {
  { T( s ) };
  { t.attention_0_gemm( cptr, lc, ptr, size, int_arr ) } -> std::same_as<void>;
  { t.attention_2_gemm( cptr, lc, ptr, size, int_arr ) } -> std::same_as<void>;
  { t.attention_softmax( ptr, int_arr, ptr, size ) } -> std::same_as<void>;
  { t.apply_rope( size, int_arr, cptr, cptr, ptr, tc ) } -> std::same_as<void>;
  { t.copy_kv_cache( tc, cptr, size ) } -> std::same_as<void>;
  { t.template convert_and_copy<void, void>( ptr_void, ptr_void, size, cpt ) } -> std::same_as<void>;
};

template<typename T, typename DType, typename Settings>
concept LlamaOperationsConcept = AdditionalLlamaOperationsConcept<T, DType, Settings> && OperationsConcept<T, DType>;

} // namespace glint
