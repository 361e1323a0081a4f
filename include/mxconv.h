/*
 * mxconv - MI355X (gfx950) forward convolution behind a C ABI.
 *
 * This is the boundary a PopLibs maintainer binds instead of building a
 * Poplar graph: every entry point takes plain pointers, sizes and a HIP
 * stream, never a C++ or framework type, and reports failure through a status
 * code plus a thread-local message (mxconv_last_error).  No exception crosses
 * it.  Each declaration cites the reference interface it stands in for
 * (paths relative to the PopLibs source tree).
 *
 * Device tensors:
 *   activations / output  channels-last  [B][field...][G*C]
 *   weights               packed by mxconv_pack_weights for the chosen plan
 *   bias                  [G*Co] in the output element type
 * The external layouts of the reference ([B][G*C][field...] activations,
 * [G][Co][Ci][kernel...] weights; include/poplin/Convolution.hpp:323-328) are
 * converted on the device by mxconv_acts_to_internal / mxconv_pack_weights /
 * mxconv_acts_to_external, the counterpart of creating tensors with
 * createInput / createWeights and letting convolution() rearrange others
 * (lib/poplin/Convolution.cpp:2569-2628).
 */
#ifndef MXCONV_H
#define MXCONV_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MXCONV_MAX_FIELD_DIMS 4
/* "No such element", as poplin::getInputIndex returns it
 * (include/poplin/ConvUtil.hpp:22-26). */
#define MXCONV_NO_INDEX 0xFFFFFFFFu

typedef enum mxconv_status {
  MXCONV_OK = 0,
  /* poputil::poplibs_error (include/poputil/exceptions.hpp:17-21): bad shape,
   * rank, type or parameter combination. */
  MXCONV_INVALID_PARAMS = 1,
  /* poplar::invalid_option: unknown option key or value
   * (tests/poplin/ConvTest.cpp:684-698). */
  MXCONV_INVALID_OPTION = 2,
  /* A valid request this build has no kernel for. */
  MXCONV_UNSUPPORTED = 3,
  /* poplar::graph_memory_allocation_error; the harness maps it to exit code
   * 77 (tools/single_conv_layer.cpp:1531-1537). */
  MXCONV_OUT_OF_MEMORY = 4,
  MXCONV_WORKSPACE_TOO_SMALL = 5,
  MXCONV_BUFFER_TOO_SMALL = 6,
  MXCONV_HIP_ERROR = 7,
  MXCONV_NULL_ARGUMENT = 8
} mxconv_status;

/* poplar::QUARTER / HALF / FLOAT as used for ConvParams::inputType and
 * outputType (include/poplin/ConvParams.hpp:96-97). */
typedef enum mxconv_type {
  MXCONV_QUARTER = 0, /* 8-bit float + metadata byte, see mxconv_fwd_quarter */
  MXCONV_HALF = 1,    /* IEEE binary16 */
  MXCONV_FLOAT = 2    /* IEEE binary32 */
} mxconv_type;

/* poplin::ConvParams::InputTransform (include/poplin/ConvParams.hpp:17-59). */
typedef struct mxconv_input_transform {
  uint32_t truncation_lower[MXCONV_MAX_FIELD_DIMS];
  uint32_t truncation_upper[MXCONV_MAX_FIELD_DIMS];
  uint32_t dilation[MXCONV_MAX_FIELD_DIMS];
  uint32_t padding_lower[MXCONV_MAX_FIELD_DIMS];
  uint32_t padding_upper[MXCONV_MAX_FIELD_DIMS];
  uint8_t flip[MXCONV_MAX_FIELD_DIMS];
} mxconv_input_transform;

/* poplin::ConvParams::OutputTransform (include/poplin/ConvParams.hpp:61-94). */
typedef struct mxconv_output_transform {
  uint32_t truncation_lower[MXCONV_MAX_FIELD_DIMS];
  uint32_t truncation_upper[MXCONV_MAX_FIELD_DIMS];
  uint32_t stride[MXCONV_MAX_FIELD_DIMS];
  uint32_t padding_lower[MXCONV_MAX_FIELD_DIMS];
  uint32_t padding_upper[MXCONV_MAX_FIELD_DIMS];
} mxconv_output_transform;

/* poplin::ConvParams (include/poplin/ConvParams.hpp:16-224).  Only the first
 * num_field_dims entries of each array are meaningful. */
typedef struct mxconv_params {
  int32_t input_type;  /* mxconv_type */
  int32_t output_type; /* mxconv_type */
  uint32_t num_field_dims;
  uint32_t reserved;
  uint64_t batch_size;
  uint64_t input_field_shape[MXCONV_MAX_FIELD_DIMS];
  uint64_t kernel_shape[MXCONV_MAX_FIELD_DIMS];
  uint64_t input_channels_per_conv_group;
  uint64_t output_channels_per_conv_group;
  uint64_t num_conv_groups;
  mxconv_input_transform input_transform;
  mxconv_input_transform kernel_transform;
  mxconv_output_transform output_transform;
} mxconv_params;

typedef struct mxconv_plan mxconv_plan;
/* hipStream_t without pulling in the HIP headers. */
typedef struct ihipStream_t *mxconv_stream;

/* Message of the last failing call on this thread (empty string if none). */
const char *mxconv_last_error(void);
const char *mxconv_status_string(mxconv_status status);

/* ---- descriptor algebra (host only, no GPU needed) ---------------------- */

/* ConvParams(inputType, outputType, batchSize, inputFieldShape, kernelShape,
 * inputChannels, outputChannels, numConvGroups) with identity transforms:
 * dilation and stride 1, everything else 0 / false
 * (lib/poplin/ConvParams.cpp:132-152, 268-290). */
mxconv_status mxconv_params_init(mxconv_params *p, int32_t input_type,
                                 int32_t output_type, uint64_t batch_size,
                                 uint32_t num_field_dims,
                                 const uint64_t *input_field_shape,
                                 const uint64_t *kernel_shape,
                                 uint64_t input_channels_per_conv_group,
                                 uint64_t output_channels_per_conv_group,
                                 uint64_t num_conv_groups);

/* ConvParams::validate (lib/poplin/ConvParams.cpp:172-266). */
mxconv_status mxconv_params_validate(const mxconv_params *p);

/* ConvParams::canonicalize (lib/poplin/ConvParams.cpp:468-629), including the
 * all-zero-output normal form of getZeroConv
 * (lib/poplin/ConvUtilInternal.cpp:40-76). */
mxconv_status mxconv_params_canonicalize(const mxconv_params *p,
                                         mxconv_params *canonical);

/* getGradientParams (lib/poplin/ConvUtil.cpp:728-795): the convolution that
 * turns the gradient w.r.t. the forward output into the gradient w.r.t. the
 * forward input, given the weights of mxconv_weights_transpose_chans_flip_xy.
 * The result is canonical. */
mxconv_status mxconv_get_gradient_params(const mxconv_params *p,
                                         mxconv_params *gradient);

/* getWeightUpdateParams (include/poplin/ConvUtil.hpp:114,
 * lib/poplin/Convolution.cpp:3390-3435): the convolution that computes the
 * gradient w.r.t. the forward weights - batch and input channels exchanged,
 * the forward output field as kernel.  The result is canonical. */
mxconv_status mxconv_get_weight_update_params(const mxconv_params *p,
                                              mxconv_params *weight_update);

/* isZeroConvolution (lib/poplin/ConvUtilInternal.cpp:24-38); canonicalizes
 * first, as CanonicalConvParams does. */
mxconv_status mxconv_params_is_zero_convolution(const mxconv_params *p,
                                                int *is_zero);

/* Size queries of ConvParams (lib/poplin/ConvParams.cpp:631-698). */
typedef enum mxconv_size_query {
  MXCONV_TRUNCATED_INPUT_SIZE = 0,     /* getTruncatedInputSize */
  MXCONV_TRUNCATED_KERNEL_SIZE = 1,    /* getTruncatedKernelSize */
  MXCONV_TRANSFORMED_INPUT_SIZE = 2,   /* getTransformedInputSize */
  MXCONV_TRANSFORMED_KERNEL_SIZE = 3,  /* getTransformedKernelSize */
  MXCONV_UNTRANSFORMED_OUTPUT_SIZE = 4, /* getUntransformedOutputSize */
  MXCONV_OUTPUT_SIZE = 5               /* getOutputSize */
} mxconv_size_query;
mxconv_status mxconv_params_size(const mxconv_params *p, int32_t query,
                                 uint32_t dim, uint64_t *size);

/* operator== and operator< of ConvParams (lib/poplin/ConvParams.cpp:103-119):
 * *order is <0, 0 or >0. */
mxconv_status mxconv_params_compare(const mxconv_params *a,
                                    const mxconv_params *b, int *order);
/* std::hash<poplin::ConvParams> (lib/poplin/ConvParams.cpp:734-751): equal
 * parameters hash equally; the value itself is this build's. */
mxconv_status mxconv_params_hash(const mxconv_params *p, uint64_t *hash);

/* operator>>(std::istream&, ConvParams&) (lib/poplin/ConvParams.cpp:365-458):
 * JSON with keys dataType | inputType, outputType, batchSize, numConvGroups,
 * inputChannelsPerConvGroup, outputChannelsPerConvGroup, inputFieldShape,
 * kernelShape, inputTransform, kernelTransform, outputTransform. */
mxconv_status mxconv_params_from_json(const char *json, mxconv_params *p);
/* operator<<(std::ostream&, const ConvParams&)
 * (lib/poplin/ConvParams.cpp:292-363).  Writes at most `capacity` bytes
 * including the terminator; *needed receives the full length + 1. */
mxconv_status mxconv_params_to_string(const mxconv_params *p, char *buffer,
                                      size_t capacity, size_t *needed);

/* poplin::getInputIndex / getKernelIndex (lib/poplin/ConvUtil.cpp:234-309). */
mxconv_status mxconv_get_input_index(const mxconv_params *p, uint32_t dim,
                                     uint32_t output_index,
                                     uint32_t kernel_index, uint32_t *index);
mxconv_status mxconv_get_kernel_index(const mxconv_params *p, uint32_t dim,
                                      uint32_t output_index,
                                      uint32_t input_index, uint32_t *index);

/* Range queries of include/poplin/ConvUtil.hpp:34-86; every range is
 * half-open {begin, end} and {0, 0} when empty. */
typedef enum mxconv_range_query {
  /* getOutputRangeForKernelRange(dim, a, b): a = output bounds, b = kernels */
  MXCONV_OUTPUT_RANGE_FOR_KERNEL_RANGE = 0,
  /* getOutputRangeForInputRange(dim, a, b): a = output bounds, b = inputs */
  MXCONV_OUTPUT_RANGE_FOR_INPUT_RANGE = 1,
  /* getInputRange(dim, a, b): a = output range, b = kernel range */
  MXCONV_INPUT_RANGE = 2,
  /* getKernelRange(dim, a, b): a = output range, b = input range */
  MXCONV_KERNEL_RANGE = 3
} mxconv_range_query;
mxconv_status mxconv_get_range(const mxconv_params *p, int32_t query,
                               uint32_t dim, const uint32_t a[2],
                               const uint32_t b[2], uint32_t result[2]);

/* getNumberOfMACs (lib/poplin/PerformanceEstimation.hpp:1641-1666) and
 * getFwdFlops = 2 * MACs (lib/poplin/Convolution.cpp:3217-3221).  MACs that
 * fall on padding are not counted. */
mxconv_status mxconv_get_number_of_macs(const mxconv_params *p, uint64_t *macs);
mxconv_status mxconv_get_fwd_flops(const mxconv_params *p, uint64_t *flops);

/* convolutionValidateOptions (include/poplin/Convolution.hpp:719): the
 * key/value pairs of a poplar::OptionFlags.  Keys of
 * lib/poplin/ConvOptions.cpp:105-152 are recognised; partialsType, pass and
 * planConstraints influence the plan, the remaining (IPU-only) ones are
 * checked for well-formed values and otherwise ignored. */
mxconv_status mxconv_validate_options(const char *const *keys,
                                      const char *const *values,
                                      size_t num_options);

/* ---- planning ----------------------------------------------------------- */

/* getPlan (lib/poplin/ConvPlan.cpp:1877-1923): validates and canonicalizes
 * the parameters, applies validateLayerParams
 * (lib/poplin/ConvValidation.cpp:11-70) and chooses the gfx950 kernel and its
 * tile shape.  Touches no GPU.  The plan is immutable and may be shared
 * between threads and streams. */
mxconv_status mxconv_plan_create(const mxconv_params *p,
                                 const char *const *option_keys,
                                 const char *const *option_values,
                                 size_t num_options, mxconv_plan **plan);
void mxconv_plan_destroy(mxconv_plan *plan);

/* reportPlanInfo (include/poplin/Convolution.hpp:584-587). */
mxconv_status mxconv_plan_describe(const mxconv_plan *plan, char *buffer,
                                   size_t capacity, size_t *needed);

/* getPlanConstraints (lib/poplin/ConvPlan.cpp:1574-1636): the plan as a
 * complete `planConstraints` JSON document ({"gfx950": {...}}).  Passed back
 * as that option with the same parameters it reproduces the plan exactly.
 * The option `planConstraintsOutputFilename`
 * (include/poplin/Convolution.hpp:191-199) makes mxconv_plan_create and
 * mxconv_weight_update_plan_create write the same text to
 * <name>_FWD.json / _BWD.json / _WU.json by the `pass` option, <name>.json
 * without one (lib/poplin/ConvPlan.cpp:1638-1666, 1764).  Same buffer
 * protocol as mxconv_plan_describe. */
mxconv_status mxconv_plan_constraints(const mxconv_plan *plan, char *buffer,
                                      size_t capacity, size_t *needed);

/* reportPlanEstimatedCosts (include/poplin/Convolution.hpp:590-611,
 * lib/poplin/Convolution.cpp:3923-3936): the planner's estimate for one
 * launch of the plan.  *cycles: shader-clock cycles from the cost model the
 * tilings were weighed with, or MXCONV_COST_UNKNOWN where the model does not
 * cover the kernel (the generic one).  The model is in microseconds (its
 * constants are measured launch and k-step times); cycles = microseconds x
 * MXCONV_ESTIMATE_CLOCK_MHZ, the one clock figure used for the conversion:
 * 2100 MHz, what the chip holds with the matrix cores of 224 of its 256 CUs
 * busy (2120 MHz measured; 1930 MHz with all 256, 2390 MHz with one).
 * *memory_bytes: the temporary device memory of a launch (the workspace).
 * Touches no GPU. */
#define MXCONV_COST_UNKNOWN UINT64_MAX
#define MXCONV_ESTIMATE_CLOCK_MHZ 2100
mxconv_status mxconv_plan_estimated_costs(const mxconv_plan *plan,
                                          uint64_t *cycles,
                                          uint64_t *memory_bytes);

/* reportDetailedPlanEstimatedCosts (include/poplin/Convolution.hpp:613-676,
 * lib/poplin/Convolution.cpp:3940-3962): the same estimate taken apart.  Of
 * the reference's phases a launch on this device has three: rearrangement
 * (the zero-padded copy of an input whose channels do not fill a vector, the
 * fill of an output field the kernel does not cover), compute (the
 * convolution kernel) and reduction (the ordered sum of fp32 partial tiles
 * where K or the pixels are split over workgroups).  Each phase: cycles as in
 * mxconv_plan_estimated_costs and the temporary bytes it owns.
 * parallel_split: workgroups that run side by side (at most the CUs times
 * the workgroups a CU holds); serial_split: rounds of them (both 1 where the
 * model prices a kernel by its bytes alone: fills, the tiled depthwise
 * kernels).  The phases' cycles add up to total.cycles, which is what
 * mxconv_plan_estimated_costs returns; every cycles field is
 * MXCONV_COST_UNKNOWN where that is.
 * Touches no GPU. */
typedef struct mxconv_phase_cost {
  uint64_t cycles;
  uint64_t memory_bytes;
} mxconv_phase_cost;
typedef struct mxconv_detailed_costs {
  uint64_t parallel_split;
  uint64_t serial_split;
  mxconv_phase_cost rearrangement;
  mxconv_phase_cost compute;
  mxconv_phase_cost reduction;
  mxconv_phase_cost total;
} mxconv_detailed_costs;
mxconv_status mxconv_plan_detailed_costs(const mxconv_plan *plan,
                                         mxconv_detailed_costs *costs);

/* Whether weights packed for `packed_for` are laid out as `plan` reads them
 * (*same = 1) or not (0).  In the reference the options given to
 * createWeights only decide a tensor layout and convolution() rearranges a
 * tensor laid out otherwise (lib/poplin/Convolution.cpp:2569-2628); here a
 * packed buffer carries no description of itself, so the caller has to ask. */
mxconv_status mxconv_plans_pack_alike(const mxconv_plan *plan,
                                      const mxconv_plan *packed_for,
                                      int32_t *same);

/* Sizes, in bytes, of the device buffers mxconv_fwd works on; what
 * createInput / createWeights / createConvOutput / createBiases allocate in
 * the reference (lib/poplin/Convolution.cpp:1563-1577, 1713-1728, 1813-1825,
 * include/poplin/Convolution.hpp:316-319). */
typedef enum mxconv_buffer {
  MXCONV_BUFFER_INPUT = 0,
  MXCONV_BUFFER_WEIGHTS_PACKED = 1,
  MXCONV_BUFFER_OUTPUT = 2,
  MXCONV_BUFFER_BIAS = 3,
  MXCONV_BUFFER_WORKSPACE = 4,
  MXCONV_BUFFER_WEIGHTS_EXTERNAL = 5
} mxconv_buffer;
mxconv_status mxconv_plan_buffer_bytes(const mxconv_plan *plan, int32_t which,
                                       size_t *bytes);

/* ---- device work (all asynchronous on `stream`) ------------------------- */

/* Weights [G][Co][Ci][kernel...] (input element type) -> the plan's packed
 * layout.  Role of createWeights + the weight rearrangement of
 * lib/poplin/Convolution.cpp:2569-2628. */
mxconv_status mxconv_pack_weights(const mxconv_plan *plan,
                                  const void *weights_external,
                                  void *weights_packed, mxconv_stream stream);

/* Activations [B][G*Ci][field...] -> channels-last, and the output back from
 * channels-last to [B][G*Co][field...] (actsToInternalShape /
 * actsToExternalShape, lib/poplin/ConvUtilInternal.cpp:147-175). */
mxconv_status mxconv_acts_to_internal(const mxconv_plan *plan,
                                      const void *acts_external,
                                      void *acts_internal,
                                      mxconv_stream stream);
mxconv_status mxconv_acts_to_external(const mxconv_plan *plan,
                                      const void *out_internal,
                                      void *out_external, mxconv_stream stream);

/* poplin::convolutionWithOutput (include/poplin/Convolution.hpp:377-384) with
 * the optional addBias (include/poplin/Convolution.hpp:570-572) fused:
 *   out[b][o...][g*Co+oc] = cast_outputType( bias[g*Co+oc] +
 *       sum_{ic,k...} in'[b][o*s + k'...][g*Ci+ic] * w[g][oc][ic][k...] )
 * accumulated in fp32.  `bias` may be NULL.  For HALF and FLOAT inputs. */
mxconv_status mxconv_fwd(const mxconv_plan *plan, const void *in,
                         const void *weights_packed, const void *bias,
                         void *out, void *workspace, size_t workspace_bytes,
                         mxconv_stream stream);

/* mxconv_fwd for callers that cannot allocate device memory or carry a
 * workspace around (code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc): the scratch memory a plan needs - fp32
 * partial tiles when K is split, the zero-filled copy of an input whose
 * channels are padded - comes from a buffer of 32 MiB built into the library,
 * one per GPU.  No counterpart in the reference (Poplar owns all memory
 * there).  Returns MXCONV_WORKSPACE_TOO_SMALL for a plan whose workspace
 * exceeds the buffer; allocates nothing.  The first call on a GPU looks up
 * the buffer's address there, at which point the HIP runtime may load the
 * library's device data: make that call once at set-up, outside any capture.
 * All calls on one GPU share the buffer: calls that overlap in time on one
 * GPU race. */
mxconv_status mxconv_fwd_static_scratch(const mxconv_plan *plan,
                                        const void *in,
                                        const void *weights_packed,
                                        const void *bias, void *out,
                                        mxconv_stream stream);

/* The same for QUARTER inputs.  Each metadata byte is
 * (format << 7) | (scale & 0x3f): format 1 = E4M3 ("F143"), 0 = E5M2
 * ("F152"); scale is a signed 6-bit power of two, value = fp8 * 2^scale (bit
 * layout of lib/popops/Cast.cpp:168-209).  The product carries 2^(sIn + sW)
 * (lib/poplin/codelets/inlineAssemblerConv.hpp:28-33).  The 8-bit encodings
 * are OCP E4M3FN / E5M2, the ones gfx950's matrix cores consume. */
mxconv_status mxconv_fwd_quarter(const mxconv_plan *plan, const void *in,
                                 uint8_t in_metadata,
                                 const void *weights_packed,
                                 uint8_t weights_metadata, const void *bias,
                                 void *out, void *workspace,
                                 size_t workspace_bytes, mxconv_stream stream);

/* ---- several convolutions at once ---------------------------------------
 * poplin::multiconv::convolution (include/poplin/MultiConvolution.hpp:
 * 143-149): `n` independent forward passes, results as if each had been run
 * by mxconv_fwd / mxconv_fwd_quarter.  PopLibs runs them side by side on
 * disjoint tile ranges; here, with parallel != 0, convolutions that run the
 * same matrix-core kernel (same tile width, element types, fp8 formats) are
 * issued as ONE launch whose grid is the concatenation of their tiles, up to
 * eight at a time, so that convolutions too small to fill the chip share it;
 * the others, and everything with parallel == 0, run one after another.  All
 * work is enqueued on `stream`.  Arrays have `n` entries; `bias`,
 * `workspaces` / `workspace_bytes` and the two metadata arrays may be NULL
 * (no bias, no workspace, metadata byte 0); metadata is read for plans with
 * QUARTER inputs only. */
mxconv_status mxconv_multi_fwd(size_t n, const mxconv_plan *const *plans,
                               const void *const *in,
                               const uint8_t *in_metadata,
                               const void *const *weights_packed,
                               const uint8_t *weights_metadata,
                               const void *const *bias, void *const *out,
                               void *const *workspaces,
                               const size_t *workspace_bytes, int parallel,
                               mxconv_stream stream);

/* Checks multi-convolution options (lib/poplin/ConvPlan.cpp:1929-1953):
 * planType = parallel | serial, perConvReservedTiles (integer), cycleBackOff
 * (number).  *parallel (may be NULL) receives 1 for planType parallel, the
 * default, else 0; the other two steer the IPU tile split only. */
mxconv_status mxconv_multiconv_validate_options(const char *const *keys,
                                                const char *const *values,
                                                size_t num_options,
                                                int *parallel);

/* ---- matrix multiplication on the same kernels --------------------------- */

/* getConvParams of lib/poplin/MatMul.cpp:236-272: C[g] = A[g] * B[g] with A
 * [groups][m][k], B [groups][k][n] is the convolution with batch m, field {1},
 * kernel {1}, k input and n output channels per group. */
mxconv_status mxconv_matmul_params(int32_t input_type, int32_t output_type,
                                   uint64_t groups, uint64_t m, uint64_t k,
                                   uint64_t n, mxconv_params *p);

/* parseMatMulOptions + getConvOptionFlags (lib/poplin/MatMul.cpp:116-195):
 * checks matMul option keys / values (partialsType, fullyConnectedPass,
 * inputRHSIsPreArranged, use128BitConvUnitLoad, enableMultiStageReduce,
 * enableFastReduce, remapOutputTensor, availableMemoryProportion,
 * planConstraints, gatherOutput, disableSRForAMPVertices). */
mxconv_status mxconv_matmul_validate_options(const char *const *keys,
                                             const char *const *values,
                                             size_t num_options);

/* mxconv_plan_create for the parameters of mxconv_matmul_params, taking
 * matMul options (translated as getConvOptionFlags does). */
mxconv_status mxconv_matmul_plan_create(int32_t input_type, int32_t output_type,
                                        uint64_t groups, uint64_t m, uint64_t k,
                                        uint64_t n,
                                        const char *const *option_keys,
                                        const char *const *option_values,
                                        size_t num_options, mxconv_plan **plan);

/* The right-hand side B [groups][k][n] -> the packed weights of a plan made
 * from mxconv_matmul_params (convWeightsFromMatrix(transpose(B)),
 * lib/poplin/MatMul.cpp:386). */
mxconv_status mxconv_matmul_pack_rhs(const mxconv_plan *plan, const void *rhs,
                                     void *weights_packed,
                                     mxconv_stream stream);

/* A [groups][m][k] -> the convolution's input [m][groups*k], and its output
 * [m][groups*n] -> C [groups][m][n] (convActivationsFromMatrix /
 * matrixFromConvActivations, lib/poplin/MatMul.cpp:197-226).  With one group
 * both are plain copies and callers may pass the matrices themselves to
 * mxconv_fwd instead. */
mxconv_status mxconv_matmul_lhs_to_internal(const mxconv_plan *plan,
                                            const void *lhs, void *acts_internal,
                                            mxconv_stream stream);
mxconv_status mxconv_matmul_out_to_external(const mxconv_plan *plan,
                                            const void *out_internal,
                                            void *result, mxconv_stream stream);

/* ---- weight update pass ---------------------------------------------------
 * poplin::calculateWeightDeltas / convolutionWeightUpdate /
 * convolutionBiasUpdate (include/poplin/Convolution.hpp:460-563,
 * lib/poplin/Convolution.cpp:3437-3620).
 *
 * The plan of the pass: mxconv_plan_create on
 * mxconv_get_weight_update_params(fwd) with the forward options, whose `pass`
 * is replaced as getWeightUpdateOptions does
 * (lib/poplin/ConvUtilInternal.cpp:941-954).  For
 * mxconv_convolution_weight_update give forward parameters whose output type
 * equals the input type, as the reference does (:3535), so that the deltas
 * come out in the weights' type.  For a layer without spatial extent (every
 * field and kernel dimension 1, one group) the plan also holds the plan of
 * one matrix product, transpose(deltas) x activations, which
 * mxconv_calculate_weight_deltas then runs instead of the pass's convolution;
 * mxconv_weight_update_workspace_bytes is the size either way. */
mxconv_status mxconv_weight_update_plan_create(const mxconv_params *fwd,
                                               const char *const *option_keys,
                                               const char *const *option_values,
                                               size_t num_options,
                                               mxconv_plan **plan);

/* Bytes of device scratch the two calls below need for `plan` (the
 * rearranged operands, the pass's output before it is brought into weight
 * order and, for the update, the deltas). */
mxconv_status mxconv_weight_update_workspace_bytes(const mxconv_plan *plan,
                                                   size_t *bytes);

/* weight_deltas [G][Co][Ci][kernel...] (external layout, the plan's output
 * type) = gradient w.r.t. the forward weights, from z_deltas
 * [B][outField...][G*Co] and activations [B][field...][G*Ci], both
 * channels-last in the forward input type.  Half and float tensors. */
mxconv_status mxconv_calculate_weight_deltas(const mxconv_plan *plan,
                                             const void *z_deltas_internal,
                                             const void *acts_internal,
                                             void *weight_deltas_external,
                                             void *workspace,
                                             size_t workspace_bytes,
                                             mxconv_stream stream);

/* weights_external += scale * weight deltas (lib/poplin/Convolution.cpp:
 * 3552-3571); pack the updated weights again for the forward plan. */
mxconv_status mxconv_convolution_weight_update(const mxconv_plan *plan,
                                               const void *z_deltas_internal,
                                               void *weights_external,
                                               const void *acts_internal,
                                               float scale, void *workspace,
                                               size_t workspace_bytes,
                                               mxconv_stream stream);

/* biases[c] += scale * sum of z_deltas over batch and field
 * (lib/poplin/Convolution.cpp:3592-3620).  z_deltas is channels-last
 * [outer_elems][channels]; sums are formed in fp32 in a fixed order.
 * workspace: mxconv_bias_update_workspace_bytes. */
mxconv_status mxconv_bias_update_workspace_bytes(uint64_t outer_elems,
                                                 uint64_t channels,
                                                 size_t *bytes);
mxconv_status mxconv_convolution_bias_update(int32_t deltas_type,
                                             const void *z_deltas_internal,
                                             uint64_t outer_elems,
                                             uint64_t channels,
                                             int32_t bias_type, void *biases,
                                             float scale, void *workspace,
                                             size_t workspace_bytes,
                                             mxconv_stream stream);

/* poplin::transposeGroupedMatrix (include/poplin/MatMul.hpp:612) as a copy:
 * src [groups][rows][cols] -> dst [groups][cols][rows]; any element type. */
mxconv_status mxconv_transpose_grouped_matrix(int32_t type, uint64_t groups,
                                              uint64_t rows, uint64_t cols,
                                              const void *src, void *dst,
                                              mxconv_stream stream);

/* c[i] = scale_c * c[i] + scale_product * product[i] over `elems` half or
 * float elements, evaluated in fp32: the popops::scaledAddTo step of
 * poplin::matMulAcc / matMulGroupedAcc (lib/poplin/MatMul.cpp:499-519,
 * 578-597; scale_c = 1 there) and of a general beta * C + alpha * A * B
 * (tools/general_matrix_multiply.cpp:367). */
mxconv_status mxconv_scaled_add_to(int32_t type, void *c, float scale_c,
                                   const void *product, float scale_product,
                                   uint64_t elems, mxconv_stream stream);

/* poplin::weightsTransposeChansFlipXY (include/poplin/Convolution.hpp:407-412,
 * lib/poplin/Convolution.cpp:3262-3388) on device tensors in the external
 * layout: weights_in [G][Co][Ci][kernel...] -> weights_out
 * [G][Ci][Co][kernel...] with every spatial axis reversed.  `p` are the
 * FORWARD parameters (they give G, Co, Ci, the kernel shape and the element
 * type).  The two buffers must not overlap. */
mxconv_status mxconv_weights_transpose_chans_flip_xy(const mxconv_params *p,
                                                     const void *weights_in,
                                                     void *weights_out,
                                                     mxconv_stream stream);

/* poplin::addBias (lib/poplin/Convolution.cpp:3637-3648) on a channels-last
 * tensor of `outer_elems` x `channels` elements of `type`. */
mxconv_status mxconv_add_bias(int32_t type, void *acts_internal,
                              const void *bias, uint64_t outer_elems,
                              uint64_t channels, mxconv_stream stream);

#ifdef __cplusplus
}
#endif
#endif /* MXCONV_H */
