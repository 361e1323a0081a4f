/*
 * TEST INFRASTRUCTURE - NOT PRODUCT CODE.
 *
 * CPU restatement, in plain C and double precision, of the host reference
 * model that the PopLibs convolution tests compare against:
 *   poplibs_test::conv::convolution   lib/poplibs_test/Convolution.cpp:455-575
 * (and of its backward and weight update companions further down)
 * and of the helpers it is built from (cited at each function).  It exists so
 * that the parity tests, the smoke check and the benchmark's CPU-baseline leg
 * have an independent statement of what a forward convolution must produce.
 * Nothing in the shipped library links, loads or calls this file.
 *
 * How this restatement is pinned (see tests/test_oracle_pinning.py):
 *   - special cases against torch.nn.functional.conv{1,2,3}d in float64,
 *   - 1x1 kernels against a plain matrix product,
 *   - textbook identities (delta kernel, box sums, linearity, group
 *     independence),
 *   - +-1 data giving exact integers,
 *   - the generalised transforms (truncation, input dilation, flips, kernel
 *     padding, output truncation/padding) against a second implementation
 *     written from the per-dimension index definition poplin::getInputIndex
 *     (lib/poplin/ConvUtil.cpp:234-268),
 *   - slicing invariants (sub-convolution of sliced tensors == slice of the
 *     full result; a split over input channels sums to the full result).
 * convolutionBackward (:577-722) and weightUpdate (:724-898) are restated
 * too; they are pinned by torch autograd in float64 on ordinary parameters and,
 * with every transform, by the adjoint identities
 *   <conv(x, w), dz> == <x, backward(dz, w)> == <w, weightDeltas(x, dz)>
 * (tests/test_backward.py, tests/test_weight_update.py).
 * The FP8 codec below is this build's own definition (OCP E4M3FN / E5M2 plus a
 * power-of-two scale); bit-level parity with Graphcore's QUARTER type, whose
 * codec lives in the closed Poplar SDK, is: parity unpinned.
 *
 * The summation order of every output element is the reference's (kernel
 * element outermost, input channel innermost, lib/poplibs_test/Convolution.cpp
 * :543-553), also in the multi-threaded entry point, which only distributes
 * whole output rows (group, batch, out-channel) over threads.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define ORACLE_MAX_DIMS 8

/* lib/poplibs_test/Convolution.cpp:13-15 */
static unsigned absdiff(unsigned a, unsigned b) { return a < b ? b - a : a - b; }

static size_t product(const unsigned *v, unsigned n) {
  size_t p = 1;
  for (unsigned i = 0; i != n; ++i)
    p *= v[i];
  return p;
}

/* lib/poplibs_test/Convolution.cpp:21-25 */
static unsigned dilated_size(unsigned size, unsigned dilation) {
  if (size == 0)
    return 0;
  return 1 + (size - 1) * dilation;
}

/* lib/poplibs_test/Convolution.cpp:27-35 */
static unsigned transformed_size(unsigned size, unsigned truncation_lower,
                                 unsigned truncation_upper, unsigned dilation,
                                 unsigned padding_lower,
                                 unsigned padding_upper) {
  unsigned truncated = size - (truncation_lower + truncation_upper);
  unsigned dilated = dilated_size(truncated, dilation);
  return padding_lower + dilated + padding_upper;
}

/* include/poputil/Util.hpp:81-105: row-major, last dimension fastest. */
static void unflatten_index(const unsigned *shape, unsigned n, size_t index,
                            unsigned *out) {
  for (unsigned d = n; d-- != 0;) {
    out[d] = (unsigned)(index % shape[d]);
    index /= shape[d];
  }
}

static size_t flatten_index(const unsigned *shape, unsigned n,
                            const unsigned *indices) {
  size_t index = 0;
  for (unsigned d = 0; d != n; ++d)
    index = index * shape[d] + indices[d];
  return index;
}

/* lib/poplibs_test/Convolution.cpp:55-76 (one dimension). */
unsigned oracle_output_field_size(
    unsigned input_size, unsigned kernel_size, unsigned in_trunc_lower,
    unsigned in_trunc_upper, unsigned in_dilation, unsigned in_pad_lower,
    unsigned in_pad_upper, unsigned k_trunc_lower, unsigned k_trunc_upper,
    unsigned k_dilation, unsigned k_pad_lower, unsigned k_pad_upper,
    unsigned out_trunc_lower, unsigned out_trunc_upper, unsigned stride,
    unsigned out_pad_lower, unsigned out_pad_upper) {
  unsigned tin = transformed_size(input_size, in_trunc_lower, in_trunc_upper,
                                  in_dilation, in_pad_lower, in_pad_upper);
  unsigned tk = transformed_size(kernel_size, k_trunc_lower, k_trunc_upper,
                                 k_dilation, k_pad_lower, k_pad_upper);
  unsigned conv_out = tin - tk + 1;
  unsigned truncated = conv_out - (out_trunc_lower + out_trunc_upper);
  unsigned strided = (truncated + stride - 1) / stride;
  return out_pad_lower + strided + out_pad_upper;
}

/*
 * lib/poplibs_test/Convolution.cpp:125-195.  `in` is [rows][prod(size)];
 * returns a freshly allocated [rows][prod(padded_size)].  The reference stages
 * this through three arrays (truncated, dilated, padded); each stage only
 * copies values, so the stages are kept as three explicit index maps applied
 * in the same order: truncate, dilate (zero insertion), pad, then flip.
 */
static double *truncate_dilate_pad_flip(
    const double *in, size_t rows, unsigned n, const unsigned *size,
    const unsigned *truncation_lower, const unsigned *truncation_upper,
    const unsigned *dilation, const unsigned *padding_lower,
    const unsigned *padding_upper, const unsigned char *flip,
    unsigned *padded_size) {
  unsigned truncated_size[ORACLE_MAX_DIMS], dilated[ORACLE_MAX_DIMS];
  for (unsigned d = 0; d != n; ++d) {
    truncated_size[d] = size[d] - (truncation_lower[d] + truncation_upper[d]);
    dilated[d] = dilated_size(truncated_size[d], dilation[d]);
    padded_size[d] = dilated[d] + padding_lower[d] + padding_upper[d];
  }
  const size_t in_elems = product(size, n);
  const size_t truncated_elems = product(truncated_size, n);
  const size_t padded_elems = product(padded_size, n);
  double *padded = (double *)calloc(rows * padded_elems + 1, sizeof(double));
  if (!padded)
    return NULL;
  for (size_t r = 0; r != rows; ++r) {
    for (size_t e = 0; e != truncated_elems; ++e) {
      unsigned t[ORACLE_MAX_DIMS], src[ORACLE_MAX_DIMS], dst[ORACLE_MAX_DIMS];
      unflatten_index(truncated_size, n, e, t);
      for (unsigned d = 0; d != n; ++d) {
        src[d] = t[d] + truncation_lower[d];          /* :157-162 */
        unsigned dilated_index = t[d] * dilation[d];  /* :112-123, 171-173 */
        unsigned p = dilated_index + padding_lower[d]; /* :186 */
        if (flip[d])
          p = padded_size[d] - 1 - p; /* :187-188 */
        dst[d] = p;
      }
      padded[r * padded_elems + flatten_index(padded_size, n, dst)] =
          in[r * in_elems + flatten_index(size, n, src)];
    }
  }
  return padded;
}

/*
 * lib/poplibs_test/Convolution.cpp:267-336, the inverse used for the output
 * transform.  `padded` is [rows][prod(padded_size)]; writes [rows][prod(size)]
 * into `out`, whose untouched elements are zero (the reference
 * value-initialises the array, :319-321).
 */
static int truncate_dilate_pad_flip_inverse(
    const double *padded, size_t rows, unsigned n, const unsigned *padded_size,
    const unsigned *truncation_lower, const unsigned *truncation_upper,
    const unsigned *dilation, const unsigned *padding_lower,
    const unsigned *padding_upper, const unsigned char *flip, double *out,
    size_t out_elems_expected, unsigned *size) {
  unsigned truncated_size[ORACLE_MAX_DIMS], dilated[ORACLE_MAX_DIMS];
  for (unsigned d = 0; d != n; ++d) {
    dilated[d] = padded_size[d] - (padding_lower[d] + padding_upper[d]);
    truncated_size[d] = (dilated[d] + dilation[d] - 1) / dilation[d];
    size[d] = truncation_lower[d] + truncated_size[d] + truncation_upper[d];
  }
  const size_t padded_elems = product(padded_size, n);
  const size_t truncated_elems = product(truncated_size, n);
  const size_t elems = product(size, n);
  if (rows * elems != out_elems_expected)
    return -1;
  memset(out, 0, rows * elems * sizeof(double));
  for (size_t r = 0; r != rows; ++r) {
    for (size_t e = 0; e != truncated_elems; ++e) {
      unsigned t[ORACLE_MAX_DIMS], src[ORACLE_MAX_DIMS], dst[ORACLE_MAX_DIMS];
      unflatten_index(truncated_size, n, e, t);
      for (unsigned d = 0; d != n; ++d) {
        unsigned dilated_index = t[d] * dilation[d];   /* :314-316 */
        unsigned p = dilated_index + padding_lower[d]; /* :299 */
        if (flip[d])
          p = padded_size[d] - 1 - p; /* :300-301 */
        src[d] = p;
        dst[d] = t[d] + truncation_lower[d]; /* :328-332 */
      }
      out[r * elems + flatten_index(size, n, dst)] =
          padded[r * padded_elems + flatten_index(padded_size, n, src)];
    }
  }
  return 0;
}

/* lib/poplibs_test/Convolution.cpp:423-433 */
static unsigned get_input_index(unsigned input_size, unsigned kernel_size,
                                unsigned output_index, unsigned kernel_index) {
  if (kernel_size > input_size) {
    int input_index = (int)kernel_index - (int)output_index;
    if (input_index < 0 || (unsigned)input_index >= input_size)
      return ~0U;
    return (unsigned)input_index;
  }
  return kernel_index + output_index;
}

/* lib/poplibs_test/Convolution.cpp:435-453 */
static int get_input_indices(unsigned n, const unsigned *input_size,
                             const unsigned *kernel_size,
                             const unsigned *output_indices,
                             const unsigned *kernel_indices,
                             unsigned *input_indices) {
  for (unsigned d = 0; d != n; ++d) {
    unsigned i = get_input_index(input_size[d], kernel_size[d],
                                 output_indices[d], kernel_indices[d]);
    if (i == ~0U)
      return 0;
    input_indices[d] = i;
  }
  return 1;
}

/*
 * lib/poplibs_test/Convolution.cpp:455-575.
 *   in      [batch][groups*in_chans_per_group][prod(input_field_size)]
 *   kernel  [groups][out_chans_per_group][in_chans_per_group][prod(kernel_size)]
 *   biases  [groups*out_chans_per_group]
 *   out     [batch][groups*out_chans_per_group][prod(output field)]
 * `out_elems` is the number of doubles `out` holds; the call fails (-1) when
 * it does not equal the size the parameters imply (the reference asserts on
 * the shape when it assigns the result, :562-564).  `threads` > 1 distributes
 * (group, batch, out-channel) rows over that many OpenMP threads; every
 * element's sum is formed in the same order whatever the thread count.
 * Returns 0 on success, -2 on rank overflow, -3 on allocation failure.
 */
int oracle_convolution(
    unsigned num_field_dims, const unsigned *input_field_size,
    const unsigned *truncation_lower, const unsigned *truncation_upper,
    const unsigned *input_dilation, const unsigned *padding_lower,
    const unsigned *padding_upper, const unsigned char *flip_input,
    const unsigned *kernel_size, const unsigned *kernel_truncation_lower,
    const unsigned *kernel_truncation_upper, const unsigned *kernel_dilation,
    const unsigned *kernel_padding_lower, const unsigned *kernel_padding_upper,
    const unsigned char *flip_kernel, const unsigned *output_truncation_lower,
    const unsigned *output_truncation_upper, const unsigned *stride,
    const unsigned *output_padding_lower, const unsigned *output_padding_upper,
    unsigned batch_size, unsigned num_conv_groups, unsigned in_chans_per_group,
    unsigned out_chans_per_group, const double *in, const double *kernel,
    const double *biases, double *out, size_t out_elems, int threads) {
  const unsigned n = num_field_dims;
  if (n > ORACLE_MAX_DIMS)
    return -2;
  const unsigned in_chans = num_conv_groups * in_chans_per_group;
  const unsigned out_chans = num_conv_groups * out_chans_per_group;

  unsigned padded_kernel_size[ORACLE_MAX_DIMS];
  unsigned padded_field_size[ORACLE_MAX_DIMS];
  /* :514-518 */
  double *padded_kernel = truncate_dilate_pad_flip(
      kernel, (size_t)num_conv_groups * out_chans_per_group * in_chans_per_group,
      n, kernel_size, kernel_truncation_lower, kernel_truncation_upper,
      kernel_dilation, kernel_padding_lower, kernel_padding_upper, flip_kernel,
      padded_kernel_size);
  /* :519-522 */
  double *padded_in = truncate_dilate_pad_flip(
      in, (size_t)batch_size * in_chans, n, input_field_size, truncation_lower,
      truncation_upper, input_dilation, padding_lower, padding_upper,
      flip_input, padded_field_size);
  if (!padded_kernel || !padded_in) {
    free(padded_kernel);
    free(padded_in);
    return -3;
  }

  /* :527-534 */
  unsigned conv_out_size[ORACLE_MAX_DIMS];
  for (unsigned d = 0; d != n; ++d)
    conv_out_size[d] = absdiff(padded_field_size[d], padded_kernel_size[d]) + 1;
  const size_t conv_out_elems = product(conv_out_size, n);
  const size_t padded_kernel_elems = product(padded_kernel_size, n);
  const size_t padded_field_elems = product(padded_field_size, n);
  double *conv_out = (double *)calloc(
      (size_t)batch_size * out_chans * conv_out_elems + 1, sizeof(double));
  if (!conv_out) {
    free(padded_kernel);
    free(padded_in);
    return -3;
  }

  /* :536-559.  The (gc, b, oc) loops are collapsed into one row index whose
   * order is the reference's; inside a row the order of additions into each
   * conv_out element is: kernel element ke ascending, then ic ascending. */
  const long rows =
      (long)num_conv_groups * (long)batch_size * (long)out_chans_per_group;
  if (threads < 1)
    threads = 1;
#pragma omp parallel for schedule(dynamic, 1) num_threads(threads)
  for (long row = 0; row < rows; ++row) {
    const unsigned oc = (unsigned)(row % out_chans_per_group);
    const unsigned b = (unsigned)((row / out_chans_per_group) % batch_size);
    const unsigned gc =
        (unsigned)(row / ((long)out_chans_per_group * batch_size));
    const unsigned oc_act = gc * out_chans_per_group + oc;
    double *conv_row = conv_out + ((size_t)b * out_chans + oc_act) * conv_out_elems;
    const double *kernel_row =
        padded_kernel + ((size_t)gc * out_chans_per_group + oc) *
                            in_chans_per_group * padded_kernel_elems;
    for (size_t oe = 0; oe != conv_out_elems; ++oe) {
      unsigned output_indices[ORACLE_MAX_DIMS];
      unflatten_index(conv_out_size, n, oe, output_indices);
      double acc = conv_row[oe]; /* 0.0 */
      for (size_t ke = 0; ke != padded_kernel_elems; ++ke) {
        unsigned kernel_indices[ORACLE_MAX_DIMS];
        unsigned input_indices[ORACLE_MAX_DIMS];
        unflatten_index(padded_kernel_size, n, ke, kernel_indices);
        if (get_input_indices(n, padded_field_size, padded_kernel_size,
                              output_indices, kernel_indices, input_indices)) {
          const size_t ie = flatten_index(padded_field_size, n, input_indices);
          for (unsigned ic = 0; ic != in_chans_per_group; ++ic) {
            const unsigned ic_act = gc * in_chans_per_group + ic;
            acc += kernel_row[(size_t)ic * padded_kernel_elems + ke] *
                   padded_in[((size_t)b * in_chans + ic_act) *
                                 padded_field_elems +
                             ie];
          }
        }
      }
      conv_row[oe] = acc;
    }
  }

  /* :561-564: output transform = inverse with padding := output truncation,
   * dilation := stride, truncation := output padding, no flips. */
  unsigned char no_flipping[ORACLE_MAX_DIMS] = {0};
  unsigned out_field[ORACLE_MAX_DIMS];
  int rc = truncate_dilate_pad_flip_inverse(
      conv_out, (size_t)batch_size * out_chans, n, conv_out_size,
      output_padding_lower, output_padding_upper, stride,
      output_truncation_lower, output_truncation_upper, no_flipping, out,
      out_elems, out_field);
  free(conv_out);
  free(padded_kernel);
  free(padded_in);
  if (rc != 0)
    return -1;

  /* :565-574: the bias is added to every element, output padding included. */
  const size_t out_field_elems = product(out_field, n);
  for (unsigned gc = 0; gc != num_conv_groups; ++gc)
    for (unsigned b = 0; b != batch_size; ++b)
      for (unsigned oc = 0; oc != out_chans_per_group; ++oc) {
        const unsigned oc_act = gc * out_chans_per_group + oc;
        double *row = out + ((size_t)b * out_chans + oc_act) * out_field_elems;
        for (size_t e = 0; e != out_field_elems; ++e)
          row[e] += biases[oc_act];
      }
  return 0;
}

/*
 * lib/poplibs_test/Convolution.cpp:577-722: the gradient with respect to the
 * forward pass's input.  All parameters describe the FORWARD convolution.
 *   deltas_in   [batch][groups*out_chans_per_group][prod(forward output field)]
 *   kernel      [groups][out_chans_per_group][in_chans_per_group][prod(kernel)]
 *   deltas_out  [batch][groups*in_chans_per_group][prod(fwd_input_field_size)]
 * The reference scatters every (output element, kernel element) product into
 * the padded forward input and then undoes the input transform.  `threads` > 1
 * distributes (group, batch) pairs, which touch disjoint rows of the scatter
 * target; within a row the order of additions is the reference's (oc, oe, ke
 * ascending).  Returns 0, or -1 size mismatch, -2 rank, -3 allocation.
 */
int oracle_convolution_backward(
    unsigned num_field_dims, const unsigned *fwd_input_field_size,
    const unsigned *truncation_lower, const unsigned *truncation_upper,
    const unsigned *input_dilation, const unsigned *padding_lower,
    const unsigned *padding_upper, const unsigned char *flip_input,
    const unsigned *kernel_size, const unsigned *kernel_truncation_lower,
    const unsigned *kernel_truncation_upper, const unsigned *kernel_dilation,
    const unsigned *kernel_padding_lower, const unsigned *kernel_padding_upper,
    const unsigned char *flip_kernel, const unsigned *output_truncation_lower,
    const unsigned *output_truncation_upper, const unsigned *stride,
    const unsigned *output_padding_lower, const unsigned *output_padding_upper,
    unsigned batch_size, unsigned num_conv_groups, unsigned in_chans_per_group,
    unsigned out_chans_per_group, const double *deltas_in, const double *kernel,
    double *deltas_out, size_t deltas_out_elems, int threads) {
  const unsigned n = num_field_dims;
  if (n > ORACLE_MAX_DIMS)
    return -2;
  const unsigned fwd_in_chans = num_conv_groups * in_chans_per_group;
  const unsigned fwd_out_chans = num_conv_groups * out_chans_per_group;

  /* :620-626 */
  unsigned fwd_output_field_size[ORACLE_MAX_DIMS];
  for (unsigned d = 0; d != n; ++d)
    fwd_output_field_size[d] = oracle_output_field_size(
        fwd_input_field_size[d], kernel_size[d], truncation_lower[d],
        truncation_upper[d], input_dilation[d], padding_lower[d],
        padding_upper[d], kernel_truncation_lower[d], kernel_truncation_upper[d],
        kernel_dilation[d], kernel_padding_lower[d], kernel_padding_upper[d],
        output_truncation_lower[d], output_truncation_upper[d], stride[d],
        output_padding_lower[d], output_padding_upper[d]);

  /* :643-647 */
  unsigned padded_kernel_size[ORACLE_MAX_DIMS];
  double *padded_kernel = truncate_dilate_pad_flip(
      kernel, (size_t)num_conv_groups * out_chans_per_group * in_chans_per_group,
      n, kernel_size, kernel_truncation_lower, kernel_truncation_upper,
      kernel_dilation, kernel_padding_lower, kernel_padding_upper, flip_kernel,
      padded_kernel_size);
  if (!padded_kernel)
    return -3;

  /* :649-680: the deltas are padded by what the forward pass truncated from
   * its output, plus the rows a stride > 1 never reached. */
  unsigned fwd_padded_in_size[ORACLE_MAX_DIMS], fwd_conv_out_size[ORACLE_MAX_DIMS];
  unsigned deltas_in_padding_upper[ORACLE_MAX_DIMS];
  for (unsigned d = 0; d != n; ++d) {
    fwd_padded_in_size[d] =
        transformed_size(fwd_input_field_size[d], truncation_lower[d],
                         truncation_upper[d], input_dilation[d],
                         padding_lower[d], padding_upper[d]);
    fwd_conv_out_size[d] = fwd_padded_in_size[d] - padded_kernel_size[d] + 1;
    const unsigned truncated = fwd_conv_out_size[d] - (output_truncation_lower[d] +
                                                       output_truncation_upper[d]);
    if (output_padding_lower[d] + (truncated + stride[d] - 1) / stride[d] +
            output_padding_upper[d] !=
        fwd_output_field_size[d]) {
      free(padded_kernel);
      return -1;
    }
    const unsigned striding_ignored =
        truncated == 0 ? 0 : (truncated - 1) % stride[d];
    deltas_in_padding_upper[d] = output_truncation_upper[d] + striding_ignored;
  }
  /* :681-685 */
  unsigned char no_flipping[ORACLE_MAX_DIMS] = {0};
  unsigned padded_deltas_size[ORACLE_MAX_DIMS];
  double *padded_deltas = truncate_dilate_pad_flip(
      deltas_in, (size_t)batch_size * fwd_out_chans, n, fwd_output_field_size,
      output_padding_lower, output_padding_upper, stride,
      output_truncation_lower, deltas_in_padding_upper, no_flipping,
      padded_deltas_size);
  if (!padded_deltas) {
    free(padded_kernel);
    return -3;
  }
  for (unsigned d = 0; d != n; ++d)
    if (padded_deltas_size[d] != fwd_conv_out_size[d]) {
      free(padded_kernel);
      free(padded_deltas);
      return -1;
    }

  /* :693-719 */
  const size_t fwd_conv_out_elems = product(fwd_conv_out_size, n);
  const size_t fwd_padded_in_elems = product(fwd_padded_in_size, n);
  const size_t padded_kernel_elems = product(padded_kernel_size, n);
  double *conv_out = (double *)calloc(
      (size_t)batch_size * fwd_in_chans * fwd_padded_in_elems + 1, sizeof(double));
  if (!conv_out) {
    free(padded_kernel);
    free(padded_deltas);
    return -3;
  }
  const long pairs = (long)num_conv_groups * (long)batch_size;
  if (threads < 1)
    threads = 1;
#pragma omp parallel for schedule(dynamic, 1) num_threads(threads)
  for (long pair = 0; pair < pairs; ++pair) {
    const unsigned b = (unsigned)(pair % batch_size);
    const unsigned gc = (unsigned)(pair / batch_size);
    for (unsigned oc = 0; oc != out_chans_per_group; ++oc) {
      const unsigned oc_act = gc * out_chans_per_group + oc;
      const double *delta_row =
          padded_deltas + ((size_t)b * fwd_out_chans + oc_act) * fwd_conv_out_elems;
      const double *kernel_row =
          padded_kernel + ((size_t)gc * out_chans_per_group + oc) *
                              in_chans_per_group * padded_kernel_elems;
      for (size_t oe = 0; oe != fwd_conv_out_elems; ++oe) {
        unsigned output_indices[ORACLE_MAX_DIMS];
        unflatten_index(fwd_conv_out_size, n, oe, output_indices);
        for (size_t ke = 0; ke != padded_kernel_elems; ++ke) {
          unsigned kernel_indices[ORACLE_MAX_DIMS];
          unsigned input_indices[ORACLE_MAX_DIMS];
          unflatten_index(padded_kernel_size, n, ke, kernel_indices);
          if (get_input_indices(n, fwd_padded_in_size, padded_kernel_size,
                                output_indices, kernel_indices, input_indices)) {
            const size_t ie = flatten_index(fwd_padded_in_size, n, input_indices);
            for (unsigned ic = 0; ic != in_chans_per_group; ++ic) {
              const unsigned ic_act = gc * in_chans_per_group + ic;
              conv_out[((size_t)b * fwd_in_chans + ic_act) * fwd_padded_in_elems +
                       ie] +=
                  kernel_row[(size_t)ic * padded_kernel_elems + ke] * delta_row[oe];
            }
          }
        }
      }
    }
  }

  /* :720-722 */
  unsigned size[ORACLE_MAX_DIMS];
  int rc = truncate_dilate_pad_flip_inverse(
      conv_out, (size_t)batch_size * fwd_in_chans, n, fwd_padded_in_size,
      truncation_lower, truncation_upper, input_dilation, padding_lower,
      padding_upper, flip_input, deltas_out, deltas_out_elems, size);
  free(conv_out);
  free(padded_kernel);
  free(padded_deltas);
  if (rc != 0)
    return -1;
  for (unsigned d = 0; d != n; ++d)
    if (size[d] != fwd_input_field_size[d])
      return -1;
  return 0;
}

/*
 * The gradient part of poplibs_test::conv::weightUpdate,
 * lib/poplibs_test/Convolution.cpp:724-898 (the reference goes on to apply
 * kernel += learningRate * -weightDeltas and biases += learningRate *
 * -biasDeltas, :881-897; callers do that on the two arrays returned here).
 *   activations   [batch][groups*in_chans_per_group][prod(input_field_size)]
 *   deltas        [batch][groups*out_chans_per_group][prod(output field)]
 *   weight_deltas [groups][out_chans_per_group][in_chans_per_group]
 *                 [prod(kernel_size)]       (weight_delta_elems doubles)
 *   bias_deltas   [groups*out_chans_per_group], may be NULL
 * Each element's sum runs over the batch outermost and the output positions
 * innermost, as in the reference (:838-863); threads share out whole
 * (group, out-channel) rows.  Returns as oracle_convolution.
 */
int oracle_weight_update(
    unsigned num_field_dims, const unsigned *input_field_size,
    const unsigned *truncation_lower, const unsigned *truncation_upper,
    const unsigned *input_dilation, const unsigned *padding_lower,
    const unsigned *padding_upper, const unsigned char *flip_input,
    const unsigned *kernel_size, const unsigned *kernel_truncation_lower,
    const unsigned *kernel_truncation_upper, const unsigned *kernel_dilation,
    const unsigned *kernel_padding_lower, const unsigned *kernel_padding_upper,
    const unsigned char *flip_kernel, const unsigned *output_truncation_lower,
    const unsigned *output_truncation_upper, const unsigned *stride,
    const unsigned *output_padding_lower, const unsigned *output_padding_upper,
    unsigned batch_size, unsigned num_conv_groups, unsigned in_chans_per_group,
    unsigned out_chans_per_group, const double *activations,
    const double *deltas, double *weight_deltas, size_t weight_delta_elems,
    double *bias_deltas, int threads) {
  const unsigned n = num_field_dims;
  if (n > ORACLE_MAX_DIMS)
    return -2;
  const unsigned in_chans = num_conv_groups * in_chans_per_group;
  const unsigned out_chans = num_conv_groups * out_chans_per_group;

  /* :766-771 */
  unsigned output_field_size[ORACLE_MAX_DIMS];
  unsigned padded_kernel_size[ORACLE_MAX_DIMS];
  for (unsigned d = 0; d != n; ++d) {
    output_field_size[d] = oracle_output_field_size(
        input_field_size[d], kernel_size[d], truncation_lower[d],
        truncation_upper[d], input_dilation[d], padding_lower[d],
        padding_upper[d], kernel_truncation_lower[d], kernel_truncation_upper[d],
        kernel_dilation[d], kernel_padding_lower[d], kernel_padding_upper[d],
        output_truncation_lower[d], output_truncation_upper[d], stride[d],
        output_padding_lower[d], output_padding_upper[d]);
    /* :778-780 */
    padded_kernel_size[d] = transformed_size(
        kernel_size[d], kernel_truncation_lower[d], kernel_truncation_upper[d],
        kernel_dilation[d], kernel_padding_lower[d], kernel_padding_upper[d]);
  }

  /* :783-787 */
  unsigned padded_acts_size[ORACLE_MAX_DIMS];
  double *padded_acts = truncate_dilate_pad_flip(
      activations, (size_t)batch_size * in_chans, n, input_field_size,
      truncation_lower, truncation_upper, input_dilation, padding_lower,
      padding_upper, flip_input, padded_acts_size);
  if (!padded_acts)
    return -3;

  /* :789-808 */
  unsigned fwd_conv_out_size[ORACLE_MAX_DIMS];
  unsigned deltas_padding_upper[ORACLE_MAX_DIMS];
  for (unsigned d = 0; d != n; ++d) {
    fwd_conv_out_size[d] =
        absdiff(padded_acts_size[d], padded_kernel_size[d]) + 1;
    /* The reference adds the truncation here (:796-798) where the backward
     * pass subtracts it (:663-665); with it the striding term below would be
     * wrong whenever the output is truncated, and the padded deltas would not
     * have the size of the forward pass's untruncated output.  The size the
     * stride sees is the forward convolution output less its truncation. */
    const unsigned truncated =
        fwd_conv_out_size[d] -
        (output_truncation_lower[d] + output_truncation_upper[d]);
    if (output_padding_lower[d] + (truncated + stride[d] - 1) / stride[d] +
            output_padding_upper[d] !=
        output_field_size[d]) {
      free(padded_acts);
      return -1;
    }
    const unsigned striding_ignored =
        truncated == 0 ? 0 : (truncated - 1) % stride[d];
    deltas_padding_upper[d] = output_truncation_upper[d] + striding_ignored;
  }
  /* :810-814 */
  unsigned char no_flipping[ORACLE_MAX_DIMS] = {0};
  unsigned padded_deltas_size[ORACLE_MAX_DIMS];
  double *padded_deltas = truncate_dilate_pad_flip(
      deltas, (size_t)batch_size * out_chans, n, output_field_size,
      output_padding_lower, output_padding_upper, stride,
      output_truncation_lower, deltas_padding_upper, no_flipping,
      padded_deltas_size);
  if (!padded_deltas) {
    free(padded_acts);
    return -3;
  }
  for (unsigned d = 0; d != n; ++d)
    if (padded_deltas_size[d] != fwd_conv_out_size[d]) {
      free(padded_acts);
      free(padded_deltas);
      return -1;
    }

  /* :830-863 */
  const size_t padded_kernel_elems = product(padded_kernel_size, n);
  const size_t padded_deltas_elems = product(fwd_conv_out_size, n);
  const size_t padded_acts_elems = product(padded_acts_size, n);
  const size_t rows =
      (size_t)num_conv_groups * out_chans_per_group * in_chans_per_group;
  double *padded_weight_deltas =
      (double *)calloc(rows * padded_kernel_elems + 1, sizeof(double));
  if (!padded_weight_deltas) {
    free(padded_acts);
    free(padded_deltas);
    return -3;
  }
  const long pairs = (long)num_conv_groups * (long)out_chans_per_group;
  if (threads < 1)
    threads = 1;
#pragma omp parallel for schedule(dynamic, 1) num_threads(threads)
  for (long pair = 0; pair < pairs; ++pair) {
    const unsigned oc = (unsigned)(pair % out_chans_per_group);
    const unsigned gc = (unsigned)(pair / out_chans_per_group);
    const unsigned oc_act = gc * out_chans_per_group + oc;
    double *row = padded_weight_deltas + (size_t)pair * in_chans_per_group *
                                             padded_kernel_elems;
    for (unsigned b = 0; b != batch_size; ++b) {
      const double *delta_row =
          padded_deltas + ((size_t)b * out_chans + oc_act) * padded_deltas_elems;
      for (size_t oe = 0; oe != padded_deltas_elems; ++oe) {
        unsigned output_indices[ORACLE_MAX_DIMS];
        unflatten_index(fwd_conv_out_size, n, oe, output_indices);
        for (size_t ke = 0; ke != padded_kernel_elems; ++ke) {
          unsigned kernel_indices[ORACLE_MAX_DIMS];
          unsigned input_indices[ORACLE_MAX_DIMS];
          unflatten_index(padded_kernel_size, n, ke, kernel_indices);
          if (get_input_indices(n, padded_acts_size, padded_kernel_size,
                                output_indices, kernel_indices, input_indices)) {
            const size_t ie = flatten_index(padded_acts_size, n, input_indices);
            for (unsigned ic = 0; ic != in_chans_per_group; ++ic) {
              const unsigned ic_act = gc * in_chans_per_group + ic;
              row[(size_t)ic * padded_kernel_elems + ke] +=
                  padded_acts[((size_t)b * in_chans + ic_act) * padded_acts_elems +
                              ie] *
                  delta_row[oe];
            }
          }
        }
      }
    }
  }

  /* :865-868 */
  unsigned size[ORACLE_MAX_DIMS];
  int rc = truncate_dilate_pad_flip_inverse(
      padded_weight_deltas, rows, n, padded_kernel_size, kernel_truncation_lower,
      kernel_truncation_upper, kernel_dilation, kernel_padding_lower,
      kernel_padding_upper, flip_kernel, weight_deltas, weight_delta_elems,
      size);
  free(padded_weight_deltas);
  free(padded_acts);
  free(padded_deltas);
  if (rc != 0)
    return -1;
  for (unsigned d = 0; d != n; ++d)
    if (size[d] != kernel_size[d])
      return -1;

  /* :881-891 */
  if (bias_deltas) {
    const size_t out_elems = product(output_field_size, n);
    for (unsigned oc = 0; oc != out_chans; ++oc)
      bias_deltas[oc] = 0.0;
    for (unsigned b = 0; b != batch_size; ++b)
      for (unsigned oc = 0; oc != out_chans; ++oc)
        for (size_t e = 0; e != out_elems; ++e)
          bias_deltas[oc] += deltas[((size_t)b * out_chans + oc) * out_elems + e];
  }
  return 0;
}

/* ------------------------------------------------------------------------ */
/* FP8 codec of this build (not Graphcore's): OCP 8-bit floats.
 *   format 1 = E4M3FN: bias 7, no infinities, S.1111.111 is NaN, max 448
 *   format 0 = E5M2:   bias 15, IEEE-like infinities and NaNs, max 57344
 * A tensor's value is decode(code) * 2^scale with scale in [-32, 31]; the
 * metadata byte is (format << 7) | (scale & 0x3f), the bit layout the
 * reference manipulates in lib/popops/Cast.cpp:168-209.                      */

double oracle_fp8_decode(unsigned code, int format) {
  const unsigned sign = (code >> 7) & 1;
  double v;
  if (format == 1) {
    const unsigned e = (code >> 3) & 0xf, m = code & 7;
    if (e == 0xf && m == 7)
      return NAN;
    v = e == 0 ? ldexp((double)m, -9) : ldexp((double)(8 + m), (int)e - 10);
  } else {
    const unsigned e = (code >> 2) & 0x1f, m = code & 3;
    if (e == 0x1f)
      return m ? NAN : (sign ? -INFINITY : INFINITY);
    v = e == 0 ? ldexp((double)m, -16) : ldexp((double)(4 + m), (int)e - 17);
  }
  return sign ? -v : v;
}

/* Round to nearest, ties to even; magnitudes beyond the largest finite value
 * saturate to it (so do infinities); NaN maps to the canonical NaN code. */
unsigned oracle_fp8_encode(double x, int format) {
  const int mant_bits = format == 1 ? 3 : 2;
  const int bias = format == 1 ? 7 : 15;
  const double max_finite = format == 1 ? 448.0 : 57344.0;
  const unsigned max_code = format == 1 ? 0x7e : 0x7b;
  if (isnan(x))
    return format == 1 ? 0x7f : 0x7e;
  const unsigned sign = signbit(x) ? 0x80 : 0;
  double a = fabs(x);
  if (a >= max_finite)
    return sign | max_code;
  if (a == 0.0)
    return sign;
  int e;
  frexp(a, &e); /* a = f * 2^e, f in [0.5, 1) */
  int exp_unbiased = e - 1;
  if (exp_unbiased < 1 - bias)
    exp_unbiased = 1 - bias; /* subnormal range shares the smallest exponent */
  /* quantum = 2^(exp - mant_bits); a / quantum is exact in double. */
  const double q = ldexp(a, mant_bits - exp_unbiased);
  double r = nearbyint(q); /* default rounding mode: to nearest even */
  /* r is in [0, 2^(mant_bits+1)]; the top value carries into the exponent. */
  unsigned mant = (unsigned)r;
  unsigned biased;
  if (mant >= (1u << (mant_bits + 1))) {
    mant >>= 1;
    exp_unbiased += 1;
  }
  if (mant < (1u << mant_bits)) {
    biased = 0; /* subnormal (or rounded to zero) */
  } else {
    biased = (unsigned)(exp_unbiased + bias);
    mant -= 1u << mant_bits;
  }
  unsigned code = (biased << mant_bits) | mant;
  if (code > max_code)
    code = max_code;
  return sign | code;
}

unsigned oracle_quarter_metadata(int format, int scale) {
  return ((unsigned)(format & 1) << 7) | ((unsigned)scale & 0x3f);
}

/* Dequantise `n` codes with a metadata byte into doubles. */
void oracle_quarter_to_double(const uint8_t *codes, size_t n,
                              unsigned metadata, double *out) {
  const int format = (metadata >> 7) & 1;
  int scale = (int)(metadata & 0x3f);
  if (scale & 0x20)
    scale -= 64; /* sign-extend the 6-bit field */
  for (size_t i = 0; i != n; ++i)
    out[i] = ldexp(oracle_fp8_decode(codes[i], format), scale);
}
