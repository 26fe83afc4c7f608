/*
 * flyvec_legacy.h -- the C ABI of the reference's five CUDA shared objects, exported by
 * libflyvec_hip.so as well, so that the reference's own driver (flyvec/train_flyvec.py:62-263) can
 * load this library under the five names it opens (model_descriptor.so, model_arrays.so,
 * cuda_helpers.so, cuda_funcs.so, prune_input.so: `python -m flyvec_amd.build --legacy-names DIR`
 * writes them as links to the one library). Names, argument order and argument types are the
 * reference's; every function forwards to the fv_* entry points of flyvec_hip.h.
 *
 * As in the reference (flyvec/src/cuda_funcs.cu:36-54) these functions return nothing: an error is
 * printed to stderr and the process exits. One GPU: get_cuda_num_devices answers 1 and the per-GPU
 * arguments must be 0. The handles are opaque; the reference never frees its own, flyvec_legacy_release
 * (an addition) does.
 */
#ifndef FLYVEC_LEGACY_H
#define FLYVEC_LEGACY_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- cuda_helpers.so (flyvec/src/cuda_helpers.cu:8-35) ------------------------------------- */
void *do_gpu_cudaMallocManaged(unsigned long bytes); /* :8  host-visible memory (page-locked here) */
void *do_cpu_malloc(unsigned long bytes);            /* :17 */
void *do_gpu_cudaHostAlloc(unsigned long bytes);     /* :22 page-locked host memory */
int get_cuda_num_devices(void);                      /* :31 always 1: this build uses one GPU */

/* ---- prune_input.so (flyvec/src/prune_input.cpp) ------------------------------------------------ */
void prune_input_data(void *data_i32, uint64_t rows, uint64_t cols);                                /* :14 */
uint64_t getnum_samples(void *offsets_u64, uint64_t n_sentences, uint64_t W);                        /* :64 */
void compute_offset_phrases(void *out_u64, void *offsets_u64, uint64_t n_sentences, uint64_t W);     /* :88 */

/* ---- model_descriptor.so (flyvec/src/model_descriptor.cu) --------------------------------------- */
void *model_create_descriptor(int num_gpus);                                 /* :18 */
/* :51 keys IM_HEIGHT IM_WIDTH Nchannels Ns_1 W ST hid Num p m vocabulary_size sparse_input
 * frequency_scaling; the image-model keys are stored and not used */
void set_model_param_int(uint64_t value, const char *key, void *descriptor);
/* :74 keys initial_learning_rate delta prec mu sigma Lmid Lbase */
void set_model_param_float(float value, const char *key, void *descriptor);
void compute_model_derived_parameters(void *descriptor);                     /* :91 N = 2 * vocabulary_size */
void copy_model_params(void *descriptor, int source, int destination);       /* :115 one GPU: nothing to copy */
void print_model_params(void *descriptor);                                   /* :145 */

/* ---- model_arrays.so (flyvec/src/model_arrays.cu) ------------------------------------------------ */
void *model_create_arrays(int num_gpus);                                               /* :15 */
/* :22 creates the trainer; p and m other than 2 (the reference's defaults, which its driver never sets) are refused;
 * the shuffle of the window order that the reference makes here (:180-198) is applied as soon as the order exists */
void model_arrays_allocate_memory(void *descriptor, void *arrays, int num_gpus);
void push_INPUT_memory_to_GPU(void *arrays, void *descriptor, int device, const char *type); /* :250 the corpus is
                                                                                          always resident here */
/* :305 "synapses": K x 2V fp32 row-major in page-locked host memory; the driver fills it before the first
 * epoch and saves it after any epoch. launch_epoch_INPUT_AS_INT uploads it first and downloads it last. */
void *get_data_pointer(const char *name, void *arrays, int device);
/* :320 "INPUT", type "i4": a matrix of Ns_1 windows already cut out, IM_HEIGHT * IM_WIDTH * Nchannels (>= W) token
 * ids per row; 1/frequency is then counted over that matrix. The image types ("f", "u1") report that they are
 * outside this library and exit; another name is reported and ignored, as in the reference. */
void set_data_pointer(const char *name, void *arrays, void *descriptor, void *ptr, const char *type, int device);
/* :358 type "i4": the corpus (int32) and the window-start table compute_offset_phrases wrote */
void set_up_INPUT_pointer(const char *name, void *arrays, void *descriptor, void *corpus, void *starts,
                          const char *type, int device);
/* :396 also the moment the corpus goes to the device: it tells the corpus length */
void compute_inverse_word_frequency(void *arrays, void *descriptor, void *corpus, uint64_t n_tokens, int device);
void do_reshuffle_indices(void *descriptor, void *arrays, int device);                 /* :442 */

/* No counterpart in the reference (it never frees its handles): destroys the trainer, the matrix and both
 * handles. For hosts that create more than one model in a process. */
void flyvec_legacy_release(void *descriptor, void *arrays);
/* No counterpart in the reference (its matrix is managed memory of its own): from now on get_data_pointer("synapses")
 * serves `ptr`, K x 2V fp32 row-major in host memory of the caller, and the epochs read and write it. */
void flyvec_legacy_set_synapses(void *arrays, void *ptr);

/* ---- cuda_funcs.so (flyvec/src/cuda_funcs.cu) ---------------------------------------------------- */
/* :1220 one epoch over the current window order */
void launch_epoch_INPUT_AS_INT(void *descriptor, void *arrays, int num_gpus, uint64_t epoch_id, uint64_t n_epochs);
/* :1164, :1184 the image and dense-float models are outside this library: they report that and exit */
void launch_epoch_INPUT_AS_IMAGE(void *descriptor, void *arrays, int num_gpus, uint64_t epoch_id, uint64_t n_epochs);
void launch_epoch_INPUT_AS_FLOAT(void *descriptor, void *arrays, int num_gpus, uint64_t epoch_id, uint64_t n_epochs);

#ifdef __cplusplus
}
#endif
#endif /* FLYVEC_LEGACY_H */
