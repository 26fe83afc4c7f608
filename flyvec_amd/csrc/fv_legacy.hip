// The reference's C ABI (flyvec/train_flyvec.py:62-139 binds it from five CUDA shared objects) on top
// of this library's own entry points: the reference's unchanged driver can open libflyvec_hip.so under
// those five names. Host code only; see include/flyvec_legacy.h for the surface and its limits.
#include <stdlib.h>
#include <string.h>

#include "flyvec_legacy.h"
#include "fv_internal.h"

namespace {

struct legacy_descriptor {
  // what the driver sets (flyvec/src/model_descriptor.cu:51-87); defaults as at :24-40
  uint64_t IM_HEIGHT = 32, IM_WIDTH = 32, Nchannels = 3, Ns_1 = 0, W = 4, ST = 1, hid = 100, Num = 100, p = 2, m = 2;
  uint64_t vocabulary_size = 0, sparse_input = 0, frequency_scaling = 0, N = 0;
  float initial_learning_rate = 0.001f, delta = 0.0f, prec = 1.0e-30f, mu = 0.0f, sigma = 1.0f, Lmid = 1.0f, Lbase = 1.0f;
};

struct legacy_arrays {
  fv_trainer *trainer = nullptr;
  float *synapses = nullptr;  // page-locked host mirror of the matrix, K x 2V row-major
  bool synapses_owned = false;
  const int32_t *corpus = nullptr;
  const uint64_t *starts = nullptr;
  uint64_t *starts_owned = nullptr;  // the table set_data_pointer("INPUT") builds for a window matrix
  uint64_t n_tokens = 0;
  bool corpus_on_device = false;
  uint64_t shuffles = 0;          // shuffles applied so far: the seed of the next one
  bool shuffle_pending = false;   // the shuffle of the allocation, applied once the window order exists
};

[[noreturn]] void die(const char *where) {
  fprintf(stderr, "%s: %s\n", where, fv_last_error());
  exit(EXIT_FAILURE);
}

[[noreturn]] void die_msg(const char *where, const char *what) {
  fprintf(stderr, "%s: %s\n", where, what);
  exit(EXIT_FAILURE);
}

void one_gpu(const char *where, int device) {
  if (device != 0) die_msg(where, "this build runs on one GPU: the device argument must be 0");
}

// The corpus goes to the device once its length is known: from compute_inverse_word_frequency, or, for a
// driver that never calls it, from the farthest window of the table.
void upload_corpus(legacy_arrays *A, const legacy_descriptor *D, const char *where) {
  if (A->corpus_on_device) return;
  if (!A->trainer) die_msg(where, "model_arrays_allocate_memory has not been called");
  if (!A->corpus || (!A->starts && D->Ns_1)) die_msg(where, "set_up_INPUT_pointer has not been called");
  uint64_t n_tokens = A->n_tokens;
  if (n_tokens == 0)
    for (uint64_t i = 0; i < D->Ns_1; ++i)
      if (A->starts[i] + D->W > n_tokens) n_tokens = A->starts[i] + D->W;
  if (fv_trainer_set_corpus_starts(A->trainer, A->corpus, n_tokens, A->starts, D->Ns_1) != FV_OK) die(where);
  A->corpus_on_device = true;
  // flyvec/src/model_arrays.cu:180-198: the order is shuffled once when the arrays are allocated; here the order
  // exists from this moment on (a corpus handed over again starts from the identity and is shuffled again)
  if (A->shuffle_pending && fv_trainer_shuffle(A->trainer, A->shuffles++) != FV_OK) die(where);
}

}  // namespace

// ---- cuda_helpers ------------------------------------------------------------------------------

extern "C" void *do_gpu_cudaHostAlloc(unsigned long bytes) {
  void *p = nullptr;
  if (fv_host_alloc_pinned(bytes ? bytes : 1, &p) != FV_OK) die("do_gpu_cudaHostAlloc");
  return p;
}

extern "C" void *do_gpu_cudaMallocManaged(unsigned long bytes) { return do_gpu_cudaHostAlloc(bytes); }

extern "C" void *do_cpu_malloc(unsigned long bytes) { return malloc(bytes ? bytes : 1); }

extern "C" int get_cuda_num_devices(void) {
  int n = 0;
  if (fv_device_count(&n) != FV_OK || n < 1) die_msg("get_cuda_num_devices", "no HIP device is visible");
  return 1;
}

// ---- prune_input -------------------------------------------------------------------------------

extern "C" uint64_t getnum_samples(void *offsets, uint64_t n_sentences, uint64_t W) {
  uint64_t n = 0;
  if (fv_count_windows((const uint64_t *)offsets, n_sentences, W, &n) != FV_OK) die("getnum_samples");
  return n;
}

extern "C" void compute_offset_phrases(void *out, void *offsets, uint64_t n_sentences, uint64_t W) {
  uint64_t n = 0;
  if (fv_count_windows((const uint64_t *)offsets, n_sentences, W, &n) != FV_OK ||
      fv_build_window_starts((const uint64_t *)offsets, n_sentences, W, (uint64_t *)out, n) != FV_OK)
    die("compute_offset_phrases");
}

extern "C" void prune_input_data(void *data, uint64_t rows, uint64_t cols) {
  if (fv_prune_windows((int32_t *)data, rows, cols) != FV_OK) die("prune_input_data");
}

// ---- model_descriptor --------------------------------------------------------------------------

extern "C" void *model_create_descriptor(int num_gpus) {
  (void)num_gpus;
  return new legacy_descriptor();
}

extern "C" void set_model_param_int(uint64_t value, const char *key, void *descriptor) {
  legacy_descriptor *D = (legacy_descriptor *)descriptor;
  if (!D || !key) die_msg("set_model_param_int", "null argument");
#define FV_KEY(name)        \
  if (0 == strcmp(key, #name)) { \
    D->name = value;        \
    return;                 \
  }
  FV_KEY(IM_HEIGHT) FV_KEY(IM_WIDTH) FV_KEY(Nchannels) FV_KEY(Ns_1) FV_KEY(W) FV_KEY(ST) FV_KEY(hid) FV_KEY(Num)
  FV_KEY(p) FV_KEY(m) FV_KEY(vocabulary_size) FV_KEY(sparse_input) FV_KEY(frequency_scaling)
#undef FV_KEY
  fprintf(stderr, "set_model_param_int: unknown parameter %s\n", key);
}

extern "C" void set_model_param_float(float value, const char *key, void *descriptor) {
  legacy_descriptor *D = (legacy_descriptor *)descriptor;
  if (!D || !key) die_msg("set_model_param_float", "null argument");
#define FV_KEY(name)        \
  if (0 == strcmp(key, #name)) { \
    D->name = value;        \
    return;                 \
  }
  FV_KEY(initial_learning_rate) FV_KEY(delta) FV_KEY(prec) FV_KEY(mu) FV_KEY(sigma) FV_KEY(Lmid) FV_KEY(Lbase)
#undef FV_KEY
  fprintf(stderr, "set_model_param_float: unknown parameter %s\n", key);
}

extern "C" void compute_model_derived_parameters(void *descriptor) {
  legacy_descriptor *D = (legacy_descriptor *)descriptor;
  if (!D) die_msg("compute_model_derived_parameters", "null descriptor");
  // flyvec/src/model_descriptor.cu:91-112: with sparse input the matrix has a context and a target block
  D->N = D->sparse_input ? 2 * D->vocabulary_size : D->W * D->W * D->Nchannels;
}

extern "C" void copy_model_params(void *descriptor, int source, int destination) {
  (void)descriptor;
  (void)source;
  (void)destination;
}

extern "C" void print_model_params(void *descriptor) {
  const legacy_descriptor *D = (const legacy_descriptor *)descriptor;
  if (!D) return;
  printf(" hid = %llu  W = %llu  Num = %llu  Ns_1 = %llu  vocabulary_size = %llu  N = %llu\n",
         (unsigned long long)D->hid, (unsigned long long)D->W, (unsigned long long)D->Num, (unsigned long long)D->Ns_1,
         (unsigned long long)D->vocabulary_size, (unsigned long long)D->N);
  printf(" initial_learning_rate = %g  delta = %g  prec = %g  Lmid = %g  Lbase = %g  sparse_input = %llu  frequency_scaling = %llu\n",
         (double)D->initial_learning_rate, (double)D->delta, (double)D->prec, (double)D->Lmid, (double)D->Lbase,
         (unsigned long long)D->sparse_input, (unsigned long long)D->frequency_scaling);
}

// ---- model_arrays ------------------------------------------------------------------------------

extern "C" void *model_create_arrays(int num_gpus) {
  (void)num_gpus;
  return new legacy_arrays();
}

extern "C" void model_arrays_allocate_memory(void *descriptor, void *arrays, int num_gpus) {
  const legacy_descriptor *D = (const legacy_descriptor *)descriptor;
  legacy_arrays *A = (legacy_arrays *)arrays;
  if (!D || !A) die_msg("model_arrays_allocate_memory", "null argument");
  if (num_gpus != 1) die_msg("model_arrays_allocate_memory", "this build runs on one GPU");
  if (!D->sparse_input || !D->frequency_scaling)
    die_msg("model_arrays_allocate_memory",
            "only the text model of flyvec_train is built: sparse_input = 1 and frequency_scaling = 1");
  if (A->trainer) die_msg("model_arrays_allocate_memory", "called twice");
  // flyvec/src/model_descriptor.cu:30 sets p = m = 2 and the reference's driver never changes them; the update
  // rule built here is the p = 2 one (ds = -xx W + input) with the anti-Hebbian term on the 2nd neuron
  if (D->p != 2) die_msg("model_arrays_allocate_memory", "only p = 2 (the reference's default) is built");
  if (D->m != 2) die_msg("model_arrays_allocate_memory", "only m = 2 (the reference's default) is built");
  fv_train_config cfg;
  memset(&cfg, 0, sizeof cfg);
  cfg.vocab = D->vocabulary_size;
  cfg.hid = (uint32_t)D->hid;
  cfg.window = (uint32_t)D->W;
  cfg.batch = (uint32_t)D->Num;
  cfg.tie_rule = 1;  // the reference's own reduction order on exact ties (flyvec/src/cuda_funcs.cu:488-561)
  cfg.initial_learning_rate = D->initial_learning_rate;
  cfg.delta = D->delta;
  cfg.prec = D->prec;
  cfg.lmid = D->Lmid;
  cfg.lbase = D->Lbase;
  cfg.prune_duplicates = 0;
  if (fv_trainer_create(&cfg, &A->trainer) != FV_OK) die("model_arrays_allocate_memory");
  // a final partial minibatch as the reference's launch sizes treat it (flyvec/src/cuda_funcs.cu:1679, :1700-1732)
  if (fv_trainer_set_stale_tail(A->trainer, 1) != FV_OK) die("model_arrays_allocate_memory");
  if (!A->synapses) {
    void *p = nullptr;
    if (fv_host_alloc_pinned((size_t)D->hid * 2 * D->vocabulary_size * sizeof(float), &p) != FV_OK)
      die("model_arrays_allocate_memory");
    memset(p, 0, (size_t)D->hid * 2 * D->vocabulary_size * sizeof(float));
    A->synapses = (float *)p;
    A->synapses_owned = true;
  }
  A->shuffle_pending = true;  // flyvec/src/model_arrays.cu:180-198, see upload_corpus
}

extern "C" void push_INPUT_memory_to_GPU(void *arrays, void *descriptor, int device, const char *type) {
  (void)type;
  one_gpu("push_INPUT_memory_to_GPU", device);
  upload_corpus((legacy_arrays *)arrays, (const legacy_descriptor *)descriptor, "push_INPUT_memory_to_GPU");
}

extern "C" void *get_data_pointer(const char *name, void *arrays, int device) {
  legacy_arrays *A = (legacy_arrays *)arrays;
  one_gpu("get_data_pointer", device);
  if (!A || !name || 0 != strcmp(name, "synapses")) die_msg("get_data_pointer", "only \"synapses\" is served");
  if (!A->synapses) die_msg("get_data_pointer", "model_arrays_allocate_memory has not been called");
  return A->synapses;
}

// flyvec/src/model_arrays.cu:320: "INPUT" is a matrix of Ns_1 rows of IM_HEIGHT * IM_WIDTH * Nchannels values, row i
// being input i. For the text model (type "i4") that is a matrix of windows already cut out: window i starts at
// token i * row of it. The image types belong to the models that are not built here.
extern "C" void set_data_pointer(const char *name, void *arrays, void *descriptor, void *ptr, const char *type,
                                 int device) {
  legacy_arrays *A = (legacy_arrays *)arrays;
  const legacy_descriptor *D = (const legacy_descriptor *)descriptor;
  one_gpu("set_data_pointer", device);
  if (!A || !D || !name || !ptr || !type) die_msg("set_data_pointer", "null argument");
  if (0 != strcmp(name, "INPUT")) {
    fprintf(stderr, "set_data_pointer: unknown array %s\n", name);  // what the reference does with another name
    return;
  }
  if (0 != strcmp(type, "i4") && 0 != strcmp(type, "I4"))
    die_msg("set_data_pointer", "only int32 token ids (type \"i4\") are served: the image models are outside this library");
  const uint64_t row = D->IM_HEIGHT * D->IM_WIDTH * D->Nchannels;
  if (row == 0 || D->Ns_1 == 0) die_msg("set_data_pointer", "IM_HEIGHT * IM_WIDTH * Nchannels and Ns_1 must be set first");
  if (row < D->W) die_msg("set_data_pointer", "a row of the INPUT matrix is shorter than the window W");
  free(A->starts_owned);
  A->starts_owned = (uint64_t *)malloc(D->Ns_1 * sizeof(uint64_t));
  if (!A->starts_owned) die_msg("set_data_pointer", "out of memory");
  for (uint64_t i = 0; i < D->Ns_1; ++i) A->starts_owned[i] = i * row;
  A->corpus = (const int32_t *)ptr;
  A->starts = A->starts_owned;
  A->n_tokens = D->Ns_1 * row;
  A->corpus_on_device = false;
}

// No counterpart in the reference, whose matrix lives in managed memory of its own: makes `ptr` (K x 2V fp32,
// row-major, host memory of the caller that outlives the model) the matrix get_data_pointer("synapses") serves
// and the epochs read and write.
extern "C" void flyvec_legacy_set_synapses(void *arrays, void *ptr) {
  legacy_arrays *A = (legacy_arrays *)arrays;
  if (!A || !ptr) die_msg("flyvec_legacy_set_synapses", "null argument");
  if (A->synapses_owned) (void)fv_host_free_pinned(A->synapses);
  A->synapses = (float *)ptr;
  A->synapses_owned = false;
}

extern "C" void set_up_INPUT_pointer(const char *name, void *arrays, void *descriptor, void *corpus, void *starts,
                                     const char *type, int device) {
  (void)name;
  (void)descriptor;
  legacy_arrays *A = (legacy_arrays *)arrays;
  one_gpu("set_up_INPUT_pointer", device);
  if (!A || !corpus) die_msg("set_up_INPUT_pointer", "null argument");
  if (!type || (0 != strcmp(type, "i4") && 0 != strcmp(type, "I4")))
    die_msg("set_up_INPUT_pointer", "only int32 token ids (type \"i4\") are served");
  A->corpus = (const int32_t *)corpus;
  A->starts = (const uint64_t *)starts;
  A->corpus_on_device = false;
}

extern "C" void compute_inverse_word_frequency(void *arrays, void *descriptor, void *corpus, uint64_t n_tokens,
                                               int device) {
  legacy_arrays *A = (legacy_arrays *)arrays;
  one_gpu("compute_inverse_word_frequency", device);
  if (!A || !descriptor || !corpus) die_msg("compute_inverse_word_frequency", "null argument");
  if (A->corpus && A->corpus != (const int32_t *)corpus)
    die_msg("compute_inverse_word_frequency", "the corpus differs from the one given to set_up_INPUT_pointer");
  A->corpus = (const int32_t *)corpus;
  A->n_tokens = n_tokens;
  A->corpus_on_device = false;
  upload_corpus(A, (const legacy_descriptor *)descriptor, "compute_inverse_word_frequency");
}

extern "C" void do_reshuffle_indices(void *descriptor, void *arrays, int device) {
  legacy_arrays *A = (legacy_arrays *)arrays;
  one_gpu("do_reshuffle_indices", device);
  upload_corpus(A, (const legacy_descriptor *)descriptor, "do_reshuffle_indices");
  if (fv_trainer_shuffle(A->trainer, A->shuffles++) != FV_OK) die("do_reshuffle_indices");
}

// No counterpart in the reference, which never frees its handles: returns the trainer, the matrix and the
// two handles, for hosts that create more than one model in a process.
extern "C" void flyvec_legacy_release(void *descriptor, void *arrays) {
  legacy_arrays *A = (legacy_arrays *)arrays;
  if (A) {
    if (A->trainer) (void)fv_trainer_destroy(A->trainer);
    if (A->synapses_owned && A->synapses) (void)fv_host_free_pinned(A->synapses);
    free(A->starts_owned);
    delete A;
  }
  delete (legacy_descriptor *)descriptor;
}

// ---- cuda_funcs --------------------------------------------------------------------------------

extern "C" void launch_epoch_INPUT_AS_INT(void *descriptor, void *arrays, int num_gpus, uint64_t epoch_id,
                                          uint64_t n_epochs) {
  legacy_arrays *A = (legacy_arrays *)arrays;
  const legacy_descriptor *D = (const legacy_descriptor *)descriptor;
  if (!A || !D) die_msg("launch_epoch_INPUT_AS_INT", "null argument");
  if (num_gpus != 1) die_msg("launch_epoch_INPUT_AS_INT", "this build runs on one GPU");
  upload_corpus(A, D, "launch_epoch_INPUT_AS_INT");
  // the driver reads and writes the matrix through get_data_pointer between the epochs
  if (fv_trainer_set_weights(A->trainer, A->synapses) != FV_OK) die("launch_epoch_INPUT_AS_INT");
  float eps = 0.0f;
  (void)fv_trainer_epoch_eps(A->trainer, epoch_id, n_epochs, &eps);
  printf("epoch %llu of %llu: learning rate %g\n", (unsigned long long)epoch_id, (unsigned long long)n_epochs, (double)eps);
  if (fv_trainer_run_epoch(A->trainer, epoch_id, n_epochs) != FV_OK) die("launch_epoch_INPUT_AS_INT");
  if (fv_trainer_get_weights(A->trainer, A->synapses) != FV_OK) die("launch_epoch_INPUT_AS_INT");
}

extern "C" void launch_epoch_INPUT_AS_IMAGE(void *descriptor, void *arrays, int num_gpus, uint64_t epoch_id,
                                            uint64_t n_epochs) {
  (void)descriptor; (void)arrays; (void)num_gpus; (void)epoch_id; (void)n_epochs;
  die_msg("launch_epoch_INPUT_AS_IMAGE", "the image model is outside this library (text model only)");
}

extern "C" void launch_epoch_INPUT_AS_FLOAT(void *descriptor, void *arrays, int num_gpus, uint64_t epoch_id,
                                            uint64_t n_epochs) {
  (void)descriptor; (void)arrays; (void)num_gpus; (void)epoch_id; (void)n_epochs;
  die_msg("launch_epoch_INPUT_AS_FLOAT", "the dense-input model is outside this library (text model only)");
}
