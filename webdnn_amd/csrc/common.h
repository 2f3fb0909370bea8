// Internal helpers shared by the translation units of libwebdnn_hip.so.
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

#include "webdnn_hip.h"

namespace wdh {

// Records `code` + a printf-style message as the calling thread's last error
// and returns `code`, so call sites can `return fail(...)`.
int fail(int code, const char *fmt, ...) __attribute__((format(printf, 2, 3)));
void clear_error();

bool initialised();
bool capturing();        // a graph capture is open on the stream
void poison_capture();   // the open capture cannot be completed (wdh_graph_end will fail)
hipStream_t stream();
int compute_units();
int device();           // the device wdh_init selected
int lane();             // the current lane (wdh_set_lane)
bool branch_open();     // a side branch of the run being recorded is open (wdh_branch_begin .. wdh_branch_join)
// The pool asks the driver for at most `bytes` in total (0 = no limit); blocks it already holds stay.
void set_memory_limit(uint64_t bytes);
// Looks up the device address of the static workspace of wdh_gemm_static for `device`,
// which must be the current device (called by wdh_init).
int init_static_scratch(int device);
// Raises the dynamic LDS limit of the attention kernels on the current device (called by wdh_init).
int init_attention();
// Device resources of the contraction kernels that outlive a call (called by wdh_init / at shutdown).
int init_contraction(int device);
int contraction_lane_init(int lane);   // (when wdh_set_lane creates a side lane)
void release_contraction();
// The buffer behind `h` is about to be freed or overwritten: drops what the conv code derived from it.
void conv_forget_weights(wdh_buf h);
// After a synchronisation: fails if a contraction kernel reported that it gave up a wait.
int contraction_check();

// Handle -> device pointer.  Returns nullptr (and records WDH_EINVAL) for an
// unknown handle.  A zero-byte buffer resolves to a non-null dummy pointer.
void *resolve(wdh_buf h, size_t *bytes);

// Resolves `h` and checks that it holds at least `need` bytes.
// On failure returns false after recording the error (`what` names the operand).
bool operand(wdh_buf h, size_t need, const char *what, void **out);

// The stem convolution's own kernel (conv_patch.hip): whether a geometry qualifies, and the launch.
bool conv_patch_applies(int c, int cout, int kh, int kw, int sh, int sw, int dh, int dw, int group, int h, int w,
                        int pt, int pl, int oh, int ow);
int conv_patch_launch(const float *X, const float *W, const float *Bias, const float *R, float *Y, int n,
                      int h, int w, int oh, int ow, int pt, int pl, int relu);

// The transforms of the minimal-filtering forms of a 3x3 stride-1 conv (winograd.hip), r = 2 for F(2x2, 3x3)
// (16 positions) or 4 for F(4x4, 3x3) (36 positions): filters -> U [positions][cout][c], input ->
// V [positions][c][pitch], products M [positions][cout][pitch] (+ bias, residual, Relu) -> Y.
long long wino_tiles(int r, int n, int oh, int ow);
long long wino_pitch(long long tiles);
int wino_filter_launch(int r, const float *W, float *U, int cout, int c);
int wino_input_launch(int r, const float *X, float *V, int n, int c, int h, int w, int oh, int ow, int pt, int pl);
int wino_output_launch(int r, const float *M, const float *Bias, const float *R, float *Y, int n, int cout, int oh,
                       int ow, int relu);

// Frees the per-geometry tap tables of the conv kernel (called at shutdown).
void release_conv_tables();

}  // namespace wdh

#define WDH_REQUIRE_INIT()                                                   \
  do {                                                                       \
    if (!wdh::initialised())                                                 \
      return wdh::fail(WDH_ESTATE, "%s: wdh_init() has not succeeded",       \
                       __func__);                                            \
  } while (0)

// Operator entry points: side lanes take recorded work only (their buffers come from a pool whose
// hand-overs are ordered on lane 0).
#define WDH_REQUIRE_COMPUTE_LANE()                                           \
  do {                                                                       \
    if (wdh::lane() != 0 && !wdh::capturing())                               \
      return wdh::fail(WDH_ESTATE, "%s: lane %d takes recorded work only (wdh_graph_begin first, or wdh_set_lane(0))", \
                       __func__, wdh::lane());                               \
  } while (0)

#define WDH_HIP_CHECK(expr)                                                  \
  do {                                                                       \
    hipError_t e_ = (expr);                                                  \
    if (e_ != hipSuccess)                                                    \
      return wdh::fail(WDH_EHIP, "%s: %s failed: %s", __func__, #expr,       \
                       hipGetErrorString(e_));                               \
  } while (0)

// Checked after every kernel launch: catches bad launch configurations.
#define WDH_LAUNCH_CHECK()                                                   \
  do {                                                                       \
    hipError_t e_ = hipGetLastError();                                       \
    if (e_ != hipSuccess)                                                    \
      return wdh::fail(WDH_EHIP, "%s: kernel launch failed: %s", __func__,   \
                       hipGetErrorString(e_));                               \
  } while (0)
