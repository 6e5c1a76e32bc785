/*
 * trips_oracle.h -- CPU oracle of the TRIPS splat path. TEST INFRASTRUCTURE, NOT PRODUCT CODE.
 *
 * Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may load this library.
 * Same descriptor structs as the device library (include/trips_splat.h) but every pointer is a
 * HOST pointer. See trips_oracle.cpp for which reference lines each function restates and for
 * what pins it.
 */
#ifndef TRIPS_ORACLE_H
#define TRIPS_ORACLE_H

#include "../include/trips_splat.h"

#ifdef __cplusplus
extern "C" {
#endif

typedef struct OracleForwardOut {
    float* image[TRIPS_MAX_LAYERS]; /* per layer, layout per desc->layout; required */
    /* everything below is view-major and may be NULL if not wanted (lists/retained/alpha are
       required when a backward follows) */
    float* ip;          /* [B,N,2] layer-0 image position (temp_full_buffer cols 0,1) */
    float* depth;       /* [B,N]   -1 = culled (temp_depth_buffer) */
    float* size_px;     /* [B,N]   projected point size (temp_full_buffer col 3) */
    int32_t* max_layer; /* [B,N]   layers written (temp_max_layer_buffer) */
    int32_t* lengths;   /* [B,P]   per-pixel list length before the top-K cut */
    int32_t* lists;     /* [B,P,K] sorted point ids, -1 padded */
    int32_t* retained;  /* [B,P]   entries with transmittance >= 0.001 */
    float* alpha;       /* [B,P,K] alpha of retained entries (bw_sorted_maxed[...,2]); -1 elsewhere */
    int64_t* counters;  /* [B,4]   valid points, E, R, P */
} OracleForwardOut;

int oracle_num_threads(void);
void oracle_set_num_threads(int n);

int oracle_layer_sizes(const TripsSplatDesc* desc, int32_t* w, int32_t* h);
int oracle_splat_forward(const TripsSplatDesc* desc, const TripsSplatIn* in, const OracleForwardOut* out);
int oracle_splat_backward(const TripsSplatDesc* desc, const TripsSplatIn* in, const OracleForwardOut* fwd,
                          const float* const grad_image[TRIPS_MAX_LAYERS], const TripsSplatGrads* grads);
int oracle_adam_step(const TripsAdamTensor* tensors, int n_tensors);
int oracle_apply_tangent(double* tangent, double* poses_se3, int n);

/* scalar pieces exported so that tests can pin them one by one */
float oracle_softplus(float x);
float oracle_softplus_backward(float x);
float oracle_layer_factor(float size_px, int layer, int num_layers, float* grad);
void oracle_log2_floor_ceil(float s, int* lo, int* hi);
/* projects one world point with pose row `pose` (8 doubles) and intrinsics row `intr` (13 floats);
   out = {ip.x, ip.y, z, size_px_per_unit (= K.fx*crop.fx / z)} */
void oracle_project_point(const double* pose, const float* intr, const TripsView* view, float dist_cutoff,
                          const float* xyz, float* out4);
/* image-space gradient (2) -> g_point(3), g_pose(6), g_k(5), g_dis(8); PointRendererHelper.h:434-494 */
void oracle_project_point_backward(const double* pose, const float* intr, const TripsView* view, float dist_cutoff,
                                   const float* xyz, const float* grad2, float* g_point3, float* g_pose6, float* g_k5,
                                   float* g_dis8);
#ifdef __cplusplus
}
#endif
#endif
