/*
 * libditango_probes.so -- measurement aids of bench.py for the MI355X (gfx950) kernels of
 * libditango_hip.so.  NOT part of the drop-in ABI: nothing here replaces a call site of the
 * reference, no stability is promised, and the product library neither exports nor needs them.
 * Each probe puts a measured ceiling next to a nominal peak (dense bf16 MFMA rate, HBM bandwidth).
 * Every function enqueues one kernel on `stream` (a hipStream_t passed as void*), allocates nothing,
 * does not synchronise, and returns DTP_OK or a negative code; dtp_last_error() holds the message.
 */
#ifndef DITANGO_PROBES_H
#define DITANGO_PROBES_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define DTP_OK 0
#define DTP_ERR_INVALID (-1)
#define DTP_ERR_HIP (-3)
#define DTP_MAX_STREAMS 64 /* streams one read-probe launch can address */

const char* dtp_last_error(void);

/*
 * Reads n_streams device buffers of `bytes` bytes
 * each (a multiple of 256) with the access pattern of dt_merge_states (libditango_hip.so) (a workgroup takes 32
 * consecutive 256-byte rows of every stream, eight streams in flight at a time) and discards the
 * data.  Its rate is what this part's memory system delivers to that pattern, the yardstick next to
 * the nominal HBM peak for the merge and cache kernels.  sink: one device word, (almost) never written.
 */
int dtp_hbm_read_probe(const void* const* streams, int32_t n_streams, int64_t bytes, uint32_t* sink, void* stream);

/*
 * `workgroups` workgroups of 8 wavefronts (two per
 * SIMD, the attention kernel's launch shape) each issue 4 * iters (iters a multiple of 4) back-to-back
 * v_mfma_f32_32x32x16_bf16 on registers -- 32768 FLOP apiece, so a launch does
 * workgroups * 8 * 4 * iters * 32768 FLOP -- and nothing else.  Its rate is what the part sustains
 * when only the matrix pipes work (the power limit holds the shader clock below nominal): the
 * yardstick next to the nominal MFMA peak for dt_attn_*.  sink: one device word, (almost) never written.
 */
int dtp_mfma_probe(int32_t workgroups, int32_t iters, float* sink, void* stream);

/*
 * The launch shape of dtp_mfma_probe, but only ONE wavefront of each SIMD issues the 4 * iters MFMAs (a launch does workgroups * 4 * 4 * iters * 32768 FLOP); with
 * with_softmax != 0 the other wavefront of the SIMD issues, per MFMA of its neighbour, the vector
 * instructions that the online softmax of dt_attn_* spends per MFMA at that head dimension: at 128 one
 * v_fma_f32, one v_exp_f32, one v_add_f32 and half a v_cvt_pk_bf16_f32; at 64 twice that.  The launch
 * reserves the attention kernel's LDS for head_dim, so one (128) or two (64) workgroups share a CU as
 * they do there.  The MFMA rate with the softmax against the rate without is the share of the matrix pipe
 * that the wavefronts of a SIMD can keep busy side by side for that instruction mix: the ceiling of the
 * attention kernel's MFMA utilisation before any LDS traffic, barrier or tile load.  sink: one device
 * word, (almost) never written.
 */
int dtp_coissue_probe(int32_t workgroups, int32_t iters, int32_t head_dim, int32_t with_softmax, float* sink,
                      void* stream);

/*
 * Launches a kernel of `workgroups` x `threads` that does nothing.  Timed back to back it gives the floor of a
 * launch of that grid (dispatch of the workgroups included) -- what a short HBM-bound launch (a merge or a
 * cache copy of a few MB) pays before it moves a byte.
 */
int dtp_empty_launch(int32_t workgroups, int32_t threads, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* DITANGO_PROBES_H */
