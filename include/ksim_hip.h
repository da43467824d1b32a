/* ksim_hip.h — C ABI of libksimhip.so: the MI355X (gfx950) rollout hot path of ksim.
 *
 * Every entry point is asynchronous on the caller's HIP stream, allocates nothing,
 * never synchronises the host, keeps no mutable global state (re-entrant) and
 * returns 0 on success or a negative KS_E* code; ks_last_error() gives the
 * calling thread's last message.  All pointers are DEVICE pointers unless a
 * parameter says "host".  The caller owns every buffer.
 *
 * Each declaration cites the reference (kscalelabs/ksim 0.2.10) interface it
 * replaces as file:line.
 */
#ifndef KSIM_HIP_H_
#define KSIM_HIP_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void* ks_stream_t; /* a hipStream_t; NULL = the default stream */

enum {
  KS_OK = 0,
  KS_EINVAL = -1,  /* bad size / flag / null pointer */
  KS_ELAUNCH = -2, /* HIP reported a launch error */
  KS_ELIMIT = -3   /* size beyond a compiled-in maximum */
};

/* Library identity / error text (host). */
const char* ks_version(void);
const char* ks_last_error(void);

/* ------------------------------------------------------------------ GAE / returns
 * Replaces compute_ppo_inputs, ksim/task/ppo.py:54-121.
 * Layout "bt": arrays are (B, T) row-major like the reference's *_bt arguments;
 * one wavefront scans one env row with shuffles (segmented reverse scan).
 * Layout "tn": arrays are (T, N) time-major with env fastest (the rollout
 * buffer's own layout); one lane walks one env back in time.
 *   values, rewards : f32     dones, successes : 1 byte per element, non-zero = true
 *   successes may be NULL (treated as all false).
 *   gae, returns, targets : f32 outputs (targets = returns when monte_carlo_returns
 *   else gae + values, ppo.py:107).  Any output may be NULL.
 */
int ks_gae_bt(ks_stream_t stream, int64_t B, int64_t T, const float* values, const float* rewards,
              const uint8_t* dones, const uint8_t* successes, float gamma, float lam,
              int monte_carlo_returns, float* gae, float* returns, float* targets);
int ks_gae_tn(ks_stream_t stream, int64_t T, int64_t N, const float* values, const float* rewards,
              const uint8_t* dones, const uint8_t* successes, float gamma, float lam,
              int monte_carlo_returns, float* gae, float* returns, float* targets);

/* Advantage normalisation over ALL n elements, population std clipped at 1e-6
 * (ppo.py:116-119).  workspace: >= KS_REDUCE_WORKSPACE_BYTES bytes of device memory. */
#define KS_REDUCE_WORKSPACE_BYTES (2 * 1024 * 8 + 64)
int ks_normalize_advantages(ks_stream_t stream, int64_t n, const float* gae, float* advantages,
                            void* workspace);

/* ------------------------------------------------------------------ PPO loss
 * Replaces compute_ppo_loss + clipped_value_loss (ppo.py:124-135,149-246) and the
 * total "mean over (B,T) of the summed terms" (ppo.py:473-486).
 *   n = B*T elements, A = action dims; log-probs / entropy are (n, A) row-major.
 *   entropy may be NULL (term omitted, ppo.py:237-239).
 *   policy/value/kl/entropy_loss: per-element outputs (n), each may be NULL.
 *   loss_out: one f32 (device), may be NULL.  workspace as above.
 */
typedef struct KsPpoLossParams {
  float clip_param;      /* ppo.py:259 default 0.2 */
  float value_loss_coef; /* 0.5 */
  float entropy_coef;    /* 0.008 */
  float kl_coef;         /* 1e-3 */
  float log_clip_value;  /* 5.0 */
  float kl_scale;        /* adaptive-KL runtime factor, ppo.py:475; 1.0 */
  int32_t use_clipped_value_loss; /* 1 */
} KsPpoLossParams;
int ks_ppo_loss(ks_stream_t stream, int64_t n, int32_t A, const KsPpoLossParams* params /*host*/,
                const float* advantages, const float* value_targets, const float* on_log_probs,
                const float* on_values, const float* off_log_probs, const float* off_values,
                const float* off_entropy, float* policy_loss, float* value_loss, float* kl_loss,
                float* entropy_loss, float* loss_out, void* workspace);

/* ------------------------------------------------------------------ reward total + done/success
 * Replaces the scale/sum/clip of get_rewards (ksim/task/rl.py:219-239) and the
 * ternary -> boolean combination of terminations (rl.py:1049-1050).
 *   components: (K, n) f32, scales: K host floats (sign already folded for *Penalty).
 *   use_clip_min/max: 0 = no clip.  total: (n) f32, may be NULL.
 *   terminations: (k, n) int8 in {-1,0,+1}; done/success: (n) uint8; pass k = 0 to skip.
 */
#define KS_MAX_REWARD_TERMS 32
int ks_reward_total(ks_stream_t stream, int64_t n, int32_t K, const float* components,
                    const float* scales /*host*/, int32_t use_clip_min, float clip_min,
                    int32_t use_clip_max, float clip_max, float* total, int32_t k,
                    const int8_t* terminations, uint8_t* done, uint8_t* success);

#ifdef __cplusplus
}
#endif
#endif /* KSIM_HIP_H_ */
