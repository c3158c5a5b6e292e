// Arguments of the streaming decode kernel (decode_stream.hip), shared with the text session (text_model.hip).
#pragma once
#include "moon_internal.hpp"

struct StreamParams {
    // small vectors and the embedding table
    const half_t *wte, *ln_w, *ln_b, *qkv_b, *fc1_b, *fc2_b, *out_b, *lin_b, *lno_w, *lno_b;
    // the streamed matrices live in one allocation of w_bytes (< 4 GiB) at w_base, each at its byte offset:
    // qkv_w [L][3d][d], fc1_w [L][ffn][d], lin_w [V][d] in the text layout; fc2_wt [L][ffn][d] (row j = fc2_w[:, j]) and
    // out_wt [L][d][d] (row k = out_w[:, k]) transposed
    const half_t *w_base;
    size_t w_bytes;
    uint32_t off_qkv, off_fc1, off_fc2t, off_outt, off_lin;
    half_t *cache_k, *cache_v; // [L][H][max_seq][64]
    const float *freqs;        // [max_seq][rot_dim/2][2]
    const half_t *hidden_first; // [d] hidden row the first LM head reads (last row of the preceding forward)
    half_t *hidden_out;         // [d] hidden state after the last step (plain store)
    half_t *logits;             // [V] of the last LM head
    // exchange buffers; every word carries the tag of the layer-step that wrote it
    uint32_t *hid_t;            // [d]      f16 bits | tag16 << 16 : hidden state after a layer
    uint32_t *qkv_t;            // [3d]     f16 bits | tag16 << 16 : q | k | v of the new token
    unsigned long long *ap_t;   // [H][8][66]       f32 bits | tag << 32 : attention partials (o[64], m, l) per (head, split)
    float *rp;                  // [2 kinds: fc2, out_proj][256 source units][256 slots][8] f32: partial sums for a reducer
    uint32_t *rp_flag;          // [2 kinds][256 source units][8 wavefronts]: tag of the layer-step whose partial sums are complete
    unsigned long long *am_t;   // [512]   f16 bits | tag16 << 16 | index << 32 : arg-max pair of a workgroup
    uint32_t *error;            // raised when a wait expires; every wait ends when it is up
    uint32_t *out_ids;          // [n_steps]
    int L, V, rot_dim, max_seq, pos0, n_steps;
    float eps;
    uint32_t gen0;              // tags used by earlier launches on these buffers
    long long timeout_ticks;    // bound of every wait, 100 MHz ticks
    int debug;                  // tuning builds only: bit 0 = the MLP workgroups stream nothing (wrong results)
    long long *trace;           // optional [L][512][8] stamps of the last step (tuning aid), or null
};

constexpr int STREAM_GRID = 512, STREAM_THREADS = 512;
constexpr int STREAM_D = 2048, STREAM_FFN = 8192, STREAM_H = 32, STREAM_HD = 64;
constexpr size_t STREAM_HID_WORDS = STREAM_D, STREAM_QKV_WORDS = 3 * STREAM_D;
constexpr size_t STREAM_AP_WORDS = size_t(STREAM_H) * 8 * 66, STREAM_RP_FLOATS = size_t(2) * 256 * 256 * 8, STREAM_RP_FLAGS = 2 * 256 * 8, STREAM_AM_WORDS = 512;

bool decode_stream_supported(moon_ctx *ctx, size_t d, size_t ffn, size_t H, size_t D, size_t max_seq, size_t L, size_t V);
int launch_decode_stream(moon_ctx *ctx, const StreamParams &p);
