// Plain C++ references of the HIP kernels: one loop nest per operation, double precision inside,
// float arrays in and out, no blocking, no vector types, no GPU.  The kernel tests run each kernel
// and its reference on the same arrays.  Formulas cite the reference engine they come from
// (paths under crates/burn-lm-llama/src/).
#pragma once

#ifdef __cplusplus
extern "C" {
#endif

// out[t, :] = table[ids[t], :]                                        (nn/transformer.rs:95)
void ref_embed_gather(const float* table, const int* ids, float* out, int T, int D);

// v = h[r] + sum_p delta[p][r];  h[r] = v if write_h;  out[i] = v / sqrt(mean(v^2) + eps) * gamma,
// r = rows ? rows[i] : i                                              (nn/transformer.rs:60-62, 248-255)
void ref_add_rmsnorm(float* h, const float* delta, int n_planes, long long plane_stride, const float* gamma,
                     float* out, const int* rows, int n_out, int D, float eps, int write_h);

// Rotation of the q and k heads of packed rows [T][(nh + 2 nkv) hd] by the angles of each token's
// position (cos_sin [positions][hd/2][2]); pairing 0: lanes (2i, 2i+1), 1: lanes (i, i + hd/2)
// (nn/pos_encoding.rs:56-79).  q is rotated in place; rotated k and plain v go into the paged planes
// (key plane [pages][nkv][page][hd], value plane [pages][nkv][hd][page]) at the token's position;
// tokens of no sequence (token_seq < 0) are left alone.
void ref_rope_kv_write(float* qkv, const int* positions, const int* token_seq, const int* block_table, int table_width,
                       const float* cos_sin, float* kcache, float* vcache, int page_size, int T, int nh, int nkv, int hd,
                       int pairing);

// out = silu(gate) * up for rows [T][2 I] = [gate | up]               (nn/fftn.rs:44-46)
void ref_swiglu(const float* gate_up, float* out, int T, int I);

// Attention of every token's query heads over its sequence's cached keys 0..position (and, with a
// window w > 0, the last w of them): softmax(q k^T * scale) v, query head h reading key-value head
// h / (nh / nkv)                                                      (nn/attention/mha.rs:143-185)
void ref_attention(const float* q, int q_row_stride, float* out, const int* positions, const int* token_seq,
                   const int* block_table, int table_width, const float* kcache, const float* vcache, int page_size,
                   int T, int nh, int nkv, int hd, float scale, int window);

// C[M][N] = A[M][K] W[N][K]^T                                         (a Linear without bias, nn/attention/mha.rs:121-140)
void ref_linear(const float* A, const float* W, float* C, int M, int N, int K);
// C[M][I] = silu(A gate^T) * (A up^T) for W = [gate rows; up rows] ([2 I][K])
void ref_gated_linear(const float* A, const float* W, float* C, int M, int I, int K);

// First index of each row's maximum                                   (generation/sampling.rs:18)
void ref_argmax(const float* logits, int* out, int R, int V, int ld);
// softmax(logits / temperature); the nucleus keeps a token while the mass of the tokens strictly more
// likely than it is below top_p; the pick is the first kept token, in index order, at which the kept
// mass so far exceeds u * (kept mass)                                 (generation/sampling.rs:50-69)
void ref_sample(const float* logits, const float* uniforms, int* out, int R, int V, int ld, float temperature,
                float top_p);

#ifdef __cplusplus
}
#endif
