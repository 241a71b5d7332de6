// Thunk specs of the LLaMA path: type inference, kernel dispatch through the C ABI, and
// adjoint rules.  Forward specs stand for the reference's thunk chains
// (src/librarium/llama.rs:420-548); each pop_adj stages the fused adjoint thunk(s) in the
// order the reference's AD emits the corresponding contributions (src/spine.rs:447-690).
#pragma once
#include "runtime.h"

namespace cacti {

std::unique_ptr<ThunkSpec> make_embed();                              // (W, tok) -> y
std::unique_ptr<ThunkSpec> make_rms_norm(float eps);                  // (x, w) -> y
std::unique_ptr<ThunkSpec> make_matmul(bool ta, bool tb, float alpha);   // (a, b) -> c, 2-d
std::unique_ptr<ThunkSpec> make_block_matmul(bool ta, bool tb, float alpha, int64_t H);   // [R,H*C]
// n products x W_i^T of one shape in one launch: (x, W_1 .. W_n) -> (y_1 .. y_n), 2 <= n <= 4; group_adjoints:
// their weight gradients as one grouped thunk too (else the adjoint thunks of n separate matmul thunks)
std::unique_ptr<ThunkSpec> make_projections(int n, bool group_adjoints);
// the two block products of causal attention, computed on the lower triangle only
std::unique_ptr<ThunkSpec> make_causal_scores(float alpha, int64_t H);   // (q, k) -> a q k^T
std::unique_ptr<ThunkSpec> make_causal_pv(int64_t H);                    // (p16, v) -> p16 v
// the whole block (scores, mask, softmax, product with v) as one thunk: (q, k, v) -> o, row statistics
std::unique_ptr<ThunkSpec> make_attention(float alpha, int64_t H);
std::unique_ptr<ThunkSpec> make_rope(int64_t H);                      // (x [S,H*Dh], cos, sin) -> y
std::unique_ptr<ThunkSpec> make_rope2(int64_t H);                     // (q, k, cos, sin) -> (qr, kr), one launch
std::unique_ptr<ThunkSpec> make_causal_softmax(int64_t H);            // (s16 [S,H*S]) -> p16
std::unique_ptr<ThunkSpec> make_add();                                // (a, b) -> y
std::unique_ptr<ThunkSpec> make_add_rms_norm(float eps);              // (a, b, w) -> a + b, norm
std::unique_ptr<ThunkSpec> make_copy();                               // (x) -> y
std::unique_ptr<ThunkSpec> make_silu_gate();                          // (g, u) -> h
std::unique_ptr<ThunkSpec> make_softmax_ce(bool want_prob);           // (logit, tok) -> loss, amax[, prob]

}  // namespace cacti
