// Forward of the int8 transformer projection stack (LayerNorm -> per-token int8 ->
// QKV Linear -> stand-in attention -> output Linear + residual -> LayerNorm ->
// per-token int8 -> fc1 -> GELU -> per-token int8 -> fc2 + residual), composed
// from the library's own entry points.  Eight kernels per layer; the fp32
// intermediates that only feed a quantizer are never written to memory.  The fc2
// skip connection is not added in the GEMM's epilogue but by the next layer's first
// LayerNorm kernel, which reads the row anyway (after the last layer: by an add): the
// GEMM then runs in its large-tile form, whose registers have no room for
// residual values, and the stream is read and written once less.
#include "hipq_internal.h"

namespace {
size_t align256(size_t v) { return (v + 255) & ~size_t(255); }
}  // namespace

extern "C" {

size_t hipq_transformer_stack_workspace_bytes(size_t tokens, size_t d_model, size_t d_ff) {
    const size_t widest = d_model > d_ff ? d_model : d_ff;
    return align256(tokens * widest)                          // int8 activations
           + align256(tokens * sizeof(float))                 // per-token scales
           + align256(tokens * 3 * d_model * sizeof(float))   // qkv
           + align256(tokens * d_ff * sizeof(float));         // fc1 output
}

int32_t hipq_transformer_stack_forward_f32(hipq_ctx *ctx, const hipq_block_weights *blocks, size_t n_layers,
                                           size_t tokens, size_t d_model, size_t d_ff, float eps, int32_t mode,
                                           float *x, void *workspace, size_t workspace_bytes) {
    HIPQ_ENTER(ctx);
    if (n_layers == 0 || tokens == 0) return HIPQ_SUCCESS;
    HIPQ_REQUIRE_PTR(blocks);
    HIPQ_REQUIRE_PTR(x);
    HIPQ_REQUIRE_PTR(workspace);
    if (d_model == 0 || d_ff == 0) return hipq::fail(HIPQ_SHAPE_ERROR, "%s: empty model dimension", __func__);
    if (workspace_bytes < hipq_transformer_stack_workspace_bytes(tokens, d_model, d_ff))
        return hipq::fail(HIPQ_INVALID_ARGUMENT, "%s: workspace of %zu bytes is smaller than the %zu needed", __func__,
                          workspace_bytes, hipq_transformer_stack_workspace_bytes(tokens, d_model, d_ff));
    if (reinterpret_cast<uintptr_t>(workspace) & 255u)
        return hipq::fail(HIPQ_INVALID_ARGUMENT, "%s: workspace must be 256-byte aligned", __func__);
    const size_t widest = d_model > d_ff ? d_model : d_ff;
    char *p = static_cast<char *>(workspace);
    int8_t *q8 = reinterpret_cast<int8_t *>(p);
    p += align256(tokens * widest);
    float *scales = reinterpret_cast<float *>(p);
    p += align256(tokens * sizeof(float));
    float *qkv = reinterpret_cast<float *>(p);
    p += align256(tokens * 3 * d_model * sizeof(float));
    float *hidden = reinterpret_cast<float *>(p);
    const int32_t round_bits = mode & HIPQ_ROUND_HALF_EVEN;

    for (size_t l = 0; l < n_layers; ++l) {
        const hipq_block_weights &b = blocks[l];
        int32_t rc;
        // attention half: x += W_out * quant(V(LN1(x)))
        // (from the second layer on: x += the previous layer's fc2 output, held in the qkv buffer)
        if (l == 0)
            rc = hipq_layer_norm_quantize_f32_i8(ctx, x, tokens, d_model, b.ln1_gamma, b.ln1_beta, eps, round_bits, q8, scales);
        else
            rc = hipq_add_layer_norm_quantize_f32_i8(ctx, x, qkv, tokens, d_model, b.ln1_gamma, b.ln1_beta, eps,
                                                     round_bits, q8, scales);
        if (rc) return rc;
        rc = hipq_linear_i8_f32(ctx, q8, scales, 1, b.w_qkv, b.s_qkv, b.b_qkv, tokens, 3 * d_model, d_model, qkv);
        if (rc) return rc;
        // Stand-in for the attention mixing, which is outside this path: the value slice passes through.
        rc = hipq_quantize_per_row_strided_f32_i8(ctx, qkv + 2 * d_model, tokens, d_model, 3 * d_model,
                                                  HIPQ_PARAMS_SYMMETRIC, round_bits, q8, scales, nullptr, nullptr);
        if (rc) return rc;
        rc = hipq_linear_i8_f32_residual(ctx, q8, scales, 1, b.w_out, b.s_out, b.b_out, x, tokens, d_model, d_model, x);
        if (rc) return rc;
        // MLP half: x += W_fc2 * quant(GELU(W_fc1 * quant(LN2(x))))
        rc = hipq_layer_norm_quantize_f32_i8(ctx, x, tokens, d_model, b.ln2_gamma, b.ln2_beta, eps, round_bits, q8, scales);
        if (rc) return rc;
        rc = hipq_linear_i8_f32(ctx, q8, scales, 1, b.w_fc1, b.s_fc1, b.b_fc1, tokens, d_ff, d_model, hidden);
        if (rc) return rc;
        rc = hipq_gelu_tanh_quantize_f32_i8(ctx, hidden, tokens, d_ff, round_bits, q8, scales);
        if (rc) return rc;
        rc = hipq_linear_i8_f32(ctx, q8, scales, 1, b.w_fc2, b.s_fc2, b.b_fc2, tokens, d_model, d_ff, qkv);
        if (rc) return rc;
        if (l + 1 == n_layers) {
            // no next LayerNorm to carry the skip connection: a plain add (still cheaper than the
            // small-tile GEMM that has room for residual values)
            rc = hipq_add_f32(ctx, x, qkv, tokens * d_model, x);
            if (rc) return rc;
        }
    }
    return HIPQ_SUCCESS;
}

// ---- the same forward on prepared (fragment-packed) weights: five kernels per layer ---------------------------
// Every Linear that feeds a row operation runs as a row-panel GEMM with that operation in its epilogue
// (hipq_gemm_rows.h): out-proj + skip + LayerNorm 2 + quantize, fc1 + GELU + quantize, fc2 + skip + the next
// layer's LayerNorm 1 + quantize.  Activations travel between them as packed int8; the only fp32 tensors that
// touch memory are the stream x and the qkv output (which the attention outside this path would read).

size_t hipq_transformer_stack_prepared_workspace_bytes(size_t tokens, size_t d_model, size_t d_ff) {
    const size_t widest = d_model > d_ff ? d_model : d_ff;
    size_t a = 0, b = 0;
    if (hipq_packed_size(tokens, d_model, &a) || hipq_packed_size(tokens, widest, &b)) return 0;
    return align256(a) + align256(b)                          // packed int8 activations (two in flight)
           + 2 * align256(tokens * sizeof(float))             // their per-token scales
           + align256(tokens * 3 * d_model * sizeof(float));  // qkv
}

int32_t hipq_transformer_stack_forward_prepared_f32(hipq_ctx *ctx, const hipq_block_weights *blocks, size_t n_layers,
                                                    size_t tokens, size_t d_model, size_t d_ff, float eps,
                                                    int32_t mode, float *x, void *workspace, size_t workspace_bytes) {
    HIPQ_ENTER(ctx);
    if (n_layers == 0 || tokens == 0) return HIPQ_SUCCESS;
    HIPQ_REQUIRE_PTR(blocks);
    HIPQ_REQUIRE_PTR(x);
    HIPQ_REQUIRE_PTR(workspace);
    if (d_model == 0 || d_ff == 0) return hipq::fail(HIPQ_SHAPE_ERROR, "%s: empty model dimension", __func__);
    if (d_model % 128 || d_ff % 128 || d_model > 3072 || d_ff > 3072)
        return hipq::fail(HIPQ_SHAPE_ERROR,
                          "%s: d_model = %zu and d_ff = %zu must be multiples of 128 and at most 3072 (a workgroup "
                          "holds whole rows of each Linear's output); use hipq_transformer_stack_forward_f32",
                          __func__, d_model, d_ff);
    const size_t need = hipq_transformer_stack_prepared_workspace_bytes(tokens, d_model, d_ff);
    if (need == 0) return hipq::fail(HIPQ_SHAPE_ERROR, "%s: dimension too large", __func__);
    if (workspace_bytes < need)
        return hipq::fail(HIPQ_INVALID_ARGUMENT, "%s: workspace of %zu bytes is smaller than the %zu needed", __func__,
                          workspace_bytes, need);
    if (reinterpret_cast<uintptr_t>(workspace) & 255u)
        return hipq::fail(HIPQ_INVALID_ARGUMENT, "%s: workspace must be 256-byte aligned", __func__);
    const size_t widest = d_model > d_ff ? d_model : d_ff;
    size_t bytes_a = 0, bytes_b = 0;
    hipq_packed_size(tokens, d_model, &bytes_a);
    hipq_packed_size(tokens, widest, &bytes_b);
    char *p = static_cast<char *>(workspace);
    int8_t *qa = reinterpret_cast<int8_t *>(p);  // LayerNorm outputs (the operand of qkv and fc1)
    p += align256(bytes_a);
    int8_t *qb = reinterpret_cast<int8_t *>(p);  // the value slice, the GELU output (the operand of out-proj and fc2)
    p += align256(bytes_b);
    float *sa = reinterpret_cast<float *>(p);
    p += align256(tokens * sizeof(float));
    float *sb = reinterpret_cast<float *>(p);
    p += align256(tokens * sizeof(float));
    float *qkv = reinterpret_cast<float *>(p);
    const int32_t round_bits = mode & HIPQ_ROUND_HALF_EVEN;

    // quant(LN1(x)) of the first layer: the row kernel, then the packing pass (row-major codes parked in qb)
    int32_t rc = hipq_layer_norm_quantize_f32_i8(ctx, x, tokens, d_model, blocks[0].ln1_gamma, blocks[0].ln1_beta, eps,
                                                 round_bits, qb, sa);
    if (rc) return rc;
    if ((rc = hipq_pack_rows_i8(ctx, qb, tokens, d_model, qa))) return rc;
    for (size_t l = 0; l < n_layers; ++l) {
        const hipq_block_weights &b = blocks[l];
        // attention half: x += W_out * quant(V(LN1(x))), then quant(LN2(x))
        // (the same bits from either kernel; between the row-panel kernels of the other projections the row-panel
        // form is ~2 us per layer faster than the tiled one at 8192 tokens, d_model 768 - 1.83 against 1.855 ms for
        // twelve layers - although alone it is level with it: 28.9 against 28.4 us)
        if (3 * d_model <= 3072)
            rc = hipq_linear_rows_packed_i8_f32(ctx, qa, sa, 1, b.w_qkv, b.s_qkv, b.b_qkv, tokens, 3 * d_model, d_model,
                                                qkv);
        else
            rc = hipq_linear_packed_i8_f32(ctx, qa, sa, 1, b.w_qkv, b.s_qkv, b.b_qkv, tokens, 3 * d_model, d_model, qkv);
        if (rc) return rc;
        // Stand-in for the attention mixing, which is outside this path: the value slice passes through.  Its
        // per-token quantizer runs inside the out-projection where a workgroup can hold its rows' codes on chip.
        if (d_model <= 1536 && ctx->gemm_variant != 6) {
            rc = hipq_linear_from_f32_residual_layer_norm_quantize_packed_i8(
                ctx, qkv + 2 * d_model, 3 * d_model, b.w_out, b.s_out, b.b_out, tokens, d_model, d_model, x, b.ln2_gamma,
                b.ln2_beta, eps, round_bits, qa, sa);
        } else {
            rc = hipq::quantize_activations_per_row_strided(ctx, qkv + 2 * d_model, tokens, d_model, 3 * d_model,
                                                            round_bits, qb, sb, /*packed=*/true);
            if (rc) return rc;
            rc = hipq_linear_residual_layer_norm_quantize_packed_i8(ctx, qb, sb, 1, b.w_out, b.s_out, b.b_out, tokens,
                                                                    d_model, d_model, x, b.ln2_gamma, b.ln2_beta, eps,
                                                                    round_bits, qa, sa);
        }
        if (rc) return rc;
        // MLP half: x += W_fc2 * quant(GELU(W_fc1 * quant(LN2(x)))), then the next layer's quant(LN1(x))
        rc = hipq_linear_gelu_quantize_packed_i8(ctx, qa, sa, 1, b.w_fc1, b.s_fc1, b.b_fc1, tokens, d_ff, d_model,
                                                 round_bits, qb, sb);
        if (rc) return rc;
        const bool last = l + 1 == n_layers;
        rc = hipq_linear_residual_layer_norm_quantize_packed_i8(
            ctx, qb, sb, 1, b.w_fc2, b.s_fc2, b.b_fc2, tokens, d_model, d_ff, x, last ? nullptr : blocks[l + 1].ln1_gamma,
            last ? nullptr : blocks[l + 1].ln1_beta, eps, round_bits, last ? nullptr : qa, last ? nullptr : sa);
        if (rc) return rc;
    }
    return HIPQ_SUCCESS;
}

}  // extern "C"
