// C entry points onto the reference's own translation units.  TEST
// INFRASTRUCTURE ONLY (see ucm_oracle.c): this file contains no arithmetic of
// its own, it only forwards to the classes declared in the reference headers
//   ucm/sparse/gsa/offload_ops/include/{vec_product,k_repre,select_topk_block}.h
// so that ctypes can call them.  It is compiled together with the reference's
//   ucm/sparse/gsa/offload_ops/src/{vec_product,k_repre,select_topk_block}.cpp
// where they lie; the result goes to oracle/_ref/ and never into history.
#include <cstdint>
#include <vector>

#include "k_repre.h"
#include "select_topk_block.h"
#include "vec_product.h"

extern "C" {

const char* ref_simd_name() { return VecProduct::CompileTimeSimd::SIMD_NAME; }

float ref_vector_dot(const float* q, const float* k, uint32_t dim)
{
    VecProduct::VecProduct vp;
    return vp.VectorDot(q, k, dim);
}

void ref_vector_mean(const float* vectors, float* mean, uint32_t dim, uint32_t numK)
{
    VecProduct::VecProduct vp;
    vp.VectorMean(vectors, mean, dim, numK);
}

void ref_k_repre_block(const float* kArray, uint32_t kHead, uint32_t blockSize, uint32_t headSize,
                       float* out)
{
    KRepre::KRepreComputer c;
    c.ComputeKRepreBlock(kArray, kHead, blockSize, headSize, out);
}

void ref_q_head_mean(float* q, uint32_t kHead, uint32_t qHead, uint32_t headSize)
{
    SelectTopkBlock::TopkBlockSelector s;
    s.ComputeQHeadMean(q, kHead, qHead, headSize);
}

void ref_kq_scores(const float* qMean, const float* kRepre, uint32_t numBlock, uint32_t kHead,
                   uint32_t numKrepre, uint32_t headSize, float* out)
{
    SelectTopkBlock::TopkBlockSelector s;
    const std::vector<float> v = s.ComputeKQDotScores(qMean, kRepre, numBlock, kHead, numKrepre, headSize);
    for (uint32_t i = 0; i < numBlock; ++i) { out[i] = v[i]; }
}

void ref_select_topk(float* q, const float* kRepre, uint32_t numBlock, uint32_t kHead,
                     uint32_t qHead, uint32_t numKrepre, uint32_t headSize, uint32_t topk,
                     uint32_t startW, uint32_t endW, int32_t* out)
{
    SelectTopkBlock::TopkBlockSelector s;
    s.SetWindowSize(startW, endW);
    s.SelectTopK(q, kRepre, numBlock, kHead, qHead, numKrepre, headSize, topk, out);
}

// One batch through SelectTopKBS over a ragged representative table (request r
// owns rows seg_off[r] .. +seg_len[r]); the timed CPU baseline calls this.
void ref_select_topk_bs(float* q, const float* repre, const int32_t* seg_off, const int32_t* seg_len,
                        const int32_t* topk_len, uint32_t numBatch, uint32_t kHead, uint32_t qHead,
                        uint32_t numKrepre, uint32_t headSize, int32_t* out, uint32_t out_stride)
{
    static SelectTopkBlock::TopkBlockSelector s;
    const size_t row = static_cast<size_t>(kHead) * numKrepre * headSize;
    std::vector<float*> qv;
    std::vector<const float*> kv;
    std::vector<int32_t*> ov;
    std::vector<uint32_t> nb, tk;
    for (uint32_t r = 0; r < numBatch; ++r) {
        qv.push_back(q + static_cast<size_t>(r) * qHead * headSize);
        kv.push_back(repre + static_cast<size_t>(seg_off[r]) * row);
        ov.push_back(out + static_cast<size_t>(r) * out_stride);
        nb.push_back(static_cast<uint32_t>(seg_len[r]));
        tk.push_back(static_cast<uint32_t>(topk_len[r]));
    }
    s.SelectTopKBS(qv, kv, ov, numBatch, nb, kHead, qHead, numKrepre, headSize, tk);
}

}  // extern "C"
