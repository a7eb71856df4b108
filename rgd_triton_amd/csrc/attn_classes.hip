// Host side of the tile classification of a head-shared attention bias (attn_classes.h).
#include "attn_classes.h"

template <typename TB>
static hipError_t classify_launch(const void* bias, int64_t sb, int64_t sn, int nb, int Tq, int Tk, uint64_t* words, hipStream_t s) {
    BiasClasses c = cls_layout(words, nb, Tq, Tk, sn == 0);
    const int nrow32 = c.nrow32, nstrips = cls_nwords(Tk) * 4;
    const unsigned gx = (unsigned)(((int64_t)nrow32 * nstrips + 3) / 4);
    void (*kern)(const TB*, int64_t, int64_t, int, int, int, int, uint16_t*) = attn_bias_classify_kernel<TB>;
    const TB* bp = static_cast<const TB*>(bias);
    uint16_t* out = reinterpret_cast<uint16_t*>(words);
    void* args[] = {&bp, &sb, &sn, &Tq, &Tk, const_cast<int*>(&nrow32), const_cast<int*>(&nstrips), &out};
    hipError_t e = hipLaunchKernel(reinterpret_cast<const void*>(kern), dim3(gx, (unsigned)nb), dim3(256), args, 0, s);
    if (e != hipSuccess) return e;
    // the summaries behind the map, from the map and the bias
    uint32_t* info = const_cast<uint32_t*>(c.info);
    void (*sum)(const TB*, int64_t, int64_t, int, int, BiasClasses, uint32_t*) = attn_bias_summary_kernel<TB>;
    void* sargs[] = {&bp, &sb, &sn, &Tq, &Tk, &c, &info};
    return hipLaunchKernel(reinterpret_cast<const void*>(sum), dim3((unsigned)cls_nkb(Tk) + 1, (unsigned)nb), dim3(256), sargs, 0, s);
}

// bias: (nb, Tq, Tk) by batch and row strides (elements), 16-byte aligned rows; words: cls_bytes(nb, Tq, Tk) bytes
int attn_classify(const void* bias, int64_t sb, int64_t sn, int bias_dtype, int nb, int64_t Tq, int64_t Tk, uint64_t* words,
                  hipStream_t s) {
    hipError_t e;
    if (bias_dtype == RGD_F32) e = classify_launch<float>(bias, sb, sn, nb, (int)Tq, (int)Tk, words, s);
    else if (bias_dtype == RGD_F16) e = classify_launch<f16_t>(bias, sb, sn, nb, (int)Tq, (int)Tk, words, s);
    else e = classify_launch<bf16_t>(bias, sb, sn, nb, (int)Tq, (int)Tk, words, s);
    return rgd_launch_status("rgd_attn_bias_classify", e);
}
