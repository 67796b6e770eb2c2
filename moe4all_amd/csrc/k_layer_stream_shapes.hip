// The streaming single-launch kernel of Op::MoeFfn instantiated for the benchmark shapes with hidden size, intermediate
// size and token rows as compile-time constants: the lane placement, the item counts and every index division of the
// kernel then fold, which is worth a tenth of the launch (measured on one box, same bits: hidden 2048 / 768, one row
// 19.4 -> 17.5 us per layer; hidden 4096 / 1536 with the always-on expert 39.9 -> 35.0 us).  A separate translation
// unit so that the two sets of instantiations compile side by side.
#include "layer_stream.h"

namespace infr {

bool launch_stream_fixed(hipStream_t s, const MoeLayerParams& q, const StreamShape& sh, bool launch, bool* taken) {
    const MoeGemvParams& p = q.g;
    *taken = true;
    const int norm = q.norm_w ? 1 : 0;
#define INFR_STREAM_AT_N(FGt, FDt, DGv, DDv, EPTv, NSPv, NEv, NFFv, ROWSv, NORMv)                                             \
    if (sh.dg == DGv && sh.dd == DDv && sh.ept == EPTv && sh.nsp == NSPv && p.ne == NEv && p.nff == NFFv && p.rows == ROWSv && \
        norm == NORMv)                                                                                                       \
        return launch ? launch_stream<FGt, FDt, DGv, DDv, EPTv, NSPv, NEv, NFFv, ROWSv, NORMv>(s, q, sh.lds) : true;
#define INFR_STREAM_AT(FGt, FDt, DGv, DDv, EPTv, NSPv, NEv, NFFv, ROWSv) \
    INFR_STREAM_AT_N(FGt, FDt, DGv, DDv, EPTv, NSPv, NEv, NFFv, ROWSv, 0)
    if (p.gate_dt == INFR_Q4K && p.down_dt == INFR_Q6K) {
        INFR_STREAM_AT(Q4KFmt, Q6KFmt, 2, 2, 1, 2, 2048, 768, 1)    // 128 experts, one token row
        INFR_STREAM_AT_N(Q4KFmt, Q6KFmt, 2, 2, 1, 2, 2048, 768, 1, 1)   // ... with the token row's RmsNorm folded in
        INFR_STREAM_AT(Q4KFmt, Q6KFmt, 2, 4, 1, 2, 2048, 768, 2)
        INFR_STREAM_AT(Q4KFmt, Q6KFmt, 2, 4, 1, 2, 2048, 768, 4)
        INFR_STREAM_AT(Q4KFmt, Q6KFmt, 2, 4, 2, 2, 2048, 768, 8)
        INFR_STREAM_AT(Q4KFmt, Q6KFmt, 2, 4, 1, 4, 4096, 1536, 1)   // 256 experts, with or without the always-on expert
        INFR_STREAM_AT_N(Q4KFmt, Q6KFmt, 2, 4, 1, 4, 4096, 1536, 1, 1)
        INFR_STREAM_AT(Q4KFmt, Q6KFmt, 2, 4, 2, 4, 4096, 1536, 2)
        INFR_STREAM_AT(Q4KFmt, Q6KFmt, 2, 4, 4, 4, 4096, 1536, 4)
    } else if (p.gate_dt == INFR_Q8_0 && p.down_dt == INFR_Q8_0) {
        INFR_STREAM_AT(Q80Fmt, Q80Fmt, 4, 5, 1, 2, 2048, 768, 1)
        INFR_STREAM_AT_N(Q80Fmt, Q80Fmt, 4, 5, 1, 2, 2048, 768, 1, 1)
        INFR_STREAM_AT(Q80Fmt, Q80Fmt, 2, 4, 1, 2, 2048, 768, 2)
        INFR_STREAM_AT(Q80Fmt, Q80Fmt, 2, 4, 1, 2, 2048, 768, 4)
    }
#undef INFR_STREAM_AT
#undef INFR_STREAM_AT_N
    *taken = false;
    return false;
}

}  // namespace infr
