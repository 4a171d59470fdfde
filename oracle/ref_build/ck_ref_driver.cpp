// C-ABI wrapper around host-only code that ships inside the reference tree (its vendored
// ck_tile headers).  Built by oracle/ref_build/Makefile into oracle/_ref/libck_ref.so, used
// by the tests to pin the oracle's sorter and e2m1/e8m0 arithmetic.  Test infrastructure only.
//
// The reference headers are compiled where they lie (-I /root/reference/archive/ck_tile);
// nothing from them is copied here.
#include <cstring>
#include <vector>
#include <cstdint>
#define CK_TILE_REFERENCE_MOE_SORTING_MOCK_ID 1
#include "ck_tile/host/reference/reference_moe_sorting.hpp"   // archive/ck_tile/ck_tile/host/reference/reference_moe_sorting.hpp:13-117
#include "ck_tile/core/numeric/pk_fp4.hpp"                    // archive/ck_tile/ck_tile/core/numeric/pk_fp4.hpp
#include "ck_tile/core/numeric/e8m0.hpp"                      // archive/ck_tile/ck_tile/core/numeric/e8m0.hpp

extern "C" {

// returns the padded total (unit_cnt * unit_size); outputs must hold max_padded entries.
int ck_ref_moe_sorting(const int* topk_ids, const float* weights, int tokens, int topk, int experts,
                       int unit_size, const int* expert_mask /* may be null */, int* sorted_ids,
                       float* sorted_weights, int* sorted_expert_ids, int max_padded)
{
    using namespace ck_tile;
    HostTensor<index_t> ids({tokens, topk});
    HostTensor<float> ws({tokens, topk});
    for(int i = 0; i < tokens * topk; i++)
    {
        ids.mData[i] = topk_ids[i];
        ws.mData[i]  = weights[i];
    }
    HostTensor<index_t> mask({experts});
    for(int i = 0; i < experts; i++)
        mask.mData[i] = expert_mask ? expert_mask[i] : 1;
    HostTensor<index_t> so({max_padded});
    HostTensor<float> sw({max_padded});
    HostTensor<index_t> se({max_padded / unit_size + 1});
    index_t cnt = 0;
    reference_moe_sorting<float, index_t>(ids, ws, mask, so, sw, se, cnt, experts, unit_size, tokens,
                                          expert_mask != nullptr, true);
    for(int i = 0; i < cnt; i++)
    {
        sorted_ids[i]     = so.mData[i];
        sorted_weights[i] = sw.mData[i];
    }
    for(int i = 0; i < cnt / unit_size; i++)
        sorted_expert_ids[i] = se.mData[i];
    return cnt;
}

// float -> 4-bit e2m1 code (value / scale, RNE, saturating): mxfp_convert.hpp:61-216
void ck_ref_float_to_e2m1(const float* x, float scale, uint8_t* codes, int n)
{
    for(int i = 0; i < n; i++)
        codes[i] = ck_tile::convert_to_type<ck_tile::pk_fp4_t>(x[i], scale) & 0xF;
}

// 4-bit e2m1 code -> float: mxfp_convert.hpp:50-59
void ck_ref_e2m1_to_float(const uint8_t* codes, float scale, float* out, int n)
{
    for(int i = 0; i < n; i++)
        out[i] = ck_tile::convert_to_float<ck_tile::pk_fp4_t>(codes[i] & 0xF, scale);
}

// e8m0 byte -> float: e8m0.hpp:85-100
void ck_ref_e8m0_to_float(const uint8_t* b, float* out, int n)
{
    for(int i = 0; i < n; i++)
        out[i] = static_cast<float>(ck_tile::e8m0_t{b[i]});
}

// packing order of two codes in a byte: pk_fp4.hpp:122-125
uint8_t ck_ref_pack(uint8_t even_elem, uint8_t odd_elem)
{
    return ck_tile::pk_fp4_t::_pack(even_elem, odd_elem);
}
}
