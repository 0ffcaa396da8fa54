// C-callable doorway into the reference's own CPU oracle, compiled from its sources where they lie
// (test/query.cpp, test/end-to-end.cpp and the headers they include). TEST INFRASTRUCTURE ONLY:
// used to validate the C restatement in cascade_oracle.c and as the "reference" CPU baseline.
// Nothing of the reference is copied here; this file only calls it.
#include "query_tests.hpp"    // gpu_saca::test::build_sa40      (test/query.cpp:42-55)
#include "tests.hpp"          // gpu_saca::test::is_correct_SA   (test/end-to-end.cpp:46-80)
#include "CPU_Reference.hpp"  // gpu_saca::ref::cmp_suffixes     (include/CPU_Reference.hpp:107-123)
#include "Packed_Prefix.hpp"  // gpu_saca::Packed_Prefix         (include/Packed_Prefix.hpp:91-104)
#include "bit-layout.hpp"     // gpu_saca::bit_layout::fwd_tag   (include/bit-layout.hpp:99-100)
#include "utility.hpp"        // gpu_saca::util::pack_word       (include/utility.hpp:147-162)
#include "message.hpp"        // gpu_saca::poison_pill, extract_rank, is_poison_pill (include/message.hpp:40-52)
#include "Partition_ID_Map.hpp" // gpu_saca::Partition_ID_Map::pack, bits_for (include/Partition_ID_Map.hpp:79,158-177)

#include <cstring>
#include <vector>

extern "C" {

// sa40_out: 5 * n + 128 bytes.
void ref_build_sa40_u16(const uint16_t* T, uint64_t n, uint8_t* sa40_out)
{
    const std::vector<uint16_t> text(T, T + n);
    const auto SA = gpu_saca::test::build_sa40(text);
    std::memcpy(sa40_out, SA.data(), SA.size());
}

int ref_is_correct_sa_u16(const uint64_t* sa, const uint16_t* T, uint64_t n)
{
    return gpu_saca::test::is_correct_SA<uint16_t>(sa, T, n) ? 1 : 0;
}

int ref_cmp_suffixes_u16(const uint16_t* T, uint64_t n, uint64_t i, uint64_t j, uint64_t max_cmp)
{
    return gpu_saca::ref::cmp_suffixes(T, n, i, j, max_cmp);
}

uint64_t ref_pack_word_u16(const uint16_t* T)
{
    return gpu_saca::util::pack_word<uint16_t>(T);
}

uint64_t ref_fwd_tag_single_partition(uint64_t tgt, uint64_t n, uint64_t ell)
{
    return gpu_saca::bit_layout::fwd_tag([](const uint64_t) { return 0; }, tgt, n, ell);
}

// Width of the reference's pivots in 64-bit words, as this library was compiled (include/Packed_Prefix.hpp:26-34).
int ref_pivot_words(void)
{
    return (int)gpu_saca::K_WORDS;
}

// key(T) <= pivot with the reference's own packing and comparison (include/Packed_Prefix.hpp:91-104,122-135).
// T must be readable for 4 * ref_pivot_words() symbols.
int ref_pivot_key_le_u16(const uint16_t* T, const uint64_t* pivot_words)
{
    gpu_saca::Pivot_Key piv;
    for(gpu_saca::idx_t w = 0; w < gpu_saca::K_WORDS; ++w)
        piv.word[w] = pivot_words[w];
    return gpu_saca::Pivot_Key::pack_prefix(T) <= piv ? 1 : 0;
}

uint32_t ref_partition_id_bits(uint32_t p)
{
    return gpu_saca::Partition_ID_Map::bits_for(static_cast<gpu_saca::p_id_t>(p));
}

// One group (or a trailing partial group) of the packed map (include/Partition_ID_Map.hpp:158-177).
void ref_partition_id_pack(const uint16_t* src, uint64_t sz, uint32_t bits, uint64_t* dst)
{
    gpu_saca::Partition_ID_Map::pack(src, sz, bits, dst);
}

// The routing-tag pair of suffix j, put together with the reference's own helpers (include/bit-layout.hpp:99-100,137,152)
// the way GPU_SACA::stage_slab does (src/GPU_SACA.cu:1688-1690); ids and retirement flags come as plain arrays.
uint32_t ref_beta_u16(uint64_t j, uint64_t n, uint64_t ell, uint64_t ctx, int generation0, const uint16_t* pid, const uint8_t* retired)
{
    namespace bl = gpu_saca::bit_layout;
    const uint64_t stride = ctx / 2;
    const auto id = [pid](const uint64_t x) { return pid[x]; };
    return bl::beta_pair(j < ctx ? 0 : bl::route(pid[j - ctx], retired[j - ctx] != 0),
                         generation0 ? bl::fwd_tag(id, j + ell, n, ell)
                                     : (j < stride ? 0 : bl::route(pid[j - stride], retired[j - stride] != 0)));
}

// The messages of one cohort member, put together with the reference's own bit helpers in the order of the emission
// kernel (include/GPU_SACA.cuh:334-352): out = {dest, target, rank} of the payload, then of the forwarded pill;
// dest = 0xFFFFFFFF where there is none.
void ref_messages_of(uint64_t sa_word, uint64_t key, uint32_t beta, uint64_t i, uint64_t active_sz, uint64_t ctx, int packed,
                     uint64_t* out)
{
    namespace bl = gpu_saca::bit_layout;
    out[0] = out[3] = 0xFFFFFFFFu;
    out[1] = out[2] = out[4] = out[5] = 0;
    const auto j = bl::suffix_of(sa_word);
    if(j >= ctx && !bl::beta_cur_retired(beta))
    {
        const gpu_saca::msg_rank_t primary = packed ? bl::primary_of(key) : key;
        out[0] = bl::beta_cur_gen(beta);
        out[1] = j - ctx;
        out[2] = i < active_sz ? primary : gpu_saca::poison_pill(primary);
    }
    if(packed && bl::received_poison_pill(key) && j >= (ctx >> 1) && !bl::beta_prev_retired(beta))
    {
        out[3] = bl::beta_prev_gen(beta);
        out[4] = j - (ctx >> 1);
        out[5] = gpu_saca::poison_pill(static_cast<gpu_saca::msg_rank_t>(bl::secondary_of(key)));
    }
}

// The key a delivered message leaves at its recipient (include/GPU_SACA.cuh:386-388).
uint64_t ref_joined_key(uint32_t primary, uint32_t msg_rank)
{
    namespace bl = gpu_saca::bit_layout;
    const auto key = bl::key(primary, gpu_saca::extract_rank(msg_rank));
    return gpu_saca::is_poison_pill(msg_rank) ? bl::mark_poison_pill_receipt(key) : key;
}

}
