// n-gram matching against the time-major token history, shared by the stand-alone bad-word /
// stop-word kernels and the fused decode kernels.
//
// Word-list layout (examples/pytorch/gpt/utils/word_list.py:36-67): `words` points at [2, L] ints;
// row 0 holds all n-grams' token ids back to back (0-padded), row 1 the inclusive end offset of
// each n-gram (-1-padded). Word i spans ids [off[i-1] (or 0), off[i]).
#pragma once
#include "ftk_device.cuh"

namespace ftk {

// src/fastertransformer/kernels/ban_bad_words.cu:35-85. Returns the token id to ban, or -1.
// `row_index` = id_offset + batch_idx * beam_width (column of the history matrix for beam 0).
__device__ __forceinline__ int banned_token(const int* __restrict__ words, int words_len, int word,
                                            const int* __restrict__ output_ids, const int* __restrict__ parent_ids,
                                            int batch_size, int beam_width, int row_index, int beam_idx, int step)
{
    const int* offsets = words + words_len;
    if (offsets[word] < 0) {
        return -1;
    }
    const int item_end   = offsets[word];
    const int item_start = word > 0 ? offsets[word - 1] : 0;
    const int item_size  = item_end - item_start;
    bool      ban        = item_size == 1;
    if (item_size > 1 && step >= item_size - 1) {
        ban            = true;
        int parent_id  = beam_idx;
        for (int t = item_size - 2; t >= 0; --t) {
            const size_t pos = (size_t)(step - (item_size - 1) + t) * batch_size * beam_width + row_index + parent_id;
            if (output_ids[pos] != words[item_start + t]) {
                ban = false;
                break;
            }
            if (beam_width > 1) {
                parent_id = parent_ids[pos];
                if (parent_id < 0 || parent_id >= beam_width) {
                    ban = false;
                    break;
                }
            }
        }
    }
    return ban ? words[item_end - 1] : -1;
}

// src/fastertransformer/kernels/stop_criteria_kernels.cu:34-80: the token written at `step` is the
// last token of the n-gram and is compared first.
__device__ __forceinline__ bool stop_word_matches(const int* __restrict__ words, int words_len, int word,
                                                  const int* __restrict__ output_ids,
                                                  const int* __restrict__ parent_ids, int batch_size, int beam_width,
                                                  int row_index, int beam_idx, int step)
{
    const int* offsets = words + words_len;
    if (offsets[word] < 0) {
        return false;
    }
    const int item_end   = offsets[word];
    const int item_start = word > 0 ? offsets[word - 1] : 0;
    const int item_size  = item_end - item_start;
    if (step + 1 < item_size) {
        return false;
    }
    int parent_id = beam_idx;
    for (int t = item_size - 1; t >= 0; --t) {
        const size_t pos = (size_t)(step - (item_size - 1) + t) * batch_size * beam_width + row_index + parent_id;
        if (output_ids[pos] != words[item_start + t]) {
            return false;
        }
        if (beam_width > 1) {
            parent_id = parent_ids[pos];
            if (parent_id < 0 || parent_id >= beam_width) {
                return false;
            }
        }
    }
    return true;
}

}  // namespace ftk
