// Word lists (bad words, stop words) matched against the time-major token history.
//
// Layout (examples/pytorch/gpt/utils/word_list.py:36-67): a list is [2, L] ints; row 0 holds the token ids of
// all n-grams back to back (0-padded), row 1 the inclusive end offset of each n-gram (-1-padded): n-gram w
// spans ids [end[w-1] (or 0), end[w]). The history of a row is a column of output_ids [max_seq, batch]; with beams
// ([max_seq, batch, beam_width]) it is followed backwards through parent_ids, one beam index per time.
#pragma once
#include "ftk_device.cuh"

namespace ftk {

struct WordList {
    const int* ids;   // row 0
    const int* ends;  // row 1
    // n-gram `w`: first id and length; false for an unused slot
    __device__ __forceinline__ bool ngram(int w, const int** first, int* count) const
    {
        const int end = ends[w];
        if (end < 0) {
            return false;
        }
        const int begin = w > 0 ? ends[w - 1] : 0;
        *first          = ids + begin;
        *count          = end - begin;
        return true;
    }
};

__device__ __forceinline__ WordList word_list(const int* base, int len)
{
    return WordList{base, base + len};
}

// Do the `count` tokens written at times last-count+1 .. last of history column `column` (element (t, row) at
// column[t * stride]) equal tokens[0 .. count)? Compared from the most recent token backwards, as both
// reference kernels do; an n-gram longer than the history does not match.
__device__ __forceinline__ bool history_ends_with(const int* __restrict__ tokens, int count,
                                                  const int* __restrict__ column, size_t stride, int last)
{
    if (count > last + 1) {
        return false;
    }
    for (int t = count - 1; t >= 0; --t) {
        if (column[(size_t)(last - (count - 1) + t) * stride] != tokens[t]) {
            return false;
        }
    }
    return true;
}

// The same with beams (ban_bad_words.cu:55-74, stop_criteria_kernels.cu:52-72): `entry` points at the batch entry's
// first beam in row 0 of output_ids / parent_ids ([max_seq, stride] each), the walk starts in beam `beam`; after a
// token matches, that time's parent becomes the beam of the time before, and a parent outside [0, beams) ends the
// match.
__device__ __forceinline__ bool beam_history_ends_with(const int* __restrict__ tokens, int count,
                                                       const int* __restrict__ ids, const int* __restrict__ parents,
                                                       size_t stride, int beam, int beams, int last)
{
    if (count > last + 1) {
        return false;
    }
    for (int t = count - 1; t >= 0; --t) {
        const size_t at = (size_t)(last - (count - 1) + t) * stride;
        if (ids[at + beam] != tokens[t]) {
            return false;
        }
        beam = parents[at + beam];
        if (beam < 0 || beam >= beams) {
            return false;
        }
    }
    return true;
}

// src/fastertransformer/kernels/ban_bad_words.cu:35-85: the last token of an n-gram is banned when the
// n-gram has one token, or when the history before `step` ends with its first n-1 tokens. Returns that token
// or -1.
__device__ __forceinline__ int banned_token(const WordList& words, int w, const int* __restrict__ column,
                                            size_t stride, int step)
{
    const int* first;
    int        count;
    if (!words.ngram(w, &first, &count) || count < 1) {
        return -1;
    }
    return history_ends_with(first, count - 1, column, stride, step - 1) ? first[count - 1] : -1;
}

// src/fastertransformer/kernels/stop_criteria_kernels.cu:34-80: the history up to and including the token
// written at `step` ends with the n-gram.
__device__ __forceinline__ bool stop_word_matches(const WordList& words, int w, const int* __restrict__ column,
                                                  size_t stride, int step)
{
    const int* first;
    int        count;
    return words.ngram(w, &first, &count) && history_ends_with(first, count, column, stride, step);
}

}  // namespace ftk
