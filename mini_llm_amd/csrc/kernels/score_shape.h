// How an attention kernel shapes a score before the softmax, shared by the kernels and their callers:
//   s = scale (q . k);  softcap > 0: s <- softcap tanh(s / softcap);  r1: s <- s - r1[h] ln(1 + r2[h] (i - j));
// and which keys a query sees besides the sliding window the kernels take on their own: with chunk > 0 only those
// of the block of `chunk` positions (counted from 0) that holds the query.
// `slope` (per head, used where r1 is null) is a distance bias that grows linearly: s <- s - slope[h] (i - j).
// `sink` (per head) puts one more term into the softmax's denominator, exp(sink[h]) in natural units: a key that has
// no value, is not scaled and gets no bias. With `keep_first` > 0 a sliding window also sees the sequence's first
// keep_first positions, at their true distances.
// With `sigmoid` the weight of a visible key is sigmoid(s + score_bias[h]) on its own, not a softmax over the keys,
// and with `gate_per_head` the result's gate has one number per head and row, not one per output column.
#pragma once

struct MllmScoreShape {
    float softcap;           // <= 0: none
    int chunk;               // <= 0: none
    const float* r1;         // per head, or null: no distance bias
    const float* r2;
    int sigmoid;             // 0: softmax weights
    const float* score_bias; // per head, or null (sigmoid weights only)
    int gate_per_head;
    const float* slope;      // per head, or null: no linear distance bias
    const float* sink;       // per head, or null: nothing added to the denominator (softmax weights only)
    int keep_first;          // with a window: the first positions that stay visible; <= 0: none
};
