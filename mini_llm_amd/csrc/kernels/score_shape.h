// How an attention kernel shapes a score before the softmax, shared by the kernels and their callers:
//   s = scale (q . k);  softcap > 0: s <- softcap tanh(s / softcap);  r1: s <- s - r1[h] ln(1 + r2[h] (i - j));
// and which keys a query sees besides the sliding window the kernels take on their own: with chunk > 0 only those
// of the block of `chunk` positions (counted from 0) that holds the query.
#pragma once

struct MllmScoreShape {
    float softcap;           // <= 0: none
    int chunk;               // <= 0: none
    const float* r1;         // per head, or null: no distance bias
    const float* r2;
};
