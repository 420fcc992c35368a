// Hyper-parameters of one encoder stack.  Drop-in for the reference's Model_t (Model.h:2-10):
// the same seven int members in the same order, because callers build it with aggregate
// initialisation — Model_t{kdim, vdim, seq_len, nhead, dimFF, emdim, nlayer} (example/main.cu:30,
// test/Table2/main.cu:32, with nlayer left to its zero default).  A batch of sequences is not part of it: it is an argument of the
// Attention / Encoder constructors.
#pragma once
struct Model_t {
    int kdim, vdim;  // total width over all heads of Q and K, and of V
    int seq_len;     // token rows of ONE sequence
    int nhead;       // attention heads; head size = kdim / nhead
    int dimFF;       // feed-forward width
    int emdim;       // hidden width H of the residual stream
    int nlayer;      // encoder layers of the stack
};
static_assert(sizeof(Model_t) == 7 * sizeof(int), "Model_t is seven ints, as in the reference");
