// Hyper-parameters of one encoder stack: the reference's Model_t (Model.h:2-10),
// field for field.  seq_len is the number of token rows of ONE sequence; a batch
// of sequences is an argument of the Attention / Encoder constructors.
#pragma once
struct Model_t {
    int kdim;     // total width of Q and K (all heads)
    int vdim;     // total width of V (all heads)
    int seq_len;  // token rows per sequence
    int nhead;
    int dimFF;    // feed-forward width
    int emdim;    // hidden width H
    int nlayer;
};
