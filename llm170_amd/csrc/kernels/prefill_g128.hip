// The dense group-128 builds of the prefill kernel (128-, 96- and 64-row block tiles, f16 and bf16 scales, plain and
// gated) as a code object of their own: the build compiles this file with the max-ILP instruction scheduler
// (llm170_amd/build.py), which the rest of prefill.hip does not take well.
#define PF_DENSE_G128
#include "prefill.hip"
