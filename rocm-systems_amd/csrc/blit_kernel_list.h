// The kernel variants that exist, as X-macros: one list drives the kernel
// definitions, the HIP launch table and the name table of the code object.
#ifndef MI355_BLIT_KERNEL_LIST_H_
#define MI355_BLIT_KERNEL_LIST_H_

// X(unroll, nt_load, store_policy, realign)
#define MI355_COPY_R_(X, U, L, S) X(U, L, S, 0) X(U, L, S, 1)
#define MI355_COPY_S_(X, U, L) \
  MI355_COPY_R_(X, U, L, 0) MI355_COPY_R_(X, U, L, 1) MI355_COPY_R_(X, U, L, 2) MI355_COPY_R_(X, U, L, 3)
#define MI355_COPY_L_(X, U) MI355_COPY_S_(X, U, 0) MI355_COPY_S_(X, U, 1)
#define MI355_FOR_EACH_COPY_KERNEL(X) MI355_COPY_L_(X, 1) MI355_COPY_L_(X, 2) MI355_COPY_L_(X, 4)

// X(unroll, store_policy)
#define MI355_FILL_S_(X, U) X(U, 0) X(U, 1) X(U, 2) X(U, 3)
#define MI355_FOR_EACH_FILL_KERNEL(X) MI355_FILL_S_(X, 1) MI355_FILL_S_(X, 2) MI355_FILL_S_(X, 4)

// X(waves per chunk, nt_load, store_policy)
#define MI355_BATCH_S_(X, P, L) X(P, L, 0) X(P, L, 1) X(P, L, 2) X(P, L, 3)
#define MI355_BATCH_L_(X, P) MI355_BATCH_S_(X, P, 0) MI355_BATCH_S_(X, P, 1)
#define MI355_FOR_EACH_BATCH_RECORDS_KERNEL(X) MI355_BATCH_L_(X, 1) MI355_BATCH_L_(X, 2) MI355_BATCH_L_(X, 4)

// X(nt_load, store_policy): the batched copy over records for device-resident
// descriptors (four waves per chunk)
#define MI355_FOR_EACH_BATCH_LOOKUP_KERNEL(X) MI355_RECT_NARROW_S_(X, 0) MI355_RECT_NARROW_S_(X, 1)

// X(unroll, nt_load, store_policy): the pitched-region copy
#define MI355_FOR_EACH_RECT_KERNEL(X) MI355_BATCH_L_(X, 1) MI355_BATCH_L_(X, 2) MI355_BATCH_L_(X, 4)

// X(nt_load, store_policy): the region copy of narrow rows
#define MI355_RECT_NARROW_S_(X, L) X(L, 0) X(L, 1) X(L, 2) X(L, 3)
#define MI355_FOR_EACH_RECT_NARROW_KERNEL(X) MI355_RECT_NARROW_S_(X, 0) MI355_RECT_NARROW_S_(X, 1)

#endif  // MI355_BLIT_KERNEL_LIST_H_
