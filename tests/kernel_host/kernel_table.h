// name -> host function of every kernel in this build of the model (the test writes the table)
#pragma once
struct HmEntry {
  const char *name;
  void (*fn)(void **pointers, const void *params);
};
const HmEntry *hm_kernel_table();
