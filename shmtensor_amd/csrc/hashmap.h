// Host-side handle of the static hashmap (opaque to C callers).
#pragma once
#include <stdint.h>

#include "hashmap_dev.h"

struct shmt_hashmap {
  shmt::MapView view;     // passed by value to kernels
  int kind;               // shmt::MapKind
  int fmt;                // bucket table: shmt::kSlot16 or shmt::kSlot8
  int key_bytes;
  int val_bytes;
  int64_t n;              // number of (key, value) pairs given to the build
  int64_t table_bytes;
};
