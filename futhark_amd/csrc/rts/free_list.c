/* Pool of released memory blocks.
 *
 * Reuse policy (the observable behaviour of rts/c/free_list.h:100-166): a
 * pooled block can serve a request if it is large enough and either is
 * smaller than 4096 bytes, carries the same tag as the request, or wastes
 * less than half of its size; among the candidates the smallest one wins. */
#include "rts.h"

#include <assert.h>
#include <stdlib.h>

enum { FREE_LIST_INITIAL = 32 };

void free_list_init(struct free_list *l) {
  l->capacity = FREE_LIST_INITIAL;
  l->used = 0;
  l->entries = (struct free_list_entry *)calloc((size_t)l->capacity, sizeof(*l->entries));
  pthread_mutex_init(&l->lock, NULL);
}

void free_list_destroy(struct free_list *l) {
  assert(l->used == 0);
  free(l->entries);
  l->entries = NULL;
  pthread_mutex_destroy(&l->lock);
}

void free_list_pack(struct free_list *l) {
  pthread_mutex_lock(&l->lock);
  int kept = 0;
  for (int i = 0; i < l->capacity; i++) {
    if (l->entries[i].valid) l->entries[kept++] = l->entries[i];
  }
  int cap = kept < FREE_LIST_INITIAL ? FREE_LIST_INITIAL : kept;
  l->entries = (struct free_list_entry *)realloc(l->entries, (size_t)cap * sizeof(*l->entries));
  for (int i = kept; i < cap; i++) l->entries[i].valid = false;
  l->capacity = cap;
  pthread_mutex_unlock(&l->lock);
}

void free_list_insert(struct free_list *l, size_t size, uintptr_t mem, const char *tag) {
  pthread_mutex_lock(&l->lock);
  int slot = -1;
  for (int i = 0; i < l->capacity; i++) {
    if (!l->entries[i].valid) {
      slot = i;
      break;
    }
  }
  if (slot < 0) {
    int old = l->capacity;
    l->capacity = old * 2;
    l->entries =
        (struct free_list_entry *)realloc(l->entries, (size_t)l->capacity * sizeof(*l->entries));
    for (int i = old; i < l->capacity; i++) l->entries[i].valid = false;
    slot = old;
  }
  l->entries[slot].valid = true;
  l->entries[slot].size = size;
  l->entries[slot].mem = mem;
  l->entries[slot].tag = tag;
  l->used++;
  pthread_mutex_unlock(&l->lock);
}

static bool acceptable(const struct free_list_entry *e, size_t size, const char *tag) {
  if (!e->valid || e->size < size) return false;
  if (e->size < 4096) return true;  /* churn in tiny blocks is not worth avoiding */
  if (e->tag == tag) return true;   /* same use site: any slack is fine */
  return e->size < size * 2;        /* otherwise waste at most half */
}

int free_list_find(struct free_list *l, size_t size, const char *tag, size_t *size_out,
                   uintptr_t *mem_out) {
  pthread_mutex_lock(&l->lock);
  int best = -1;
  for (int i = 0; i < l->capacity; i++) {
    if (acceptable(&l->entries[i], size, tag) &&
        (best < 0 || l->entries[i].size < l->entries[best].size))
      best = i;
  }
  int ret = 1;
  if (best >= 0) {
    l->entries[best].valid = false;
    *size_out = l->entries[best].size;
    *mem_out = l->entries[best].mem;
    l->used--;
    ret = 0;
  }
  pthread_mutex_unlock(&l->lock);
  return ret;
}

int free_list_first(struct free_list *l, size_t *size_out, uintptr_t *mem_out) {
  pthread_mutex_lock(&l->lock);
  int ret = 1;
  for (int i = 0; i < l->capacity; i++) {
    if (l->entries[i].valid) {
      l->entries[i].valid = false;
      if (size_out) *size_out = l->entries[i].size;
      *mem_out = l->entries[i].mem;
      l->used--;
      ret = 0;
      break;
    }
  }
  pthread_mutex_unlock(&l->lock);
  return ret;
}
