/* hostmem.c - the two host-side allocators of Boat's memory header (include/boat/memory.h:58-77): a pool of equal
 * blocks and a bump arena.  Neither touches the GPU; they are here because programs written against Boat's headers
 * use them next to the training path (tests/unit/test_phase1.c:13-113).  Behaviour follows src/core/memory.c:283-520:
 * a pool never grows, hands out a block for any size up to its block size and refuses beyond that; an arena rounds
 * sizes up to 8 bytes and doubles its capacity until a request fits (earlier pointers are then no longer valid, as
 * there). */
#include "boat_internal.h"

#include <stdint.h>
#include <stdlib.h>

#define POOL_BLOCK_HEADER 24   /* what the reference accounts per block besides the payload (next, in_use, size) */

struct boat_memory_pool_t {
    size_t block_size, total_blocks, free_count;
    unsigned char* payload;    /* total_blocks x stride bytes */
    size_t stride;             /* block size rounded up to 16 bytes */
    size_t* free_stack;        /* indices of free blocks; the top is handed out next */
    unsigned char* in_use;     /* one flag per block */
};

boat_memory_pool_t* boat_memory_pool_create(size_t block_size, size_t initial_blocks) {
    if (block_size == 0 || initial_blocks == 0) return NULL;
    boat_memory_pool_t* pool = (boat_memory_pool_t*)calloc(1, sizeof(*pool));
    if (!pool) return NULL;
    pool->block_size = block_size;
    pool->total_blocks = pool->free_count = initial_blocks;
    pool->stride = (block_size + 15) & ~(size_t)15;
    pool->payload = (unsigned char*)malloc(pool->stride * initial_blocks);
    pool->free_stack = (size_t*)malloc(sizeof(size_t) * initial_blocks);
    pool->in_use = (unsigned char*)calloc(initial_blocks, 1);
    if (!pool->payload || !pool->free_stack || !pool->in_use) {
        boat_memory_pool_free(pool);
        return NULL;
    }
    for (size_t i = 0; i < initial_blocks; i++) pool->free_stack[i] = initial_blocks - 1 - i;
    return pool;
}

void boat_memory_pool_free(boat_memory_pool_t* pool) {
    if (!pool) return;
    free(pool->payload);
    free(pool->free_stack);
    free(pool->in_use);
    free(pool);
}

void* boat_memory_pool_alloc(boat_memory_pool_t* pool, size_t size) {
    if (!pool || size > pool->block_size || pool->free_count == 0) return NULL;
    const size_t index = pool->free_stack[--pool->free_count];
    pool->in_use[index] = 1;
    return pool->payload + index * pool->stride;
}

void boat_memory_pool_free_block(boat_memory_pool_t* pool, void* block) {
    if (!pool || !block) return;
    const unsigned char* p = (const unsigned char*)block;
    if (p < pool->payload || p >= pool->payload + pool->stride * pool->total_blocks) return;   /* not one of ours */
    const size_t offset = (size_t)(p - pool->payload);
    if (offset % pool->stride != 0) return;
    const size_t index = offset / pool->stride;
    if (!pool->in_use[index]) return;   /* already free */
    pool->in_use[index] = 0;
    pool->free_stack[pool->free_count++] = index;
}

void boat_memory_pool_clear(boat_memory_pool_t* pool) {
    if (!pool) return;
    for (size_t i = 0; i < pool->total_blocks; i++) {
        pool->in_use[i] = 0;
        pool->free_stack[i] = pool->total_blocks - 1 - i;
    }
    pool->free_count = pool->total_blocks;
}

size_t boat_memory_pool_allocated_blocks(const boat_memory_pool_t* pool) { return pool ? pool->total_blocks - pool->free_count : 0; }
size_t boat_memory_pool_free_blocks(const boat_memory_pool_t* pool) { return pool ? pool->free_count : 0; }
size_t boat_memory_pool_total_memory(const boat_memory_pool_t* pool) {
    return pool ? pool->total_blocks * (POOL_BLOCK_HEADER + pool->block_size) : 0;
}

struct boat_memory_arena_t {
    unsigned char* memory;
    size_t capacity, used;
};

boat_memory_arena_t* boat_memory_arena_create(size_t initial_size) {
    if (initial_size == 0) initial_size = (size_t)1 << 20;
    boat_memory_arena_t* arena = (boat_memory_arena_t*)calloc(1, sizeof(*arena));
    if (!arena) return NULL;
    arena->memory = (unsigned char*)malloc(initial_size);
    if (!arena->memory) {
        free(arena);
        return NULL;
    }
    arena->capacity = initial_size;
    return arena;
}

void boat_memory_arena_free(boat_memory_arena_t* arena) {
    if (!arena) return;
    free(arena->memory);
    free(arena);
}

void* boat_memory_arena_alloc(boat_memory_arena_t* arena, size_t size) {
    if (!arena || size == 0 || size > SIZE_MAX / 4) return NULL;
    size = (size + 7) & ~(size_t)7;
    if (arena->used + size > arena->capacity) {
        size_t capacity = arena->capacity * 2;
        while (arena->used + size > capacity) capacity *= 2;
        unsigned char* grown = (unsigned char*)realloc(arena->memory, capacity);
        if (!grown) return NULL;
        arena->memory = grown;
        arena->capacity = capacity;
    }
    void* p = arena->memory + arena->used;
    arena->used += size;
    return p;
}

void boat_memory_arena_reset(boat_memory_arena_t* arena) {
    if (arena) arena->used = 0;
}
size_t boat_memory_arena_used(const boat_memory_arena_t* arena) { return arena ? arena->used : 0; }
size_t boat_memory_arena_capacity(const boat_memory_arena_t* arena) { return arena ? arena->capacity : 0; }
