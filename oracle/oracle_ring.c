/*
 * CPU oracle (test infrastructure): bounded MPSC ring (Vyukov scheme limited
 * to one consumer) and SPSC ring, with run-time capacity and payload size.
 * Follows include/nccl_ofi_mpsc_ring.h:56-163 and include/nccl_ofi_spsc_ring.h:30-61.
 */
#include <stdatomic.h>
#include <stdlib.h>
#include <string.h>

#include "oracle.h"

struct oracle_mpsc {
	uint32_t capacity;
	uint32_t payload_bytes;
	size_t cell_bytes;
	unsigned char *cells; /* cell = {atomic u32 sequence; payload} */
	_Alignas(64) _Atomic uint32_t enqueue_pos;
	_Alignas(64) uint32_t dequeue_pos;
};

static _Atomic uint32_t *cell_seq(oracle_mpsc_t *r, uint32_t idx)
{
	return (_Atomic uint32_t *)(r->cells + (size_t)idx * r->cell_bytes);
}

static unsigned char *cell_data(oracle_mpsc_t *r, uint32_t idx)
{
	return r->cells + (size_t)idx * r->cell_bytes + 8;
}

oracle_mpsc_t *oracle_mpsc_create(uint32_t capacity, uint32_t payload_bytes)
{
	if (capacity == 0 || (capacity & (capacity - 1)) != 0) {
		return NULL; /* power of two, :57-58 */
	}
	oracle_mpsc_t *r = (oracle_mpsc_t *)aligned_alloc(64, sizeof(*r));
	if (!r) {
		return NULL;
	}
	memset(r, 0, sizeof(*r));
	r->capacity = capacity;
	r->payload_bytes = payload_bytes;
	r->cell_bytes = 8 + (((size_t)payload_bytes + 7) & ~(size_t)7);
	r->cells = (unsigned char *)calloc(capacity, r->cell_bytes);
	if (!r->cells) {
		free(r);
		return NULL;
	}
	/* ctor, :64-69: sequence of slot i starts at i */
	for (uint32_t i = 0; i < capacity; i++) {
		atomic_store_explicit(cell_seq(r, i), i, memory_order_relaxed);
	}
	atomic_store(&r->enqueue_pos, 0);
	r->dequeue_pos = 0;
	return r;
}

void oracle_mpsc_destroy(oracle_mpsc_t *r)
{
	if (r) {
		free(r->cells);
		free(r);
	}
}

void oracle_mpsc_set_positions(oracle_mpsc_t *r, uint32_t pos)
{
	/* An empty ring whose cursors both sit at `pos`: slot (pos+k) & mask is
	 * free for lap position pos+k. */
	for (uint32_t k = 0; k < r->capacity; k++) {
		uint32_t p = pos + k;
		atomic_store_explicit(cell_seq(r, p & (r->capacity - 1)), p, memory_order_relaxed);
	}
	atomic_store(&r->enqueue_pos, pos);
	r->dequeue_pos = pos;
}

/* push, :79-118 */
int oracle_mpsc_push(oracle_mpsc_t *r, const void *entry)
{
	uint32_t pos = atomic_load_explicit(&r->enqueue_pos, memory_order_relaxed);
	uint32_t idx;

	for (;;) {
		idx = pos & (r->capacity - 1);
		uint32_t seq = atomic_load_explicit(cell_seq(r, idx), memory_order_acquire);
		int32_t diff = (int32_t)seq - (int32_t)pos;
		if (diff == 0) {
			if (atomic_compare_exchange_weak_explicit(&r->enqueue_pos, &pos, pos + 1,
								  memory_order_relaxed,
								  memory_order_relaxed)) {
				break;
			}
		} else if (diff < 0) {
			return 0; /* full */
		} else {
			pos = atomic_load_explicit(&r->enqueue_pos, memory_order_relaxed);
		}
	}
	memcpy(cell_data(r, idx), entry, r->payload_bytes);
	atomic_store_explicit(cell_seq(r, idx), pos + 1, memory_order_release);
	return 1;
}

/* pop, :124-144 */
int oracle_mpsc_pop(oracle_mpsc_t *r, void *entry)
{
	uint32_t pos = r->dequeue_pos;
	uint32_t idx = pos & (r->capacity - 1);
	uint32_t seq = atomic_load_explicit(cell_seq(r, idx), memory_order_acquire);
	int32_t diff = (int32_t)seq - (int32_t)(pos + 1);

	if (diff != 0) {
		return 0; /* empty */
	}
	memcpy(entry, cell_data(r, idx), r->payload_bytes);
	r->dequeue_pos = pos + 1;
	atomic_store_explicit(cell_seq(r, idx), pos + r->capacity, memory_order_release);
	return 1;
}

struct oracle_spsc {
	uint32_t capacity;
	uint32_t payload_bytes;
	unsigned char *ring;
	_Alignas(64) _Atomic uint32_t head;
	_Alignas(64) _Atomic uint32_t tail;
};

oracle_spsc_t *oracle_spsc_create(uint32_t capacity, uint32_t payload_bytes)
{
	oracle_spsc_t *r = (oracle_spsc_t *)aligned_alloc(64, sizeof(*r));
	if (!r) {
		return NULL;
	}
	memset(r, 0, sizeof(*r));
	r->capacity = capacity;
	r->payload_bytes = payload_bytes;
	r->ring = (unsigned char *)calloc(capacity, payload_bytes);
	if (!r->ring) {
		free(r);
		return NULL;
	}
	return r;
}

void oracle_spsc_destroy(oracle_spsc_t *r)
{
	if (r) {
		free(r->ring);
		free(r);
	}
}

/* push, include/nccl_ofi_spsc_ring.h:38-48: one slot stays empty */
int oracle_spsc_push(oracle_spsc_t *r, const void *entry)
{
	uint32_t h = atomic_load_explicit(&r->head, memory_order_relaxed);
	uint32_t next = (h + 1) % r->capacity;

	if (next == atomic_load_explicit(&r->tail, memory_order_acquire)) {
		return 0;
	}
	memcpy(r->ring + (size_t)h * r->payload_bytes, entry, r->payload_bytes);
	atomic_store_explicit(&r->head, next, memory_order_release);
	return 1;
}

/* pop, :50-59 */
int oracle_spsc_pop(oracle_spsc_t *r, void *entry)
{
	uint32_t t = atomic_load_explicit(&r->tail, memory_order_relaxed);

	if (t == atomic_load_explicit(&r->head, memory_order_acquire)) {
		return 0;
	}
	memcpy(entry, r->ring + (size_t)t * r->payload_bytes, r->payload_bytes);
	atomic_store_explicit(&r->tail, (t + 1) % r->capacity, memory_order_release);
	return 1;
}

/* ---- threaded self-check, the scenario of tests/unit/mpsc_ring.cpp:118-189 ----
 * `producers` threads push (id << 28 | counter); the calling thread pops and checks
 * per-producer FIFO, no loss, no duplicate.  Returns 0 when every property held. */
#include <pthread.h>

struct stress_arg {
	oracle_mpsc_t *ring;
	uint32_t id;
	uint32_t count;
};

static void *stress_producer(void *p)
{
	struct stress_arg *a = (struct stress_arg *)p;
	uint32_t i = 0;
	while (i < a->count) {
		uint32_t v = (a->id << 28) | i;
		if (oracle_mpsc_push(a->ring, &v)) {
			++i;
		}
	}
	return NULL;
}

int oracle_mpsc_stress(uint32_t capacity, uint32_t producers, uint32_t per_producer)
{
	if (producers == 0 || producers > 15 || per_producer >= (1u << 28)) {
		return -22;
	}
	oracle_mpsc_t *ring = oracle_mpsc_create(capacity, sizeof(uint32_t));
	if (!ring) {
		return -12;
	}
	pthread_t th[15];
	struct stress_arg args[15];
	uint32_t next_expected[15] = { 0 };
	int bad = 0;

	for (uint32_t p = 0; p < producers; p++) {
		args[p].ring = ring;
		args[p].id = p;
		args[p].count = per_producer;
		pthread_create(&th[p], NULL, stress_producer, &args[p]);
	}
	uint64_t total = 0, want = (uint64_t)producers * per_producer;
	while (total < want) {
		uint32_t v;
		if (oracle_mpsc_pop(ring, &v)) {
			uint32_t p = v >> 28, c = v & ((1u << 28) - 1);
			if (p >= producers || c != next_expected[p]) {
				bad = 1;
			} else {
				next_expected[p] = c + 1;
			}
			++total;
		}
	}
	for (uint32_t p = 0; p < producers; p++) {
		pthread_join(th[p], NULL);
		if (next_expected[p] != per_producer) {
			bad = 1;
		}
	}
	uint32_t v;
	if (oracle_mpsc_pop(ring, &v)) {
		bad = 1; /* must be empty */
	}
	oracle_mpsc_destroy(ring);
	return bad;
}
