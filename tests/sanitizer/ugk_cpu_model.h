// TEST INFRASTRUCTURE ONLY: hooks of the CPU model of the kernel layer (ugk_cpu_model.cc) that have no counterpart in
// include/ugache_hip.h.  The driver uses them to play a caller that records its stream into a graph; the model keeps the
// runtime's bookkeeping of such a capture and lists every call that breaks one of its rules.
#pragma once

#include <cstddef>

extern "C" {
// work enqueued on `stream` from here on is "recorded into a graph" (it still runs at once in the model)
int ugk_model_capture_begin(void *stream);
// ends the capture begun on `stream`; *graph_id names the graph that now references what took part in it
int ugk_model_capture_end(void *stream, int *graph_id);
void ugk_model_graph_destroy(int graph_id);
// number of rule violations seen so far; their texts, one a line, into text[capacity]
size_t ugk_model_violations(char *text, size_t capacity);
void ugk_model_reset(void);
}
