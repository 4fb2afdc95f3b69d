// thrust/future.h: device_future and device_event live in thrust/event.h.
#pragma once
#include <thrust/event.h>
