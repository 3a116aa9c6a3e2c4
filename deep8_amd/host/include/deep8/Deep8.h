// Umbrella header of the MI355X host layer.
#ifndef DEEP8_HOST_DEEP8_H
#define DEEP8_HOST_DEEP8_H
#include "deep8/Exception.h"
#include "deep8/Model.h"
#include "deep8/Math.h"
#include "deep8/Nodes.h"
#include "deep8/Executor.h"
#include "deep8/Trainer.h"
#endif
