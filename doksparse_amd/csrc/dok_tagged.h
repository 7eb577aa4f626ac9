#pragma once
#include "dok_device.h"
static int tg_launch_get(const DevTable&, const void*, i64, void*, const void*, u8*, bool, hipStream_t) { return DOK_EUNSUPPORTED; }
static int tg_launch_set(const DevTable&, const void*, const void*, i64, u8*, hipStream_t) { return DOK_EUNSUPPORTED; }
static int tg_launch_remove(const DevTable&, const void*, i64, u8*, hipStream_t) { return DOK_EUNSUPPORTED; }
static int tg_launch_count(const DevTable&, const void*, i64, i64*, hipStream_t) { return DOK_EUNSUPPORTED; }
static int tg_launch_compact(const DevTable&, i64*, i64, void*, void*, i64, i64*, hipStream_t) { return DOK_EUNSUPPORTED; }
