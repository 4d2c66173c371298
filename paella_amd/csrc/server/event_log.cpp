#include <llis/server/event_log.h>

namespace llis {
namespace server {

std::string EventLog::to_text() const {
    std::string out;
    char line[160];
    for (const Event& ev : events_) {
        int n = 0;
        switch (ev.kind) {
            case 'J': n = std::snprintf(line, sizeof(line), "J %lld %lld %lld %lld\n", (long long)ev.a, (long long)ev.b, (long long)ev.c, (long long)ev.d); break;
            case 'B':
                if (ev.d >= 0) n = std::snprintf(line, sizeof(line), "B %lld %lld %lld %lld\n", (long long)ev.a, (long long)ev.b, (long long)ev.c, (long long)ev.d);
                else n = std::snprintf(line, sizeof(line), "B %lld %lld %lld\n", (long long)ev.a, (long long)ev.b, (long long)ev.c);
                break;
            case 'R': n = std::snprintf(line, sizeof(line), "R %lld %lld %lld\n", (long long)ev.a, (long long)ev.b, (long long)ev.c); break;
            case 'L': n = std::snprintf(line, sizeof(line), "L %lld %lld %a\n", (long long)ev.a, (long long)ev.b, ev.x); break;
            case 'D': n = std::snprintf(line, sizeof(line), "D %lld %lld %lld %lld %lld %lld\n", (long long)ev.a, (long long)ev.b, (long long)ev.c, (long long)ev.d, (long long)ev.e, (long long)ev.x); break;
            default:  n = std::snprintf(line, sizeof(line), "%c %lld\n", ev.kind, (long long)ev.a); break;
        }
        out.append(line, (size_t)n);
    }
    return out;
}

bool EventLog::save(const std::string& path) const {
    FILE* fp = std::fopen(path.c_str(), "w");
    if (!fp) return false;
    const std::string text = to_text();
    std::fwrite(text.data(), 1, text.size(), fp);
    std::fclose(fp);
    return true;
}

}  // namespace server
}  // namespace llis
