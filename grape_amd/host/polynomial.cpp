#include "polynomial.hpp"
#include <algorithm>
#include <ostream>

Polynomial::Polynomial() : c_(1, Fr::zero()) {}
Polynomial::Polynomial(int degree) : c_((size_t)degree + 1, Fr::zero()) {}
Polynomial::Polynomial(int degree, Fr* coefficients) : c_(coefficients, coefficients + degree + 1) {}
Polynomial::Polynomial(const Fr& constant) : c_(1, constant) {}
Polynomial::Polynomial(const std::vector<Fr>& coefficients) : c_(coefficients) {
    if (c_.empty()) c_.push_back(Fr::zero());
}
void Polynomial::setCoefficients(int degree, Fr* coefficients) { c_.assign(coefficients, coefficients + degree + 1); }

// src/polynomial.cu:40-45
Polynomial Polynomial::eq(const Fr& u) {
    Polynomial e(1);
    e.c_[0] = Fr::one() - u;
    e.c_[1] = u + u - Fr::one();
    return e;
}
// src/polynomial.cu:47-53
Fr Polynomial::eq(const Fr& u, const Fr& v) {
    Fr r = u * v;
    r += r;
    r -= (u + v);
    r += Fr::one();
    return r;
}

Polynomial Polynomial::operator+(const Polynomial& o) const {
    Polynomial r((int)std::max(c_.size(), o.c_.size()) - 1);
    for (size_t i = 0; i < r.c_.size(); i++) {
        if (i < c_.size()) r.c_[i] += c_[i];
        if (i < o.c_.size()) r.c_[i] += o.c_[i];
    }
    return r;
}
Polynomial Polynomial::operator-(const Polynomial& o) const {
    Polynomial r((int)std::max(c_.size(), o.c_.size()) - 1);
    for (size_t i = 0; i < r.c_.size(); i++) {
        if (i < c_.size()) r.c_[i] += c_[i];
        if (i < o.c_.size()) r.c_[i] -= o.c_[i];
    }
    return r;
}
Polynomial Polynomial::operator*(const Polynomial& o) const {
    Polynomial r(getDegree() + o.getDegree());
    for (size_t i = 0; i < c_.size(); i++)
        for (size_t j = 0; j < o.c_.size(); j++) r.c_[i + j] += c_[i] * o.c_[j];
    return r;
}
Polynomial Polynomial::operator*(const Fr& val) const {
    Polynomial r(*this);
    for (auto& x : r.c_) x *= val;
    return r;
}
Polynomial Polynomial::operator-() const {
    Polynomial r(*this);
    for (auto& x : r.c_) x = -x;
    return r;
}
Polynomial& Polynomial::operator+=(const Polynomial& o) { *this = *this + o; return *this; }
Polynomial& Polynomial::operator-=(const Polynomial& o) { *this = *this - o; return *this; }
Polynomial& Polynomial::operator*=(const Polynomial& o) { *this = *this * o; return *this; }

// src/polynomial.cu:127-134: p(0) is the constant term, p(1) the sum of coefficients
Fr Polynomial::operator()(const int& x) const {
    Fr r = c_[0];
    if (x == 1)
        for (size_t i = 1; i < c_.size(); i++) r += c_[i];
    return r;
}
// src/polynomial.cu:136-145
Fr Polynomial::operator()(const Fr& x) const {
    Fr r = c_.back();
    for (int i = (int)c_.size() - 2; i >= 0; i--) {
        r *= x;
        r += c_[i];
    }
    return r;
}
std::ostream& operator<<(std::ostream& os, const Polynomial& p) {
    for (size_t i = 0; i < p.c_.size(); i++) os << (i ? " + " : "") << p.c_[i] << "*t^" << i;
    return os;
}
